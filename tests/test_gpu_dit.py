"""Full denoiser forward on the MI355X: fp32 path against golden vectors of the compiled reference and the CPU oracle,
bf16 path against the fp32 path at the SD3.5-medium shape with a 512x512 image, and size-independent properties."""
import os

import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from gpu_util import M, dev, dev_params, host, max_abs, rel_l2, F32_TOL, BF16_REL_L2
from sd3_c_amd.config import DiTConfig, sd35_medium
from sd3_c_amd.params import dit_param_shapes

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = np.load(os.path.join(HERE, "golden", "reference_outputs.npz"))


def run_gpu_dit(k, precision="fp32", params=None):
    cfg = k["cfg"]
    args = [dev(k["pooled"]), dev(k["captions"]), dev(k["latent"]), dev(k["timesteps"])]
    before = [a.clone() for a in args]
    out = M.DiT(*args, params if params is not None else dev_params(k["params"]), cfg.num_layers, set(cfg.dual_attention_layers), cfg.pooled_dim,
                cfg.captions_dim, cfg.in_channels, cfg.emb_dim, cfg.attn_heads, cfg.mlp_expand, cfg.patch_size, cfg.pos_embed_max_size, cfg.base_height,
                cfg.use_qk_norm, precision=precision)
    for a, b in zip(args, before):
        assert torch.equal(a, b)  # inputs are left untouched (modules.cpp:1633)
    return host(out)


@pytest.mark.parametrize("name", list(cases.DIT_CASES))
def test_dit_fp32_vs_reference_golden_and_oracle(name):
    k = cases.dit_case(name)
    out = run_gpu_dit(k)
    assert out.shape == k["latent"].shape
    assert max_abs(out, GOLDEN[name + ".out"]) <= F32_TOL
    assert max_abs(out, ol.orc_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])) <= F32_TOL


def test_dit_fp32_reference_test_configuration():
    """The configuration of the reference's own end-to-end check (module_tests/DiT.py: width 256, 2 heads of 128, 3 blocks,
    64x64 latent, 154 text tokens), against the output of the compiled reference on the same inputs."""
    k = cases.dit_reference_test_case()
    gold = np.load(os.path.join(HERE, "golden", "reference_dit_test_config.npz"))["out"]
    assert max_abs(run_gpu_dit(k), gold) <= F32_TOL


def test_dit_bf16_vs_reference_golden():
    """The bf16 path against the output of the compiled reference directly (the one golden forward whose sizes suit the bf16
    kernels: heads of 64, every width a multiple of 64)."""
    k = cases.dit_case("dit_hs64")
    out = run_gpu_dit(k, "bf16")
    assert rel_l2(out, GOLDEN["dit_hs64.out"]) <= BF16_REL_L2


LONG = pytest.mark.skipif(not os.environ.get("SD3_LONG_TESTS"), reason="minutes of float64 numpy on the host: set SD3_LONG_TESTS=1 (and run pytest with -s)")


@pytest.mark.parametrize("layers,dual,B,side", [(4, (0, 1), 2, 64), (24, tuple(range(13)), 2, 64), (3, (0,), 1, 128),
                                                pytest.param(24, tuple(range(13)), 1, 128, marks=LONG)])
def test_dit_at_512px_and_1024px_sizes_vs_float64_forward(layers, dual, B, side):
    """Both precisions against arithmetic that is not this library's, at the sizes of BASELINE config 3 (SD3.5-medium widths, batch 2,
    64x64 latent = 1024 image tokens, 154 text tokens of width 4096): a model of four blocks (two with the extra self-attention, the
    last one discarding its context) and the full model of 24 blocks (13 dual) against the float64 forward written from the op list,
    which tests/test_oracle.py pins to the CPU oracle and to the compiled reference's outputs; and three blocks on one sample of the
    headline shape (128x128 latent = 4096 image tokens). (The CPU oracle itself would need an hour for the second of these.) The full
    24-block model on one sample of the headline shape takes the float64 forward some minutes on the host and runs only on request
    (SD3_LONG_TESTS=1, pytest -s; two minutes on 16 host cores; measured: fp32 path 2.2e-6 rel-L2 and 9.4e-6 max-abs, bf16 path 4.3e-3)."""
    import dataclasses
    from sd3_c_amd.params import synthetic_params_numpy
    from test_oracle import dit64
    cfg = dataclasses.replace(sd35_medium(), num_layers=layers, dual_attention_layers=dual)
    P = synthetic_params_numpy(dit_param_shapes(cfg), 91, 0.02 if layers == 24 else 0.03, 0.02 if layers == 24 else 0.03)
    rng = np.random.Generator(np.random.Philox(92))
    k = dict(cfg=cfg, params=P, latent=rng.standard_normal((B, cfg.in_channels, side, side), dtype=np.float32),
             captions=rng.standard_normal((B, 154, cfg.captions_dim), dtype=np.float32), pooled=rng.standard_normal((B, cfg.pooled_dim), dtype=np.float32),
             timesteps=(rng.random(B) * 1000).astype(np.float32))
    tick = (lambda l: print(f"float64 forward: block {l} done", flush=True)) if side * layers > 2000 else None
    want = dit64(k["pooled"], k["captions"], k["latent"], k["timesteps"], P, cfg, tick)
    dP = dev_params(P)
    out32, out16 = run_gpu_dit(k, "fp32", dP), run_gpu_dit(k, "bf16", dP)
    print(f"{layers} blocks, batch {B}, {side}x{side} latent vs float64: fp32 path rel-L2 {rel_l2(out32, want):.3g} max-abs {max_abs(out32, want):.3g}, "
          f"bf16 path rel-L2 {rel_l2(out16, want):.3g}", flush=True)
    assert rel_l2(out32, want) <= 2e-5 and max_abs(out32, want) <= F32_TOL   # measured 2e-6 and 3e-5 on 24 blocks
    assert rel_l2(out16, want) <= BF16_REL_L2                                # measured 4.2e-3 on 24 blocks


@pytest.mark.parametrize("file_dtype,shards", [("float32", 1), ("bfloat16", 3)])
def test_dit_from_hugging_face_safetensors_vs_reference_golden(tmp_path, file_dtype, shards):
    """Real-weight path end to end: the parameters of the reference's own full-model test configuration written the way the Hugging
    Face checkpoint stores them (its names, nn.Linear layout, separate q/k/v; module_tests/modules.py:532-612), as one fp32 file or
    as bf16 shards with an index -> load_safetensors -> Denoiser on the GPU -> the compiled reference's output."""
    import json
    from safetensors.torch import save_file
    from sd3_c_amd import hf_weights as H
    k = cases.dit_reference_test_case()
    cfg = k["cfg"]
    hf = {n: torch.from_numpy(v).to(getattr(torch, file_dtype)) for n, v in H.to_hf_state_dict(k["params"], cfg).items()}
    names = sorted(hf)
    weight_map = {}
    for i in range(shards):
        fn = f"diffusion_pytorch_model-{i + 1:05d}-of-{shards:05d}.safetensors" if shards > 1 else "diffusion_pytorch_model.safetensors"
        part = {n: hf[n].contiguous() for n in names[i::shards]}
        save_file(part, str(tmp_path / fn))
        weight_map.update({n: fn for n in part})
    if shards > 1:
        (tmp_path / "diffusion_pytorch_model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))
    loaded = H.load_safetensors(str(tmp_path), cfg)
    assert list(loaded) == list(k["params"])
    gold = np.load(os.path.join(HERE, "golden", "reference_dit_test_config.npz"))["out"]
    den = M.Denoiser(dev_params(loaded), cfg, "fp32")
    out = host(den(dev(k["pooled"]), dev(k["captions"]), dev(k["latent"]), dev(k["timesteps"])))
    if file_dtype == "float32":
        assert max_abs(out, gold) <= F32_TOL          # lossless file: the fp32 parity bar
    else:
        assert rel_l2(out, gold) <= BF16_REL_L2       # weights rounded to bf16 in the file: the bf16 bar
    den.ctx.close()


def _synthetic_device_params(cfg, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    P = {}
    for name, shape in dit_param_shapes(cfg).items():
        if "rmsnorm" in name:
            P[name] = 1 + 0.02 * torch.randn(shape, device="cuda", generator=g)
        elif name.endswith(".bias"):
            P[name] = 0.02 * torch.randn(shape, device="cuda", generator=g)
        else:
            P[name] = 0.02 * torch.randn(shape, device="cuda", generator=g)
    return P


def _inputs(cfg, B, Tc, H, W, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    return dict(cfg=cfg, latent=rng.standard_normal((B, cfg.in_channels, H, W), dtype=np.float32),
                captions=rng.standard_normal((B, Tc, cfg.captions_dim), dtype=np.float32), pooled=rng.standard_normal((B, cfg.pooled_dim), dtype=np.float32),
                timesteps=(rng.random((B,), dtype=np.float32) * 1000).astype(np.float32))


@pytest.mark.parametrize("side", [64, 128])
def test_dit_bf16_vs_fp32_sd35_medium(side):
    """Full SD3.5-medium shape (24 blocks, width 1536, 13 dual blocks), batch 2, 154 text tokens, with a 64x64 latent (512x512
    image, 1024 image tokens) and with the benchmark's 128x128 latent (1024x1024 image, 4096 image tokens). The bf16 path must
    stay within relative L2 1e-2 of the fp32 path on the final velocity."""
    cfg = sd35_medium()
    P = _synthetic_device_params(cfg, 5)
    k = _inputs(cfg, 2, 154, side, side, 6)
    o32 = run_gpu_dit(k, "fp32", P)
    o16 = run_gpu_dit(k, "bf16", P)
    assert np.isfinite(o32).all() and np.isfinite(o16).all()
    assert rel_l2(o16, o32) <= BF16_REL_L2
    # batch elements are independent: running element 1 alone gives the same answer (checks batch indexing of every kernel)
    k1 = dict(k, latent=k["latent"][1:], captions=k["captions"][1:], pooled=k["pooled"][1:], timesteps=k["timesteps"][1:])
    assert rel_l2(run_gpu_dit(k1, "bf16", P)[0], o16[1]) <= 1e-5


@pytest.mark.parametrize("B", [1, 4, 8])
def test_dit_batch_sweep_at_the_benchmark_shape(B):
    """The 1024x1024 forward at the other batch sizes of the throughput sweep (independent inputs per element): bf16 within
    relative L2 1e-2 of fp32 on every element, and the last element computed alone equals the same element inside the batch."""
    cfg = sd35_medium()
    P = _synthetic_device_params(cfg, 5)
    k = _inputs(cfg, B, 154, 128, 128, 20 + B)
    o32 = run_gpu_dit(k, "fp32", P)
    o16 = run_gpu_dit(k, "bf16", P)
    assert np.isfinite(o16).all()
    for b in range(B):
        assert rel_l2(o16[b], o32[b]) <= BF16_REL_L2, b
    if B > 1:
        k1 = dict(k, latent=k["latent"][-1:], captions=k["captions"][-1:], pooled=k["pooled"][-1:], timesteps=k["timesteps"][-1:])
        assert rel_l2(run_gpu_dit(k1, "bf16", P)[0], o16[-1]) <= 1e-5


@pytest.mark.parametrize("B,h,w,Tc", [(1, 256, 256, 154), (1, 192, 80, 77), (3, 34, 62, 333)])
def test_dit_other_image_sizes_bf16_vs_fp32_sd35_medium(B, h, w, Tc):
    """The full model away from the benchmark's sizes: a 2048x2048 image (256x256 latent, 16384 image tokens: four times the headline
    sequence, 257 key tiles per attention item), a non-square 1536x640 one with 77 text tokens, and a batch of three with a grid and a
    text length that are multiples of no tile (17 x 31 patches, 333 text tokens)."""
    cfg = sd35_medium()
    P = _synthetic_device_params(cfg, 5)
    k = _inputs(cfg, B, Tc, h, w, 40 + B)
    o32 = run_gpu_dit(k, "fp32", P)
    o16 = run_gpu_dit(k, "bf16", P)
    assert np.isfinite(o32).all() and np.isfinite(o16).all()
    assert rel_l2(o16, o32) <= BF16_REL_L2   # measured 4.4e-3, 5.0e-3, 4.9e-3


@pytest.mark.parametrize("B", [9, 16])
def test_dit_batches_beyond_eight(B):
    """More batch elements than one launch of the modulation projections takes (eight): the forward against the CPU oracle, and every
    element equal to the same element computed alone."""
    cfg = DiTConfig(num_layers=2, dual_attention_layers=(0,), emb_dim=128, attn_heads=2, pooled_dim=64, captions_dim=64, pos_embed_max_size=16, base_height=8)
    P = _synthetic_device_params(cfg, 3)
    k = _inputs(cfg, B, 3, 8, 12, 4)
    o32 = run_gpu_dit(k, "fp32", P)
    host_P = {n: host(v) for n, v in P.items()}
    assert max_abs(o32, ol.orc_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], host_P, cfg)) <= F32_TOL
    o16 = run_gpu_dit(k, "bf16", P)
    assert rel_l2(o16, o32) <= BF16_REL_L2
    for b in (0, 7, 8, B - 1):
        k1 = dict(k, latent=k["latent"][b:b + 1], captions=k["captions"][b:b + 1], pooled=k["pooled"][b:b + 1], timesteps=k["timesteps"][b:b + 1])
        assert rel_l2(run_gpu_dit(k1, "bf16", P)[0], o16[b]) <= 1e-5, b


def test_dit_ragged_shapes_bf16_vs_fp32():
    """Token counts that are not multiples of any tile (odd grid, 1 text token), reduced depth."""
    cfg = DiTConfig(num_layers=3, dual_attention_layers=(0, 1), emb_dim=512, attn_heads=8, pooled_dim=128, captions_dim=192, pos_embed_max_size=64,
                    base_height=32)
    P = _synthetic_device_params(cfg, 7)
    k = _inputs(cfg, 3, 1, 2 * 13, 2 * 9, 8)
    o32 = run_gpu_dit(k, "fp32", P)
    assert rel_l2(run_gpu_dit(k, "bf16", P), o32) <= BF16_REL_L2
    host_P = {n: host(v) for n, v in P.items()}
    small = dict(k, params=host_P)
    assert max_abs(o32, ol.orc_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], host_P, cfg)) <= F32_TOL


def test_dit_missing_parameter_is_reported():
    from sd3_c_amd import lib as L_
    k = cases.dit_case("dit_small")
    P = dev_params(k["params"])
    del P["linear_out.weight"]
    with pytest.raises(L_.Sd3Error) as e:
        run_gpu_dit(k, "fp32", P)
    assert e.value.status == 2 and "linear_out.weight" in str(e.value)


def test_forwards_on_alternating_streams_share_the_context_safely():
    """The workspace and the derived weight copies belong to the context, not to a stream: a change of stream makes the new stream
    wait for what was queued on the old one, so back-to-back forwards on two streams with different inputs give the results of the
    same forwards run one at a time."""
    k = cases.dit_case("dit_hs64")
    cfg = k["cfg"]
    den = M.Denoiser(dev_params(k["params"]), cfg, "bf16")
    args = [dev(k["pooled"]), dev(k["captions"]), dev(k["latent"]), dev(k["timesteps"])]
    args2 = [a.clone() for a in args]
    args2[2] = args2[2] * 0.5 + 0.25
    want1, want2 = den(*args).clone(), den(*args2).clone()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for i in range(6):  # nothing synchronises the host between these calls
        with torch.cuda.stream(s1 if i % 2 == 0 else s2):
            outs.append(den(*(args if i % 2 == 0 else args2), out=torch.empty_like(args[2])))
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(o, want1 if i % 2 == 0 else want2)
    den.ctx.close()


def test_cfg_euler_step_equals_forward_then_formula():
    """The guided Euler step writes latent + dsigma * (v_u + g * (v_c - v_u)) from the same velocities the plain forward
    returns (closed form; the reference has no sampler), for an odd grid so that pixels outside the patch grid are covered."""
    cfg = DiTConfig(num_layers=2, dual_attention_layers=(0,), pooled_dim=32, captions_dim=64, in_channels=16, emb_dim=128, attn_heads=2, mlp_expand=4,
                    patch_size=2, pos_embed_max_size=16, base_height=16, use_qk_norm=True)
    P = _synthetic_device_params(cfg, 21)
    g = torch.Generator(device="cuda").manual_seed(22)
    n, Tc, H, W = 2, 5, 11, 14
    lat = torch.randn((n, cfg.in_channels, H, W), device="cuda", generator=g)
    lat_pair = torch.cat([lat, lat], 0).contiguous()
    captions = torch.randn((2 * n, Tc, cfg.captions_dim), device="cuda", generator=g)
    pooled = torch.randn((2 * n, cfg.pooled_dim), device="cuda", generator=g)
    t = torch.full((2 * n,), 700.0, device="cuda")
    for precision in ("fp32", "bf16"):
        den = M.Denoiser(P, cfg, precision)
        v = den(pooled, captions, lat_pair, t)
        got = den.cfg_euler_step(pooled, captions, lat_pair, t, guidance=4.5, dsigma=-0.03)
        torch.cuda.synchronize()
        want = lat + (-0.03) * (v[:n] + 4.5 * (v[n:] - v[:n]))
        assert got.shape == lat.shape
        assert float((got - want).abs().max()) <= 1e-5
    with pytest.raises(Exception):
        den.cfg_euler_step(pooled[:3], captions[:3], lat_pair[:3], t[:3], 4.5, -0.03)   # an odd batch has no two halves


def test_warm_forward_is_graph_capturable_and_replays_bit_identically():
    """After one warm-up call a forward makes no allocation, memset or host synchronisation, so it can be captured into a
    HIP graph. The graph is replayed several times, with eager work and synchronisations in between, and every replay must
    reproduce the eager result bit for bit (both precisions, the sampler-step variant included)."""
    cfg = DiTConfig(num_layers=3, dual_attention_layers=(0, 1), pooled_dim=64, captions_dim=64, in_channels=16, emb_dim=128, attn_heads=2, mlp_expand=4,
                    patch_size=2, pos_embed_max_size=32, base_height=16, use_qk_norm=True)
    P = _synthetic_device_params(cfg, 31)
    g = torch.Generator(device="cuda").manual_seed(32)
    B, Tc, H, W = 2, 9, 24, 20
    lat = torch.randn((B, cfg.in_channels, H, W), device="cuda", generator=g)
    captions = torch.randn((B, Tc, cfg.captions_dim), device="cuda", generator=g)
    pooled = torch.randn((B, cfg.pooled_dim), device="cuda", generator=g)
    t = torch.full((B,), 300.0, device="cuda")
    for precision in ("bf16", "fp32"):
        den = M.Denoiser(P, cfg, precision)
        out, step_out = torch.empty_like(lat), torch.empty_like(lat[:1])
        for _ in range(2):
            den(pooled, captions, lat, t, out=out)
            den.cfg_euler_step(pooled, captions, lat, t, 3.0, -0.05, out=step_out)
        torch.cuda.synchronize()
        want, want_step = out.clone(), step_out.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            den(pooled, captions, lat, t, out=out)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            den(pooled, captions, lat, t, out=out)
            den.cfg_euler_step(pooled, captions, lat, t, 3.0, -0.05, out=step_out)
        for i in range(3):
            out.zero_()
            step_out.zero_()
            (lat * 2).sum().item()        # eager work and a synchronisation between replays
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want) and torch.equal(step_out, want_step), (precision, i)


@pytest.mark.parametrize("B", [2, 6])
def test_dit_at_the_width_of_sd35_large(B):
    """The forward is generic in its sizes (modules.cpp:1605-1613): a model of the SD3.5-large widths (38 heads of 64 = width 2432,
    three blocks, the first with the extra self-attention) on a 32x32 latent with 20 text tokens: fp32 path against the float64 forward,
    bf16 path against the same. (Width 2432 takes the modulation projections in groups of four batch elements and the LayerNorm rows
    through ten 16-byte loads per lane.)"""
    from sd3_c_amd.params import synthetic_params_numpy
    from test_oracle import dit64
    cfg = DiTConfig(num_layers=3, dual_attention_layers=(0,), emb_dim=2432, attn_heads=38, pooled_dim=2048, captions_dim=4096, pos_embed_max_size=192,
                    base_height=64)
    P = synthetic_params_numpy(dit_param_shapes(cfg), 61, 0.02, 0.02)
    k = _inputs(cfg, B, 20, 32, 32, 62)
    want = dit64(k["pooled"], k["captions"], k["latent"], k["timesteps"], P, cfg)
    dP = dev_params(P)
    o32 = run_gpu_dit(k, "fp32", dP)
    assert rel_l2(o32, want) <= 2e-5 and max_abs(o32, want) <= F32_TOL
    assert rel_l2(run_gpu_dit(k, "bf16", dP), want) <= BF16_REL_L2
