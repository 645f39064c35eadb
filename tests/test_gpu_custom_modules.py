"""The stand-in for the reference's `custom_modules` extension (sd3.c_amd/custom_modules.py), used the way the reference's
own drivers use the extension: host tensors, the reference's argument lists, in-place update of the block's streams."""
import os
import sys

import numpy as np
import pytest
import torch

import cases
from gpu_util import max_abs, F32_TOL

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "sd3.c_amd"))
import custom_modules as F  # noqa: E402

GOLDEN = np.load(os.path.join(HERE, "golden", "reference_outputs.npz"))


def test_dit_called_like_module_tests_DiT_py():
    """module_tests/DiT.py:33-49 with the inputs of the committed golden vector: host tensors in, host tensor out."""
    k = cases.dit_reference_test_case()
    cfg = k["cfg"]
    params = {n: torch.from_numpy(v) for n, v in k["params"].items()}
    latent, captions = torch.from_numpy(k["latent"]), torch.from_numpy(k["captions"])
    pooled, timesteps = torch.from_numpy(k["pooled"]), torch.from_numpy(k["timesteps"])
    x_out = F.DiT(pooled, captions, latent, timesteps, params, cfg.num_layers, set(cfg.dual_attention_layers), cfg.pooled_dim, cfg.captions_dim,
                  cfg.in_channels, cfg.emb_dim, cfg.attn_heads, cfg.mlp_expand, cfg.patch_size, cfg.pos_embed_max_size, cfg.base_height, cfg.use_qk_norm)
    assert x_out.device.type == "cpu" and x_out.shape == latent.shape
    gold = np.load(os.path.join(HERE, "golden", "reference_dit_test_config.npz"))["out"]
    assert max_abs(x_out.numpy(), gold) <= F32_TOL


@pytest.mark.parametrize("name", list(cases.BLOCK_CASES)[:2])
def test_block_called_like_module_tests_dit_block_py(name):
    """module_tests/dit_block.py:40-46 and :60-66: the host call and the device call update c and x in place."""
    k = cases.block_case(name)
    (B, Tc, C), Tx = k["c"].shape, k["x"].shape[1]
    params = {n: torch.from_numpy(v) for n, v in k["params"].items()}
    y, c, x = torch.from_numpy(k["y"].copy()), torch.from_numpy(k["c"].copy()), torch.from_numpy(k["x"].copy())
    c_out, x_out = F.Dit_block(y, c, x, params, B, Tc, Tx, C, k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    assert c_out is c and x_out is x
    assert max_abs(x.numpy(), GOLDEN[name + ".x"]) <= F32_TOL
    if not k["discard_context"]:
        assert max_abs(c.numpy(), GOLDEN[name + ".c"]) <= F32_TOL
    yd, cd, xd = (torch.from_numpy(k[n].copy()).cuda() for n in ("y", "c", "x"))
    c2, x2 = F.DiT_block_cuda(yd, cd, xd, {n: v.cuda() for n, v in params.items()}, B, Tc, Tx, C, k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"],
                              k["discard_context"])
    assert x2 is xd and torch.equal(xd.cpu(), x)


def test_block_at_the_sizes_of_module_tests_dit_block_py():
    """module_tests/dit_block.py:9-66 with its own sizes (batch 16, 512 image + 154 text tokens, width 768, 12 heads, mlp_expand 2, extra
    self-attention and qk-norm on, y = silu(randn)), its two calls -- host tensors through Dit_block, device tensors through
    DiT_block_cuda -- and its checks (max difference of c_out and x_out), here against the float64 statement of the block."""
    from sd3_c_amd.params import block_param_shapes, synthetic_params_numpy
    from test_oracle import block64
    B, Tc, Tx, emb_dim, attn_heads, mlp_expand = 16, 77 + 77, 512, 768, 12, 2
    torch.manual_seed(5)
    P = synthetic_params_numpy(block_param_shapes(emb_dim, mlp_expand, True, True, False, emb_dim // attn_heads), 6, emb_dim ** -0.5 / 3 ** 0.5, 0.02)
    params = {n: torch.from_numpy(v) for n, v in P.items()}
    x, y, c = torch.randn((B, Tx, emb_dim)), torch.nn.functional.silu(torch.randn((B, emb_dim))), torch.randn((B, Tc, emb_dim))
    c_true, x_true = block64(y.numpy(), c.numpy(), x.numpy(), P, attn_heads, True, True, False)
    c_clone, x_clone, y_clone = c.clone().to("cuda"), x.clone().to("cuda"), y.clone().to("cuda")
    c_out, x_out = F.Dit_block(y, c, x, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, True, True, False)
    assert max_abs(c_out.numpy(), c_true) <= F32_TOL and max_abs(x_out.numpy(), x_true) <= F32_TOL
    params_cuda = {n: v.to("cuda") for n, v in params.items()}
    c_out_cuda, x_out_cuda = F.DiT_block_cuda(y_clone, c_clone, x_clone, params_cuda, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, True, True, False)
    assert max_abs(c_out_cuda.cpu().numpy(), c_true) <= F32_TOL and max_abs(x_out_cuda.cpu().numpy(), x_true) <= F32_TOL
    F.release()


def test_module_level_precision_switch_reaches_the_bf16_path():
    """A script written against the reference's signatures selects the bf16 path with F.PRECISION; results then differ from the
    fp32 ones in the low bits only (and the switch goes back)."""
    from gpu_util import rel_l2
    k = cases.block_case("block_dual_hs64")
    (B, Tc, C), Tx = k["c"].shape, k["x"].shape[1]
    params = {n: torch.from_numpy(v) for n, v in k["params"].items()}
    try:
        F.PRECISION = "bf16"
        y, c, x = torch.from_numpy(k["y"].copy()), torch.from_numpy(k["c"].copy()), torch.from_numpy(k["x"].copy())
        F.Dit_block(y, c, x, params, B, Tc, Tx, C, k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    finally:
        F.PRECISION = "fp32"
    gold = GOLDEN["block_dual_hs64.x"]
    assert 1e-6 < rel_l2(x.numpy(), gold) <= 1e-2


def test_host_parameter_map_is_uploaded_once_and_follows_in_place_changes():
    """The reference's signatures hand the host parameter map to every call. A second call with the same map re-uses the device copies
    (and, in bf16, the weight copies derived from them); a weight changed in place is uploaded again and the result follows it; the
    per-call `precision` keyword overrides the module-level switch."""
    from gpu_util import rel_l2
    k = cases.block_case("block_dual_hs64")
    (B, Tc, C), Tx = k["c"].shape, k["x"].shape[1]
    params = {n: torch.from_numpy(v.copy()) for n, v in k["params"].items()}
    args = (B, Tc, Tx, C, k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])

    def run(precision):
        y, c, x = torch.from_numpy(k["y"].copy()), torch.from_numpy(k["c"].copy()), torch.from_numpy(k["x"].copy())
        F.Dit_block(y, c, x, params, *args, precision=precision)
        return x

    F.release()
    x1 = run("bf16")
    copies = {n: v[2].data_ptr() for n, v in F._uploaded.items()}
    ctx = F._M.shared_context("cuda")
    built = ctx.copies_built()
    assert set(copies) == set(params) and built > 0
    x2 = run("bf16")
    assert {n: v[2].data_ptr() for n, v in F._uploaded.items()} == copies and ctx.copies_built() == built
    assert torch.equal(x1, x2) and 1e-6 < rel_l2(x1.numpy(), GOLDEN["block_dual_hs64.x"]) <= 1e-2
    assert max_abs(run("fp32").numpy(), GOLDEN["block_dual_hs64.x"]) <= F32_TOL and F.PRECISION == "fp32"
    name = "latent_mlp.lin2.weight"
    params[name].mul_(0.5)  # in place: same tensor object, new version counter
    x3 = run("bf16")
    assert ctx.copies_built() == built + 1 and not torch.equal(x3, x1)
    params[name].mul_(2.0)  # (exact: back to the original values)
    assert torch.equal(run("bf16"), x1)
    F.release()
    assert not F._uploaded


def test_operator_entry_points_take_host_tensors():
    x = torch.randn(2, 5, 64)
    out = F.layer_norm(x, None, None, 1e-6, False)[0]
    assert out.device.type == "cpu"
    assert float((out - torch.nn.functional.layer_norm(x, (64,), eps=1e-6)).abs().max()) <= F32_TOL
    # `gelu` is the erf form, as in the reference's extension (modules.cpp:1795, module_tests/gelu.py:28 at its 1e-5); the tanh form
    # (up to ~5e-4 away from it) has its own name
    assert float((F.gelu(x) - torch.nn.functional.gelu(x, approximate="none")).abs().max()) <= 1e-5
    assert float((F.gelu_tanh(x) - torch.nn.functional.gelu(x, approximate="tanh")).abs().max()) <= 1e-5
    W, b = torch.randn(64, 32) * 0.1, torch.randn(32)
    assert float((F.linear(x, W, b) - (x @ W + b)).abs().max()) <= F32_TOL
