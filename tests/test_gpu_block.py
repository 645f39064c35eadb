"""One MMDiT-X block on the MI355X against the reference arithmetic: golden vectors of the compiled reference, the CPU
oracle on the same seeded inputs, a float64 statement of the block at the reference-runnable size (B=1, 256 image + 77 text tokens, width 1536), and the bf16 path
against the fp32 path."""
import os

import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from gpu_util import M, dev, dev_params, host, max_abs, rel_l2, F32_TOL, BF16_REL_L2
from test_oracle import block64
from sd3_c_amd.params import block_param_shapes, synthetic_params_numpy

pytestmark = pytest.mark.gpu
GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_outputs.npz"))


def run_gpu_block(k, precision="fp32", entry=None):
    y, c, x = dev(k["y"]), dev(k["c"]), dev(k["x"])
    B, Tc, Cd = k["c"].shape
    Tx = k["x"].shape[1]
    fn = entry or M.Dit_block
    c_out, x_out = fn(y, c, x, dev_params(k["params"]), B, Tc, Tx, Cd, k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"],
                      precision=precision)
    assert c_out.data_ptr() == c.data_ptr() and x_out.data_ptr() == x.data_ptr()  # updated in place, like the reference (modules.cpp:1602)
    assert np.array_equal(host(y), k["y"])
    return host(c_out), host(x_out)


@pytest.mark.parametrize("name", list(cases.BLOCK_CASES))
def test_block_fp32_vs_reference_golden_and_oracle(name):
    k = cases.block_case(name)
    c, x = run_gpu_block(k)
    assert max_abs(x, GOLDEN[name + ".x"]) <= F32_TOL
    co, xo = ol.orc_dit_block(k["y"], k["c"], k["x"], k["params"], k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    assert max_abs(x, xo) <= F32_TOL
    if k["discard_context"]:
        assert np.array_equal(c, k["c"])
    else:
        assert max_abs(c, GOLDEN[name + ".c"]) <= F32_TOL and max_abs(c, co) <= F32_TOL


def test_block_cuda_entry_point_is_the_same_block():
    k = cases.block_case("block_dual_hs64")
    c, x = run_gpu_block(k, entry=M.DiT_block_cuda)
    assert max_abs(x, GOLDEN["block_dual_hs64.x"]) <= F32_TOL and max_abs(c, GOLDEN["block_dual_hs64.c"]) <= F32_TOL


def _wide_case(B, Tc, Tx, dual, discard, seed, C=1536, NH=24, me=4):
    rng = np.random.Generator(np.random.Philox(seed))
    params = synthetic_params_numpy(block_param_shapes(C, me, dual, True, discard, C // NH), seed + 1, 0.02, 0.02)
    return dict(y=rng.standard_normal((B, C), dtype=np.float32), c=rng.standard_normal((B, Tc, C), dtype=np.float32),
                x=rng.standard_normal((B, Tx, C), dtype=np.float32), params=params, NH=NH, mlp_expand=me, use_dual=dual, use_qk_norm=True,
                discard_context=discard)


@pytest.mark.parametrize("dual,discard", [(True, False), (False, True)])
def test_block_fp32_width_1536_vs_oracle(dual, discard):
    """SD3.5-medium width (1536, 24 heads of 64) with few tokens so that the CPU oracle finishes in seconds."""
    k = _wide_case(2, 5, 19, dual, discard, 11)
    c, x = run_gpu_block(k)
    co, xo = ol.orc_dit_block(k["y"], k["c"], k["x"], k["params"], 24, 4, dual, True, discard)
    assert max_abs(x, xo) <= F32_TOL
    assert max_abs(c, co) <= F32_TOL
    # the bf16 path against the CPU arithmetic directly (not through the fp32 GPU path)
    c16, x16 = run_gpu_block(k, "bf16")
    assert rel_l2(x16, xo) <= BF16_REL_L2 and rel_l2(x16 - k["x"], xo - k["x"]) <= 2 * BF16_REL_L2
    if not discard:
        assert rel_l2(c16, co) <= BF16_REL_L2


@pytest.mark.parametrize("name", [n for n in cases.BLOCK_CASES if n.endswith("hs64")])
def test_block_bf16_vs_reference_golden(name):
    """The bf16 path against the outputs of the compiled reference (head_dim 64 cases; weights N(0, 0.1), so the block's update is as
    large as the stream it is added to)."""
    k = cases.block_case(name)
    c, x = run_gpu_block(k, "bf16")
    assert rel_l2(x, GOLDEN[name + ".x"]) <= BF16_REL_L2
    if k["discard_context"]:
        assert np.array_equal(c, k["c"])
    else:
        assert rel_l2(c, GOLDEN[name + ".c"]) <= BF16_REL_L2


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_rebinding_a_name_or_refreshing_drops_the_derived_weight_copies(precision):
    """Derived copies (bf16 GEMM / adaLN weights) are keyed by the bound tensor's address: binding new contents at the same address, or
    changing a bound tensor in place and calling refresh(), must be seen by the next call."""
    k = cases.block_case("block_dual_hs64")
    B, Tc, Cd = k["c"].shape
    Tx = k["x"].shape[1]
    args = (B, Tc, Tx, Cd, k["NH"], k["mlp_expand"], True, True, False)

    def fresh(params):
        c, x = M.Dit_block(dev(k["y"]), dev(k["c"]), dev(k["x"]), dev_params(params), *args, precision=precision)
        return host(c), host(x)

    P2 = dict(k["params"])
    for n in ("latent_mlp.lin2.weight", "latent_ada_lnorm.linear.weight", "context_to_qkv.weight"):
        P2[n] = np.ascontiguousarray(P2[n][::-1] * 1.5)
    want1, want2 = fresh(k["params"]), fresh(P2)
    assert not np.array_equal(want1[1], want2[1])
    ctx = M.Context()
    try:
        dP = dev_params(k["params"])
        ctx.bind(dP)
        run = lambda: tuple(host(t) for t in ctx.block(dev(k["y"]), dev(k["c"]), dev(k["x"]), *args, precision=precision))  # noqa: E731
        got = run()
        assert np.array_equal(got[1], want1[1]) and np.array_equal(got[0], want1[0])
        for n in ("latent_mlp.lin2.weight", "latent_ada_lnorm.linear.weight"):   # new contents at the same address, bound again
            dP[n].copy_(dev(P2[n]))
            ctx.bind({n: dP[n]})
        dP["context_to_qkv.weight"].copy_(dev(P2["context_to_qkv.weight"]))      # changed in place without re-binding: refresh()
        ctx.refresh(precision)
        got = run()
        assert np.array_equal(got[1], want2[1]) and np.array_equal(got[0], want2[0])
    finally:
        ctx.close()


def test_prepare_builds_the_bf16_copies_ahead_of_the_first_call():
    """After refresh() the first bf16 call finds every copy: shown with the entry point that refuses to allocate."""
    k = cases.block_case("block_dual_hs64")
    B, Tc, Cd = k["c"].shape
    Tx = k["x"].shape[1]
    args = (B, Tc, Tx, Cd, k["NH"], k["mlp_expand"], True, True, False)
    ctx = M.Context()
    try:
        ctx.bind(dev_params(k["params"]))
        ctx.refresh("bf16")
        c, x = ctx.block_static(dev(k["y"]), dev(k["c"]), dev(k["x"]), *args, precision="bf16")
        c2, x2 = ctx.block(dev(k["y"]), dev(k["c"]), dev(k["x"]), *args, precision="bf16")
        assert torch.equal(x, x2) and torch.equal(c, c2)
        assert rel_l2(host(x), GOLDEN["block_dual_hs64.x"]) <= BF16_REL_L2
    finally:
        ctx.close()


@pytest.mark.parametrize("dual", [True, False])
def test_block_fp32_baseline_config1_vs_float64(dual):
    """The CPU-runnable benchmark configuration at full size (B=1, 256 image + 77 text tokens, width 1536): the CPU oracle needs a minute for this,
    so the check is against the float64 numpy statement of the block that tests/test_oracle.py pins to the oracle."""
    k = _wide_case(1, 77, 256, dual, False, 21)
    c, x = run_gpu_block(k)
    c64, x64 = block64(k["y"], k["c"], k["x"], k["params"], 24, dual, True, False)
    assert max_abs(x, x64) <= F32_TOL and max_abs(c, c64) <= F32_TOL


@pytest.mark.parametrize("dual,discard,B,Tx", [(True, False, 2, 1024), (False, True, 2, 1024), (True, False, 1, 4096)])
def test_block_bf16_at_512px_and_1024px_token_counts_vs_float64(dual, discard, B, Tx):
    """The block at the token counts of BASELINE config 3 (batch 2, 1024 image + 154 text tokens, width 1536) and, one batch element, of
    the headline shape (4096 + 154), with weights of standard deviation 0.05 so that the modulation vectors and gates are of order 2
    and every branch weighs heavily in the result: the bf16 path against the float64 statement of the block directly (not through
    the fp32 GPU path), and the fp32 path against the same."""
    rng = np.random.Generator(np.random.Philox(71))
    C, NH = 1536, 24
    params = synthetic_params_numpy(block_param_shapes(C, 4, dual, True, discard, C // NH), 72, 0.05, 0.05)
    k = dict(y=rng.standard_normal((B, C), dtype=np.float32), c=rng.standard_normal((B, 154, C), dtype=np.float32),
             x=rng.standard_normal((B, Tx, C), dtype=np.float32), params=params, NH=NH, mlp_expand=4, use_dual=dual, use_qk_norm=True,
             discard_context=discard)
    c64, x64 = block64(k["y"], k["c"], k["x"], k["params"], NH, dual, True, discard)
    assert rel_l2(x64 - k["x"], k["x"]) > 1.0                     # the update is larger than what it is added to
    c32, x32 = run_gpu_block(k, "fp32")
    assert rel_l2(x32, x64) <= 1e-5
    c16, x16 = run_gpu_block(k, "bf16")
    assert rel_l2(x16, x64) <= BF16_REL_L2
    if not discard:
        assert rel_l2(c32, c64) <= 1e-5 and rel_l2(c16, c64) <= BF16_REL_L2
    else:
        assert np.array_equal(c16, k["c"])


def test_block_at_the_sizes_of_the_reference_block_test():
    """module_tests/dit_block.py:9-22: batch 16, 512 image + 154 text tokens, width 768, 12 heads of 64, mlp_expand 2, the extra
    self-attention and qk-norm on, y = silu(randn). The reference script only prints its differences; here both precisions are held
    to the float64 statement of the block (the CPU oracle would need minutes), and the sixteen batch elements go through the
    modulation projections in two groups of eight."""
    rng = np.random.Generator(np.random.Philox(81))
    B, Tc, Tx, C, NH, E = 16, 154, 512, 768, 12, 2
    params = synthetic_params_numpy(block_param_shapes(C, E, True, True, False, C // NH), 82, 0.03, 0.03)
    y = rng.standard_normal((B, C), dtype=np.float32)
    k = dict(y=(y / (1 + np.exp(-y))).astype(np.float32), c=rng.standard_normal((B, Tc, C), dtype=np.float32),
             x=rng.standard_normal((B, Tx, C), dtype=np.float32), params=params, NH=NH, mlp_expand=E, use_dual=True, use_qk_norm=True,
             discard_context=False)
    c64, x64 = block64(k["y"], k["c"], k["x"], k["params"], NH, True, True, False)
    c32, x32 = run_gpu_block(k, "fp32")
    assert max_abs(x32, x64) <= F32_TOL and max_abs(c32, c64) <= F32_TOL
    c16, x16 = run_gpu_block(k, "bf16")
    assert rel_l2(x16, x64) <= BF16_REL_L2 and rel_l2(c16, c64) <= BF16_REL_L2
    # every element separately (a wrong row of modulation vectors for elements 8..15 would hide in a norm over the batch)
    for b in range(B):
        assert rel_l2(x16[b], x64[b]) <= BF16_REL_L2 and max_abs(x32[b], x64[b]) <= F32_TOL, b


def test_block_zero_gates_is_identity_on_gpu():
    k = _wide_case(1, 77, 256, True, False, 31)
    P = dict(k["params"])
    for pre, nch in (("context_", 6), ("latent_", 9)):
        w, b = P[pre + "ada_lnorm.linear.weight"].copy(), P[pre + "ada_lnorm.linear.bias"].copy()
        for g in (2, 5, 8):
            if g < nch:
                w[:, g * 1536:(g + 1) * 1536] = 0
                b[g * 1536:(g + 1) * 1536] = 0
        P[pre + "ada_lnorm.linear.weight"], P[pre + "ada_lnorm.linear.bias"] = w, b
    k["params"] = P
    for prec in ("fp32", "bf16"):
        c, x = run_gpu_block(k, prec)
        assert np.array_equal(c, k["c"]) and np.array_equal(x, k["x"])


@pytest.mark.parametrize("dual,discard,Tc,Tx", [(True, False, 77, 256), (False, True, 77, 256), (True, False, 154, 1000), (False, False, 0, 130)])
def test_block_bf16_vs_fp32(dual, discard, Tc, Tx):
    k = _wide_case(2, Tc, Tx, dual, discard, 41)
    c32, x32 = run_gpu_block(k, "fp32")
    c16, x16 = run_gpu_block(k, "bf16")
    # compare the update the block applied, not the O(1) residual it was added to
    assert rel_l2(x16 - k["x"], x32 - k["x"]) <= 2 * BF16_REL_L2
    assert rel_l2(x16, x32) <= BF16_REL_L2
    if not discard and Tc:
        assert rel_l2(c16, c32) <= BF16_REL_L2


@pytest.mark.parametrize("splits", [0, 3, 8, -1])
def test_block_bf16_with_every_context_split_setting(splits):
    """The attention of a block with many latent and few context tokens is taken apart by queries, the context queries split along
    the keys (17 key tiles here, which 8 splits cannot share without leaving one empty: the library then uses fewer). Whatever the
    setting, the block stays within the bf16 criterion of the fp32 path, and the latent rows do not depend on it at all."""
    from sd3_c_amd import lib as L_
    k = _wide_case(1, 20, 1040, True, False, 61, C=128, NH=2)
    c32, x32 = run_gpu_block(k, "fp32")
    try:
        L_.call("sd3_tune", b"attention_context_splits", splits)
        c16, x16 = run_gpu_block(k, "bf16")
        L_.call("sd3_tune", b"attention_context_splits", 0)
        c0, x0 = run_gpu_block(k, "bf16")
    finally:
        L_.call("sd3_tune", b"attention_context_splits", -1)
    assert rel_l2(x16, x32) <= BF16_REL_L2 and rel_l2(c16, c32) <= BF16_REL_L2
    assert np.array_equal(x16, x0)                 # latent rows: same kernel path, same bits
    assert rel_l2(c16, c0) <= 2e-3                 # context rows: merged partial sums, bf16 rounding apart


def test_block_missing_weight_and_bad_shapes():
    from sd3_c_amd import lib as L_
    k = cases.block_case("block_dual_hs64")
    P = dict(k["params"])
    del P["latent_dual_to_qkv.weight"]
    k2 = dict(k, params=P)
    with pytest.raises(L_.Sd3Error) as e:
        run_gpu_block(k2)
    assert e.value.status == 2  # SD3_ERR_MISSING_PARAM
    run_gpu_block(dict(k2, use_dual=False, params={n: v for n, v in P.items() if "dual" not in n} | {
        "latent_ada_lnorm.linear.weight": np.ascontiguousarray(k["params"]["latent_ada_lnorm.linear.weight"][:, :6 * 128]),
        "latent_ada_lnorm.linear.bias": np.ascontiguousarray(k["params"]["latent_ada_lnorm.linear.bias"][:6 * 128])}))
    with pytest.raises(L_.Sd3Error) as e:
        M.Dit_block(dev(k["y"]), dev(k["c"]), dev(k["x"]), dev_params(k["params"]), 1, 7, 16, 128, 3, 4, True, True, False)  # 128 % 3 != 0
    assert e.value.status == 1
    with pytest.raises(L_.Sd3Error) as e:
        run_gpu_block(k, "bf16") if False else M.Dit_block(dev(k["y"]), dev(k["c"]), dev(k["x"]), dev_params(k["params"]), 1, 7, 16, 128, 4, 4, True,
                                                            True, False, precision="bf16")  # head_dim 32 on the bf16 path
    assert e.value.status == 3
