"""The fp8 (OCP e4m3) GEMM path, which has no counterpart in the reference: the kernel against float64 arithmetic on the very
values it is given (the quantised operands, decoded), the quantisers against their definition, and the forward with fp8 MLPs against
the fp32 path, measured with the bf16 path's criterion (relative L2 of the final velocity <= 1e-2), which it does not meet."""
import numpy as np
import pytest
import torch

from gpu_util import M, dev, dev_params, host, rel_l2, BF16_REL_L2
from sd3_c_amd import lib as L
from sd3_c_amd.config import sd35_medium
from test_gpu_dit import _synthetic_device_params, _inputs

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


def _quantise(A_bf16, W_f32, per_tensor):
    Mr, K = A_bf16.shape
    N = W_f32.shape[1]
    aq = torch.zeros((Mr, K), device="cuda", dtype=torch.uint8)
    sa = torch.zeros(Mr, device="cuda")
    wq = torch.zeros((N, K), device="cuda", dtype=torch.uint8)
    sw = torch.zeros(N, device="cuda")
    L.call("sd3_quantize_rows_fp8", A_bf16.data_ptr(), aq.data_ptr(), sa.data_ptr(), Mr, K, per_tensor, None)
    L.call("sd3_quantize_weight_fp8", W_f32.data_ptr(), wq.data_ptr(), sw.data_ptr(), K, N, per_tensor, None)
    torch.cuda.synchronize()
    return aq, sa, wq, sw


@pytest.mark.parametrize("per_tensor", [0, 1])
def test_quantisers_follow_their_definition(per_tensor):
    g = torch.Generator(device="cuda").manual_seed(3)
    A = (torch.randn((300, 256), device="cuda", generator=g) * torch.rand((300, 1), device="cuda", generator=g) * 5).bfloat16()
    A[7] = 0  # an all-zero row must not divide by zero
    W = torch.randn((256, 192), device="cuda", generator=g) * 0.05
    aq, sa, wq, sw = _quantise(A, W, per_tensor)
    amax_a = A.float().abs().amax(1)
    amax_w = W.abs().amax(0)
    if per_tensor:
        amax_a, amax_w = amax_a.max().expand_as(amax_a), amax_w.max().expand_as(amax_w)
    want_sa = torch.where(amax_a > 0, amax_a / 448.0, torch.ones_like(amax_a))
    assert torch.allclose(sa, want_sa, rtol=1e-6) and torch.allclose(sw, amax_w / 448.0, rtol=1e-6)
    # decoded values: the nearest e4m3 value of x / s (round to nearest even, as torch's conversion does)
    assert torch.equal(aq.view(E4M3).float(), (A.float() / sa[:, None]).to(E4M3).float())
    # (the weight is divided as W * (448 / amax), one rounding away from W / s: compare the decoded values loosely, and exactly against that expression)
    amax_w_safe = torch.where(amax_w > 0, amax_w, torch.ones_like(amax_w))
    assert torch.equal(wq.view(E4M3).float(), (W * (448.0 / amax_w_safe)).t().contiguous().to(E4M3).float())
    assert float(aq.view(E4M3).float().abs().max()) <= 448.0


@pytest.mark.parametrize("Mr,N,K,epi,out_f32", [(8192, 1536, 1536, 0, 1), (1000, 6144, 1536, 1, 0), (308, 1536, 6144, 0, 1), (5, 200, 128, 1, 0), (257, 136, 384, 0, 0)])
def test_gemm_fp8_is_exact_on_its_operands_and_close_to_the_unquantised_product(Mr, N, K, epi, out_f32):
    g = torch.Generator(device="cuda").manual_seed(Mr + N)
    A = torch.randn((Mr, K), device="cuda", generator=g).bfloat16()
    W = 0.05 * torch.randn((K, N), device="cuda", generator=g)
    bias = torch.randn(N, device="cuda", generator=g)
    aq, sa, wq, sw = _quantise(A, W, 0)
    out = torch.zeros((Mr, N), device="cuda", dtype=torch.float32 if out_f32 else torch.bfloat16)
    L.call("sd3_gemm_fp8", aq.data_ptr(), sa.data_ptr(), wq.data_ptr(), sw.data_ptr(), bias.data_ptr(), out.data_ptr(), Mr, N, K, epi, out_f32, None)
    torch.cuda.synchronize()
    act = (lambda t: torch.nn.functional.gelu(t, approximate="tanh")) if epi == 1 else (lambda t: t)
    # what the kernel is asked to compute, in float64, from the decoded operands
    exact = act((aq.view(E4M3).double() @ wq.view(E4M3).double().t()) * sa.double()[:, None] * sw.double()[None, :] + bias.double())
    # (measured 1.3e-5 with fp32 output: the instruction's 64-product sums are a little coarser than fp32 fused multiply-adds)
    assert rel_l2(host(out), host(exact)) <= (5e-5 if out_f32 else 4e-3)
    # and how far fp8 operands are from the unquantised product: e4m3 keeps 3 mantissa bits (2^-4 relative rounding on each operand)
    full = act(A.double() @ W.double() + bias.double())
    err = rel_l2(host(out), host(full))
    assert err <= 0.06, err


def _sd35_case(side, B=2, seed=77):
    cfg = sd35_medium()
    k = _inputs(cfg, B, 154, side, side, seed)
    return cfg, k, _synthetic_device_params(cfg, seed + 1)


@pytest.mark.parametrize("side", [64, 128])
def test_forward_with_fp8_mlps_vs_fp32_path(side):
    """Configurations 3 (512x512) and 4 (1024x1024, the headline shape) with the MLP layers in fp8: relative L2 of the final velocity
    against the fp32 path, beside the bf16 path's own error. MEASURED: e4m3 operands (3 mantissa bits, about 2 % r.m.s. rounding
    on each operand of every product) leave 4-5e-2 on the final velocity whichever way the factors are chosen -- per token row and
    per output channel, or one per tensor (the synthetic N(0, 0.02) weights have no outliers for the finer factors to absorb) --
    against 2-5e-3 for bf16. That is OUTSIDE the 1e-2 criterion, so fp8 stays an opt-in precision and is never the benchmark's;
    this test pins the measured error so that a regression (or an improvement) shows."""
    cfg, k, P = _sd35_case(side)
    args = [dev(k["pooled"]), dev(k["captions"]), dev(k["latent"]), dev(k["timesteps"])]
    outs = {}
    for prec in ("fp32", "bf16", "bf16+fp8", "bf16+fp8-tensor"):
        den = M.Denoiser(P, cfg, prec)
        outs[prec] = host(den(*args))
        den.ctx.close()
    e_bf16 = rel_l2(outs["bf16"], outs["fp32"])
    e_row = rel_l2(outs["bf16+fp8"], outs["fp32"])
    e_tensor = rel_l2(outs["bf16+fp8-tensor"], outs["fp32"])
    print(f"side {side}: rel-L2 vs fp32: bf16 {e_bf16:.2e}, fp8 per-row/channel {e_row:.2e}, fp8 per-tensor {e_tensor:.2e}")
    assert e_bf16 <= BF16_REL_L2
    assert BF16_REL_L2 < e_row <= 7e-2, e_row        # fails the criterion the bf16 path meets; bounded by what was measured
    assert BF16_REL_L2 < e_tensor <= 7e-2, e_tensor
