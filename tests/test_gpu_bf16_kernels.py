"""The two MFMA kernels of the bf16 path on their own, against fp32 torch arithmetic on the bf16-rounded inputs."""
import numpy as np
import pytest
import torch

from gpu_util import M, host, rel_l2
from sd3_c_amd import lib as L

pytestmark = pytest.mark.gpu


def _naive_joint_attention(qkv0, qkv1, rq, rk, B, T0, T1, NH, HS):
    """fp32 softmax(QK^T/8)V over [segment 0 ; segment 1] with per-head RMSNorm (eps 1e-6) of q and k, from bf16-rounded inputs."""
    C = NH * HS

    def split(qkv, T, wq, wk):
        q, k, v = qkv.float().view(B, T, 3, NH, HS).unbind(2)

        def rms(a, w):
            return a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + 1e-6) * w

        return rms(q, wq), rms(k, wk), v

    q0, k0, v0 = split(qkv0, T0, rq[0], rk[0])
    parts = [(q0, k0, v0)]
    if T1:
        parts.append(split(qkv1, T1, rq[1], rk[1]))
    q, k, v = (torch.cat([p[i] for p in parts], 1).transpose(1, 2) for i in range(3))  # (B,NH,T,HS)
    out = torch.empty_like(q)
    for b in range(B):
        for h0 in range(0, NH, 4):
            s = q[b, h0:h0 + 4] @ k[b, h0:h0 + 4].transpose(-1, -2) / 8.0
            out[b, h0:h0 + 4] = torch.softmax(s, -1) @ v[b, h0:h0 + 4]
    return out.transpose(1, 2).reshape(B, T0 + T1, C)


@pytest.mark.parametrize("B,T0,T1,NH", [(2, 154, 4096, 24), (1, 154, 1024, 24), (2, 7, 130, 4), (1, 0 + 64, 0, 2), (1, 1, 63, 3),
                                        (1, 64, 64, 1), (1, 3, 62, 1), (1, 1, 0, 1), (2, 33, 224, 2), (1, 100, 29, 2), (1, 60, 133, 1)])
def test_flash_attention_bf16(B, T0, T1, NH):
    """The headline attention shape is the first case: B=2, 24 heads of 64, 154 text + 4096 image tokens, q/k/v ~ N(0,1). The small cases sit
    on the edges of the 64-key tiles and 32-key halves (one tile exactly, one key into the next tile, a single key, a segment
    boundary inside a tile) and of the three-stage tile ring (1, 2, 3 and 4 tiles)."""
    HS, C = 64, NH * 64
    g = torch.Generator(device="cuda").manual_seed(T0 * 7 + T1)
    qkv0 = torch.randn((B * T0, 3 * C), device="cuda", generator=g).bfloat16()
    qkv1 = torch.randn((B * max(T1, 1), 3 * C), device="cuda", generator=g).bfloat16()
    rq = [1 + 0.1 * torch.randn(HS, device="cuda", generator=g) for _ in range(2)]
    rk = [1 + 0.1 * torch.randn(HS, device="cuda", generator=g) for _ in range(2)]
    out0 = torch.zeros((B * T0, C), device="cuda", dtype=torch.bfloat16)
    out1 = torch.zeros((B * max(T1, 1), C), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_flash_attention_bf16", qkv0.data_ptr(), qkv1.data_ptr() if T1 else None, out0.data_ptr(), out1.data_ptr() if T1 else None,
           rq[0].data_ptr(), rk[0].data_ptr(), rq[1].data_ptr(), rk[1].data_ptr(), B, T0, T1, NH, HS, None)
    ref = _naive_joint_attention(qkv0, qkv1, rq, rk, B, T0, T1, NH, HS)
    got = torch.cat([out0.view(B, T0, C)] + ([out1.view(B, T1, C)] if T1 else []), 1).float()
    assert torch.isfinite(got).all()
    assert rel_l2(host(got), host(ref)) <= 1e-2
    assert float((got - ref).abs().max()) <= 0.05  # outputs are O(1) convex combinations of N(0,1) values


@pytest.mark.parametrize("B,T0,T1,NH,S", [(2, 154, 4096, 24, 4), (1, 77, 1100, 3, 4), (1, 1, 130, 2, 2), (2, 200, 600, 2, 3), (1, 256, 64, 1, 5)])
def test_flash_attention_bf16_taken_apart_by_queries_with_key_splits(B, T0, T1, NH, S):
    """What the block does at the headline shape (first case): latent queries in one set, the context queries split along the keys and
    merged by the combining kernel. Latent rows must equal the one-set kernel bit for bit; context rows agree with it and with fp32
    arithmetic to bf16 rounding."""
    HS, C = 64, NH * 64
    g = torch.Generator(device="cuda").manual_seed(T0 * 3 + T1 + S)
    qkv0 = torch.randn((B * T0, 3 * C), device="cuda", generator=g).bfloat16()
    qkv1 = torch.randn((B * T1, 3 * C), device="cuda", generator=g).bfloat16()
    ref0 = torch.zeros((B * T0, C), device="cuda", dtype=torch.bfloat16)
    ref1 = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_flash_attention_bf16", qkv0.data_ptr(), qkv1.data_ptr(), ref0.data_ptr(), ref1.data_ptr(), None, None, None, None, B, T0, T1, NH, HS, None)
    out0, out1 = torch.zeros_like(ref0), torch.zeros_like(ref1)
    ws = torch.empty(B * NH * ((T0 + 255) // 256) * S * 256 * 66, device="cuda")
    ws.fill_(float("nan"))  # whatever is read must have been written by this call
    L.call("sd3_flash_attention_bf16_split", qkv0.data_ptr(), qkv1.data_ptr(), out0.data_ptr(), out1.data_ptr(), B, T0, T1, NH, HS, S, ws.data_ptr(),
           ws.numel() * 4, None)
    torch.cuda.synchronize()
    assert torch.equal(out1, ref1)
    assert torch.isfinite(out0.float()).all()
    assert float((out0.float() - ref0.float()).abs().max()) <= 0.03  # two bf16 roundings of O(1) values apart at most
    # fp32 softmax(q k^T / 8) v for the context queries over the joint keys (no norm in this call)
    q0, k0, v0 = qkv0.float().view(B, T0, 3, NH, HS).unbind(2)
    _, k1, v1 = qkv1.float().view(B, T1, 3, NH, HS).unbind(2)
    k, v = torch.cat([k0, k1], 1), torch.cat([v0, v1], 1)
    p = torch.softmax(torch.einsum("bqhd,bkhd->bhqk", q0, k) / 8.0, -1)
    naive = torch.einsum("bhqk,bkhd->bqhd", p, v).reshape(B * T0, C)
    assert rel_l2(host(out0), host(naive)) <= 1e-2
    with pytest.raises(L.Sd3Error):  # more splits than key tiles
        L.call("sd3_flash_attention_bf16_split", qkv0.data_ptr(), qkv1.data_ptr(), out0.data_ptr(), out1.data_ptr(), B, T0, T1, NH, HS, 4096, ws.data_ptr(),
               1 << 40, None)
    with pytest.raises(L.Sd3Error):  # workspace too small
        L.call("sd3_flash_attention_bf16_split", qkv0.data_ptr(), qkv1.data_ptr(), out0.data_ptr(), out1.data_ptr(), B, T0, T1, NH, HS, S, ws.data_ptr(), 16, None)


def test_flash_attention_bf16_headline_size_properties():
    """Size-independent properties at the benchmark's attention shape (B=2, 24 heads of 64, 154 text + 4096 image tokens), where no
    CPU reference finishes: (1) with V = 1 every output is 1 (each row of the softmax sums to one, whatever the scores);
    (2) permuting the image tokens' keys and values together leaves every output unchanged up to the order of summation."""
    B, T0, T1, NH, HS = 2, 154, 4096, 24, 64
    C = NH * HS
    g = torch.Generator(device="cuda").manual_seed(99)
    qkv0 = torch.randn((B * T0, 3 * C), device="cuda", generator=g).bfloat16()
    qkv1 = torch.randn((B * T1, 3 * C), device="cuda", generator=g).bfloat16()

    def run(a0, a1):
        o0 = torch.zeros((B * T0, C), device="cuda", dtype=torch.bfloat16)
        o1 = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
        L.call("sd3_flash_attention_bf16", a0.data_ptr(), a1.data_ptr(), o0.data_ptr(), o1.data_ptr(), None, None, None, None, B, T0, T1, NH, HS, None)
        torch.cuda.synchronize()
        return o0.float(), o1.float()

    ones0, ones1 = qkv0.clone(), qkv1.clone()
    ones0[:, 2 * C:] = 1
    ones1[:, 2 * C:] = 1
    o0, o1 = run(ones0, ones1)
    assert float((o0 - 1).abs().max()) <= 1e-2 and float((o1 - 1).abs().max()) <= 1e-2
    base0, base1 = run(qkv0, qkv1)
    perm = torch.randperm(T1, device="cuda", generator=g)
    shuffled = qkv1.view(B, T1, 3, C).clone()
    shuffled[:, :, 1:] = shuffled[:, perm][:, :, 1:]     # keys and values move together, queries stay where they are
    p0, p1 = run(qkv0, shuffled.view(B * T1, 3 * C).contiguous())
    assert float((p0 - base0).abs().max()) <= 0.02 and float((p1 - base1).abs().max()) <= 0.02
    assert rel_l2(host(p1), host(base1)) <= 5e-3 and rel_l2(host(p0), host(base0)) <= 5e-3


def test_flash_attention_bf16_without_qk_norm_and_ones_v():
    B, T0, T1, NH, HS = 1, 10, 200, 2, 64
    C = NH * HS
    qkv0 = torch.randn((B * T0, 3 * C), device="cuda").bfloat16()
    qkv1 = torch.randn((B * T1, 3 * C), device="cuda").bfloat16()
    qkv0[:, 2 * C:] = 1
    qkv1[:, 2 * C:] = 1
    out0 = torch.zeros((B * T0, C), device="cuda", dtype=torch.bfloat16)
    out1 = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_flash_attention_bf16", qkv0.data_ptr(), qkv1.data_ptr(), out0.data_ptr(), out1.data_ptr(), None, None, None, None, B, T0, T1, NH, HS, None)
    assert float((out0.float() - 1).abs().max()) <= 1e-2 and float((out1.float() - 1).abs().max()) <= 1e-2  # rows of softmax sum to one


@pytest.mark.parametrize("Mr,N,K,epi", [(8192, 1536, 1536, 0), (308, 4608, 1536, 0), (1000, 6144, 1536, 1), (130, 64, 1536, 0), (257, 1536, 6144, 0), (5, 200, 64, 1)])
def test_gemm_bf16(Mr, N, K, epi):
    g = torch.Generator(device="cuda").manual_seed(Mr + N)
    A = torch.randn((Mr, K), device="cuda", generator=g).bfloat16()
    W = (0.05 * torch.randn((K, N), device="cuda", generator=g))
    bias = torch.randn(N, device="cuda", generator=g)
    Wp = torch.empty((N, K), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_pack_weight_bf16", W.data_ptr(), Wp.data_ptr(), K, N, None)
    assert torch.equal(Wp, W.bfloat16().t().contiguous())
    out = torch.empty((Mr, N), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_gemm_bf16", A.data_ptr(), Wp.data_ptr(), bias.data_ptr(), out.data_ptr(), Mr, N, K, epi, None)
    ref = A.float() @ W.bfloat16().float() + bias
    if epi == 1:
        ref = torch.nn.functional.gelu(ref, approximate="tanh")
    assert rel_l2(host(out), host(ref)) <= 5e-3  # bf16 rounding of the output is 2^-9 relative


@pytest.mark.parametrize("Mr,N,K,epi", [(2304, 1536, 1536, 1), (300, 320, 6144, 0)])
def test_gemm_bf16_result_does_not_depend_on_tile_shape(Mr, N, K, epi):
    """Every output element is accumulated over K in the same order whatever tile it falls into: bit-identical results."""
    g = torch.Generator(device="cuda").manual_seed(K + N)
    A = torch.randn((Mr, K), device="cuda", generator=g).bfloat16()
    Wp = (0.05 * torch.randn((N, K), device="cuda", generator=g)).bfloat16()
    bias = torch.randn(N, device="cuda", generator=g)
    outs = []
    try:
        for tile in (128, 256, 0, 192):
            L.call("sd3_gemm_bf16_force_tile", tile)
            out = torch.zeros((Mr, N), device="cuda", dtype=torch.bfloat16)
            L.call("sd3_gemm_bf16", A.data_ptr(), Wp.data_ptr(), bias.data_ptr(), out.data_ptr(), Mr, N, K, epi, None)
            outs.append(out)
    finally:
        L.call("sd3_gemm_bf16_force_tile", 0)
    assert all(torch.equal(outs[0], o) for o in outs[1:])
    with pytest.raises(L.Sd3Error):
        L.call("sd3_gemm_bf16_force_tile", 64)


def test_flash_attention_bf16_late_maximum_moves_the_reference():
    """The last keys score about 40 bits above everything before them, so the reference point of the online softmax has
    to move long after the first tile (the rescale path) and the early keys must fade out without overflow. Large scores
    amplify the rounding of the pre-scaled bf16 query operand, so the comparison is against fp32 arithmetic on that same
    rounded operand (q * log2(e)/8 in bf16), which is what the kernel documents it multiplies."""
    B, T1, NH, HS = 1, 300, 2, 64
    C = NH * HS
    g = torch.Generator(device="cuda").manual_seed(11)
    qkv = torch.randn((B * T1, 3 * C), device="cuda", generator=g)
    qkv[-5:, C:2 * C] *= 12.0      # the last five keys dominate
    qkv = qkv.bfloat16()
    out = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_flash_attention_bf16", qkv.data_ptr(), None, out.data_ptr(), None, None, None, None, None, B, T1, 0, NH, HS, None)
    q, k, v = qkv.float().view(B, T1, 3, NH, HS).unbind(2)
    q2 = (q * (1.4426950408889634 / 8.0)).bfloat16().float()
    s2 = torch.einsum("bqhd,bkhd->bhqk", q2, k)
    assert float(s2.max()) > 40.0  # base-2 exponents: far beyond the 2^30 head-room of a fixed reference
    p = torch.exp2(s2 - s2.max(-1, keepdim=True).values)
    ref = torch.einsum("bhqk,bkhd->bqhd", p / p.sum(-1, keepdim=True), v).reshape(B * T1, C)
    assert torch.isfinite(out.float()).all()
    assert float((out.float() - ref).abs().max()) <= 0.05


@pytest.mark.parametrize("T0,T1", [(0, 256), (0, 257), (0, 287), (0, 288), (0, 289), (0, 319), (0, 320), (0, 321), (0, 351), (0, 352), (0, 353), (0, 383),
                                   (5, 315), (31, 289), (32, 288), (33, 330), (64, 256), (100, 412), (154, 1024 + 37)])
def test_flash_attention_bf16_where_fast_tiles_hand_over_to_masked_ones(T0, T1):
    """Sequence lengths on every side of the 64-key tile and 32-key half-tile boundaries, long enough (five tiles and more) for the
    tiles without masked keys to run with the reference fixed at zero: the last one or two tiles, which hold the keys beyond the
    sequence, go through the general path, and the unit in flight across the hand-over must be one without masked keys."""
    B, NH, HS = 1, 2, 64
    C = NH * HS
    g = torch.Generator(device="cuda").manual_seed(T0 * 1000 + T1)
    qkv0 = torch.randn((B * max(T0, 1), 3 * C), device="cuda", generator=g).bfloat16()
    qkv1 = torch.randn((B * T1, 3 * C), device="cuda", generator=g).bfloat16()
    rq = [1 + 0.1 * torch.randn(HS, device="cuda", generator=g) for _ in range(2)]
    rk = [1 + 0.1 * torch.randn(HS, device="cuda", generator=g) for _ in range(2)]
    # normalise on the host (the kernel then takes q and k as they are: the path with fast tiles)
    def normed(qkv, T, wq, wk):
        q, k, v = qkv.float().view(B, T, 3, NH, HS).unbind(2)
        rms = lambda a, w: a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + 1e-6) * w
        return torch.stack([rms(q, wq), rms(k, wk), v], 2).reshape(B * T, 3 * C).bfloat16()
    n0 = normed(qkv0, max(T0, 1), rq[0], rk[0]); n1 = normed(qkv1, T1, rq[1], rk[1])
    out0 = torch.zeros((B * max(T0, 1), C), device="cuda", dtype=torch.bfloat16)
    out1 = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
    if T0:
        L.call("sd3_flash_attention_bf16", n0.data_ptr(), n1.data_ptr(), out0.data_ptr(), out1.data_ptr(), None, None, None, None, B, T0, T1, NH, HS, None)
        parts = [n0.float().view(B, T0, 3, NH, HS), n1.float().view(B, T1, 3, NH, HS)]
        got = torch.cat([out0.view(B, T0, C), out1.view(B, T1, C)], 1).float()
    else:
        L.call("sd3_flash_attention_bf16", n1.data_ptr(), None, out1.data_ptr(), None, None, None, None, None, B, T1, 0, NH, HS, None)
        parts = [n1.float().view(B, T1, 3, NH, HS)]
        got = out1.view(B, T1, C).float()
    q, k, v = (torch.cat([p[:, :, i] for p in parts], 1).transpose(1, 2) for i in range(3))  # (B,NH,T,HS)
    ref = (torch.softmax(q @ k.transpose(-1, -2) / 8.0, -1) @ v).transpose(1, 2).reshape(B, T0 + T1, C)
    assert torch.isfinite(got).all()
    assert rel_l2(host(got), host(ref)) <= 1e-2
    assert float((got - ref).abs().max()) <= 0.05


@pytest.mark.parametrize("case", ["overflow_mid", "overflow_to_inf", "first_tile_vanishes", "everything_vanishes", "harmless"])
def test_flash_attention_bf16_fast_tiles_give_way_to_the_general_path(case):
    """Tiles in which no key is masked run with the softmax reference fixed at zero, as long as every lane's row sums stay between
    2^-64 (after the first tile) and 2^40; otherwise the work item starts again on the general path. Cases: scores of 2^40 and more
    in the middle of the sequence; scores beyond the fp32 exponent range (the fast tiles produce infinities before the check
    sees them); queries whose scores against the whole first tile are below -100 (their probabilities there round to nothing)
    while later keys are ordinary; queries whose scores against every key are below -100 (with a reference of zero their row sums
    would be zero); and an ordinary input, which stays on the fast tiles. Reference as in the test above."""
    B, T1, NH, HS = 1, 1000, 2, 64
    C = NH * HS
    g = torch.Generator(device="cuda").manual_seed(23)
    qkv = torch.randn((B * T1, 3 * C), device="cuda", generator=g)
    if case == "overflow_mid":
        qkv[400:405, C:2 * C] *= 12.0
    elif case == "overflow_to_inf":
        qkv[130:140, C:2 * C] *= 60.0
    elif case == "first_tile_vanishes":
        u = torch.nn.functional.normalize(torch.randn(NH, HS, device="cuda", generator=g), dim=-1)
        qkv[:64, C:2 * C] = (-40.0 * u).reshape(1, C) + 0.1 * qkv[:64, C:2 * C]     # the first tile's keys all point one way ...
        qkv[500:, 0:C] = (24.0 * u).reshape(1, C) + qkv[500:, 0:C]                  # ... and half of the queries the opposite way
    elif case == "everything_vanishes":
        u = torch.nn.functional.normalize(torch.randn(NH, HS, device="cuda", generator=g), dim=-1)
        qkv[:, C:2 * C] = (-40.0 * u).reshape(1, C) + qkv[:, C:2 * C]
        qkv[500:, 0:C] = (24.0 * u).reshape(1, C) + qkv[500:, 0:C]
    qkv = qkv.bfloat16()
    out = torch.zeros((B * T1, C), device="cuda", dtype=torch.bfloat16)
    L.call("sd3_flash_attention_bf16", qkv.data_ptr(), None, out.data_ptr(), None, None, None, None, None, B, T1, 0, NH, HS, None)
    q, k, v = qkv.float().view(B, T1, 3, NH, HS).unbind(2)
    q2 = (q * (1.4426950408889634 / 8.0)).bfloat16().float()
    s2 = torch.einsum("bqhd,bkhd->bhqk", q2, k)
    if case == "everything_vanishes":
        assert float(s2[:, :, 500:].max()) < -130.0  # 2^-130 is below the smallest normal fp32 number
    elif case == "overflow_mid":
        assert 40.0 < float(s2.max()) < 120.0
    elif case == "overflow_to_inf":
        assert float(s2.max()) > 200.0
    elif case == "first_tile_vanishes":
        assert float(s2[:, :, 500:, :64].max()) < -100.0 and float(s2[:, :, 500:, 64:].max(-1).values.min()) > -40.0
    else:
        assert float(s2.abs().max()) < 30.0
    p = torch.exp2(s2 - s2.max(-1, keepdim=True).values)
    ref = torch.einsum("bhqk,bkhd->bqhd", p / p.sum(-1, keepdim=True), v).reshape(B * T1, C)
    assert torch.isfinite(out.float()).all()
    assert float((out.float() - ref).abs().max()) <= 0.05
    assert rel_l2(host(out.float()), host(ref)) <= 1e-2


def test_cast_rounds_to_nearest_even():
    x = torch.randn(100000, device="cuda") * 100
    x[:4] = torch.tensor([0.0, -0.0, float("inf"), 1.00390625])  # the last one is exactly halfway between two bf16 values
    out = torch.empty(100000, device="cuda", dtype=torch.bfloat16)
    L.call("sd3_cast_f32_to_bf16", x.data_ptr(), out.data_ptr(), x.numel(), None)
    assert torch.equal(out, x.bfloat16())


def test_mfma_probe_reports_a_plausible_rate_and_rejects_bad_arguments():
    """The register-only matrix-instruction loop must land between a tenth of the published bf16 peak and a little above
    it (2.5 PFLOP/s at the maximum clock) for zero operands, and random operands must not be faster than zeros."""
    import ctypes
    z, r = ctypes.c_double(0.0), ctypes.c_double(0.0)
    L.call("sd3_probe_mfma_bf16", 0, 4000, ctypes.byref(z))
    L.call("sd3_probe_mfma_bf16", 1, 4000, ctypes.byref(r))
    assert 250.0 < z.value < 2800.0, z.value
    assert 250.0 < r.value <= z.value * 1.05, (r.value, z.value)
    with pytest.raises(L.Sd3Error):
        L.call("sd3_probe_mfma_bf16", 0, 0, ctypes.byref(z))
    with pytest.raises(L.Sd3Error):
        L.call("sd3_probe_mfma_bf16", 0, 100, None)
