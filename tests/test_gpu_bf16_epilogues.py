"""The fused epilogues and the grouped launches of the bf16 GEMM, each on its own through the C ABI (sd3_gemm_bf16_grouped),
against the CPU oracle's statement of what the epilogue replaces -- linear / partial_linear + rmsnorm_group + gating_mechanism
+ add (modules.cpp:192-198, 475-518, 1223-1236) -- evaluated on the bf16-rounded operands, and at shapes too large for the
oracle against float64 torch arithmetic plus bit-identity across tile shapes and groupings."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as ol
from oracle_lib import fp
from gpu_util import host, rel_l2, max_abs
from sd3_c_amd import lib as L

pytestmark = pytest.mark.gpu


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a)).bfloat16().float().numpy()


class Layer:
    """One linear layer with bf16-rounded operands on both sides: numpy for the oracle, device tensors for the library."""

    def __init__(self, rng, M, K, N, wstd=0.08):
        self.M, self.K, self.N = M, K, N
        self.A = bf16_round(rng.standard_normal((M, K), dtype=np.float32))
        self.W = bf16_round(wstd * rng.standard_normal((K, N), dtype=np.float32))
        self.b = rng.standard_normal(N, dtype=np.float32) * 0.1
        self.dA = torch.from_numpy(self.A).cuda().bfloat16()
        self.dW = torch.from_numpy(self.W).cuda()
        self.db = torch.from_numpy(self.b).cuda()
        self.dWp = torch.empty((N, K), device="cuda", dtype=torch.bfloat16)
        L.call("sd3_pack_weight_bf16", self.dW.data_ptr(), self.dWp.data_ptr(), K, N, None)

    def oracle_linear(self):
        y = np.empty((self.M, self.N), np.float32)
        ol.oracle().orc_linear(fp(self.A), fp(self.W), fp(self.b), fp(y), self.M, self.K, self.N)
        return y

    def problem(self, out, **kw):
        p = L.GemmBf16Problem(A=self.dA.data_ptr(), wpacked=self.dWp.data_ptr(), bias=self.db.data_ptr(), out=out.data_ptr(), M=self.M, N=self.N, K=self.K)
        for k, v in kw.items():
            setattr(p, k, v.data_ptr() if isinstance(v, torch.Tensor) else v)
        return p


def launch(problems, epi, out_f32):
    arr = (L.GemmBf16Problem * len(problems))(*problems)
    L.call("sd3_gemm_bf16_grouped", C.cast(arr, C.c_void_p), len(problems), epi, int(out_f32), None)
    torch.cuda.synchronize()


def oracle_qkv_norm(layer, wq, wk, Cm):
    """partial_linear thirds (modules.cpp:1391-1393) then rmsnorm_group on q and k (modules.cpp:1396-1399)."""
    o = ol.oracle()
    parts = []
    for third, w in ((0, wq), (1, wk), (2, None)):
        y = np.empty((layer.M, Cm), np.float32)
        o.orc_partial_linear(fp(layer.A), fp(layer.W), fp(layer.b), fp(y), layer.M, layer.K, Cm, 3 * Cm, third * Cm)
        if w is not None:
            o.orc_rmsnorm_heads(fp(y), fp(w), C.c_float(1e-6), layer.M * (Cm // 64), 64)
        parts.append(y)
    return np.concatenate(parts, axis=1)


@pytest.mark.parametrize("tile", [0, 128, 256])
def test_qkv_norm_epilogue_three_problems_in_one_launch(tile):
    """The dual block's launch: latent, dual-branch and context projections together, q and k normalised per head."""
    rng = np.random.Generator(np.random.Philox(50))
    Cm = 128
    layers = [Layer(rng, M, Cm, 3 * Cm) for M in (1100, 1100, 77)]
    ws = [(1 + 0.2 * rng.standard_normal(64, dtype=np.float32), 1 + 0.2 * rng.standard_normal(64, dtype=np.float32)) for _ in layers]
    dws = [(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()) for a, b in ws]
    outs = [torch.zeros((l.M, 3 * Cm), device="cuda", dtype=torch.bfloat16) for l in layers]
    try:
        L.call("sd3_gemm_bf16_force_tile", tile)
        launch([l.problem(o, rms_q=q, rms_k=k) for l, o, (q, k) in zip(layers, outs, dws)], 5, False)
    finally:
        L.call("sd3_gemm_bf16_force_tile", 0)
    for l, o, (wq, wk) in zip(layers, outs, ws):
        want = oracle_qkv_norm(l, wq, wk, Cm)
        got = host(o)
        assert rel_l2(got, want) <= 4e-3            # the bf16 output rounding alone is 2^-9 relative per element
        assert max_abs(got, bf16_round(want)) <= 0.04  # at most a couple of bf16 steps on O(1) values
    # each problem alone gives the same bits as inside the group
    alone = torch.zeros_like(outs[2])
    launch([layers[2].problem(alone, rms_q=dws[2][0], rms_k=dws[2][1])], 5, False)
    assert torch.equal(alone, outs[2])


@pytest.mark.parametrize("tile", [0, 128, 256])
def test_gate_residual_epilogue_latent_and_context_in_one_launch(tile):
    """linear + gating_mechanism + add (modules.cpp:1435-1436, 1459-1462): x += gate[b] * (h @ W + bias), fp32 in place."""
    rng = np.random.Generator(np.random.Philox(51))
    B, Tx, Tc, K, N = 2, 600, 19, 256, 192
    lx, lc = Layer(rng, B * Tx, K, N), Layer(rng, B * Tc, K, N)
    gate_ld = 9 * N  # the gate is one chunk of a longer modulation row, as in the block
    res = []
    for l, T, chunk in ((lx, Tx, 2), (lc, Tc, 5)):
        ada = rng.standard_normal((B, gate_ld), dtype=np.float32)
        resid = rng.standard_normal((l.M, N), dtype=np.float32)
        lin = l.oracle_linear()
        gated, want = np.empty_like(lin), np.empty_like(lin)
        gate = np.ascontiguousarray(ada[:, chunk * N:(chunk + 1) * N])
        ol.oracle().orc_gate(fp(lin), fp(gated), fp(gate), B, T, N)
        ol.oracle().orc_add(fp(resid), fp(gated), fp(want), C.c_long(resid.size))
        d_ada, d_x = torch.from_numpy(ada).cuda(), torch.from_numpy(resid).cuda()
        res.append((l, T, chunk, d_ada, d_x, resid, want))
    probs = []
    for l, T, chunk, d_ada, d_x, resid, want in res:
        p = l.problem(d_x, resid=d_x, gate_ld=gate_ld, rows_per_batch=T)
        p.gate = d_ada.data_ptr() + chunk * N * 4
        probs.append(p)
    try:
        L.call("sd3_gemm_bf16_force_tile", tile)
        launch(probs, 3, True)
    finally:
        L.call("sd3_gemm_bf16_force_tile", 0)
    for l, T, chunk, d_ada, d_x, resid, want in res:
        got = host(d_x)
        assert rel_l2(got - resid, want - resid) <= 2e-5   # fp32 accumulation in a different order, nothing else
        assert max_abs(got, want) <= 1e-4


def test_bias_silu_and_row_table_epilogues():
    rng = np.random.Generator(np.random.Philox(52))
    l = Layer(rng, 333, 64, 200)
    lin = l.oracle_linear()
    want = np.empty_like(lin)
    ol.oracle().orc_silu(fp(lin), fp(want), C.c_long(lin.size))
    out = torch.zeros((l.M, l.N), device="cuda")
    launch([l.problem(out)], 2, True)
    assert max_abs(host(out), want) <= 1e-4
    # row table: out[m] = acc + bias + table[m % rows_per_batch] (the position table of PatchEmbedding, modules.cpp:1110-1116)
    rpb = 111
    table = rng.standard_normal((rpb, l.N), dtype=np.float32)
    out = torch.zeros((l.M, l.N), device="cuda")
    launch([l.problem(out, table=torch.from_numpy(table).cuda(), rows_per_batch=rpb)], 4, True)
    assert max_abs(host(out), lin + np.tile(table, (3, 1))) <= 1e-4


def test_grouping_plans_at_block_shapes_give_identical_bits_and_match_float64():
    """Shapes of the headline block (too large for the CPU oracle): one launch for latent + context vs separate launches vs both
    tile shapes -- bit-identical -- and a float64 product on the same bf16 operands."""
    g = torch.Generator(device="cuda").manual_seed(53)
    Cm = 1536

    def mk(M, K, N):
        A = torch.randn((M, K), device="cuda", generator=g).bfloat16()
        Wp = (0.03 * torch.randn((N, K), device="cuda", generator=g)).bfloat16()
        return A, Wp, 0.1 * torch.randn(N, device="cuda", generator=g)

    big, small = mk(8192, Cm, 4 * Cm), mk(308, Cm, 4 * Cm)

    def run(groups, tile):
        outs = {}
        try:
            L.call("sd3_gemm_bf16_force_tile", tile)
            for grp in groups:
                ps = []
                for name in grp:
                    A, Wp, b = big if name == "big" else small
                    outs[name] = torch.zeros((A.shape[0], Wp.shape[0]), device="cuda", dtype=torch.bfloat16)
                    ps.append(L.GemmBf16Problem(A=A.data_ptr(), wpacked=Wp.data_ptr(), bias=b.data_ptr(), out=outs[name].data_ptr(), M=A.shape[0],
                                                N=Wp.shape[0], K=A.shape[1]))
                launch(ps, 1, False)
        finally:
            L.call("sd3_gemm_bf16_force_tile", 0)
        return outs

    base = run([["big", "small"]], 0)
    for groups, tile in (([["big"], ["small"]], 0), ([["big", "small"]], 128), ([["big", "small"]], 256), ([["small", "big"]], 0)):
        other = run(groups, tile)
        assert torch.equal(other["big"], base["big"]) and torch.equal(other["small"], base["small"])
    A, Wp, b = small
    ref = torch.nn.functional.gelu(A.double() @ Wp.double().t() + b.double(), approximate="tanh")
    assert rel_l2(host(base["small"]), host(ref)) <= 4e-3
    A, Wp, b = big
    rows = torch.arange(0, 8192, 37, device="cuda")
    ref = torch.nn.functional.gelu(A[rows].double() @ Wp.double().t() + b.double(), approximate="tanh")
    assert rel_l2(host(base["big"][rows]), host(ref)) <= 4e-3


@pytest.mark.parametrize("epi", [1, 5])
def test_row_split_over_two_launches_gives_identical_bits(epi):
    """A many-row problem whose 256x256 tiles leave a partial round (here 8000 x 4608: 576 tiles on 256 compute units) runs its first
    rows as full rounds of 256x256 tiles and the rest, with the few-row problem, as 128x128 tiles in a second launch. Same bits as
    without the split and as either tile shape alone, and a float64 check of rows on both sides of the split."""
    g = torch.Generator(device="cuda").manual_seed(54 + epi)
    K, N = 128, 4608
    big_A = torch.randn((8000, K), device="cuda", generator=g).bfloat16()
    small_A = torch.randn((300, K), device="cuda", generator=g).bfloat16()
    Wp = [(0.1 * torch.randn((N, K), device="cuda", generator=g)).bfloat16() for _ in range(2)]
    bias = [0.1 * torch.randn(N, device="cuda", generator=g) for _ in range(2)]
    rq, rk = (1 + 0.1 * torch.randn(64, device="cuda", generator=g) for _ in range(2))

    def run(tile, split):
        outs = [torch.zeros((a.shape[0], N), device="cuda", dtype=torch.bfloat16) for a in (big_A, small_A)]
        ps = []
        for a, w, b, o in zip((big_A, small_A), Wp, bias, outs):
            p = L.GemmBf16Problem(A=a.data_ptr(), wpacked=w.data_ptr(), bias=b.data_ptr(), out=o.data_ptr(), M=a.shape[0], N=N, K=K)
            if epi == 5:
                p.rms_q, p.rms_k = rq.data_ptr(), rk.data_ptr()
            ps.append(p)
        try:
            L.call("sd3_tune", b"gemm_bf16_tile", tile)
            L.call("sd3_tune", b"gemm_bf16_row_split", split)
            launch(ps, epi, False)
        finally:
            L.call("sd3_tune", b"gemm_bf16_tile", 0)
            L.call("sd3_tune", b"gemm_bf16_row_split", 1)
        return outs

    base = run(0, 1)  # the split plan (the default choice at this shape)
    for tile, split in ((0, 0), (256, 1), (128, 1)):
        other = run(tile, split)
        assert torch.equal(other[0], base[0]) and torch.equal(other[1], base[1]), (tile, split)
    rows = torch.tensor([0, 255, 7167, 7168, 7169, 7999], device="cuda")  # the split falls between rows 7167 and 7168
    ref = big_A[rows].double() @ Wp[0].double().t() + bias[0].double()
    if epi == 1:
        ref = torch.nn.functional.gelu(ref, approximate="tanh")
    else:
        q, k, v = ref.view(len(rows), 3, N // 192, 64).unbind(1)
        nrm = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()  # noqa: E731
        ref = torch.stack([nrm(q, rq), nrm(k, rk), v], 1).reshape(len(rows), N)
    assert rel_l2(host(base[0][rows]), host(ref)) <= 4e-3


def test_row_split_with_two_many_row_problems_gives_identical_bits():
    """The fused q|k|v launch of a dual-attention block at batch 1: two problems of 4096 rows and one of 154 (2 x 288 + 18 tiles of
    256x256 on 256 compute units: two full rounds and a partial one). The split leaves the first problem whole, cuts the second behind
    its last row tile that fits the two rounds and sends the rest with the few-row problem through 128x128 tiles: same bits as the
    unsplit launch and as either tile shape alone, and a float64 check of rows on both sides of the cut."""
    g = torch.Generator(device="cuda").manual_seed(77)
    K, N, Ms = 128, 4608, (4096, 4096, 154)
    As = [torch.randn((m, K), device="cuda", generator=g).bfloat16() for m in Ms]
    Wp = [(0.1 * torch.randn((N, K), device="cuda", generator=g)).bfloat16() for _ in Ms]
    bias = [0.1 * torch.randn(N, device="cuda", generator=g) for _ in Ms]
    rq, rk = (1 + 0.1 * torch.randn(64, device="cuda", generator=g) for _ in range(2))

    def run(tile, split):
        outs = [torch.zeros((m, N), device="cuda", dtype=torch.bfloat16) for m in Ms]
        ps = []
        for a, w, b, o in zip(As, Wp, bias, outs):
            p = L.GemmBf16Problem(A=a.data_ptr(), wpacked=w.data_ptr(), bias=b.data_ptr(), out=o.data_ptr(), M=a.shape[0], N=N, K=K)
            p.rms_q, p.rms_k = rq.data_ptr(), rk.data_ptr()
            ps.append(p)
        try:
            L.call("sd3_tune", b"gemm_bf16_tile", tile)
            L.call("sd3_tune", b"gemm_bf16_row_split", split)
            launch(ps, 5, False)
        finally:
            L.call("sd3_tune", b"gemm_bf16_tile", 0)
            L.call("sd3_tune", b"gemm_bf16_row_split", 1)
        return outs

    base = run(0, 1)
    for tile, split in ((0, 0), (256, 1), (128, 1)):
        other = run(tile, split)
        assert all(torch.equal(a, b) for a, b in zip(other, base)), (tile, split)
    rows = torch.tensor([0, 3071, 3072, 3073, 4095], device="cuda")  # (512 - 288) // 18 = 12 row tiles of the second problem stay: the cut is at row 3072
    ref = As[1][rows].double() @ Wp[1].double().t() + bias[1].double()
    q, k, v = ref.view(len(rows), 3, N // 192, 64).unbind(1)
    nrm = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()  # noqa: E731
    ref = torch.stack([nrm(q, rq), nrm(k, rk), v], 1).reshape(len(rows), N)
    assert rel_l2(host(base[1][rows]), host(ref)) <= 4e-3


def test_grouped_gemm_argument_errors():
    none = C.c_void_p(0)
    p = L.GemmBf16Problem(M=4, N=192, K=64)
    arr = (L.GemmBf16Problem * 1)(p)
    lib = L.load()
    assert lib.sd3_gemm_bf16_grouped(C.cast(arr, C.c_void_p), 1, 0, 0, none) == 1   # null operands
    assert lib.sd3_gemm_bf16_grouped(C.cast(arr, C.c_void_p), 4, 0, 0, none) == 1   # too many problems
    assert lib.sd3_gemm_bf16_grouped(C.cast(arr, C.c_void_p), 1, 9, 0, none) == 1   # unknown epilogue
    assert lib.sd3_gemm_bf16_grouped(none, 1, 0, 0, none) == 1
