"""Per-operator parity on the MI355X: each HIP operator, called through the C ABI, against the CPU oracle on the same
seeded inputs (max abs error <= 1e-4), plus the edge cases the reference's unit scripts exercise."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as ol
from oracle_lib import fp
from gpu_util import M, dev, host, max_abs, F32_TOL

pytestmark = pytest.mark.gpu
rng = np.random.default_rng(99)


def randn(*s):
    return rng.standard_normal(s, dtype=np.float32)


@pytest.mark.parametrize("shape", [(2, 3, 4), (2, 5, 96), (3, 7, 1536), (1, 9, 2048), (2, 5, 2432), (1, 3, 3072), (2, 3, 4100), (1, 4, 130)])
def test_layernorm(shape):
    B, T, Cd = shape
    x = randn(*shape) * 2 + 0.3
    ref = np.empty_like(x)
    ol.oracle().orc_layernorm(fp(x), fp(ref), C.c_float(1e-6), B * T, Cd)
    y, mean, rstd = M.layer_norm(dev(x), None, None, 1e-6, True)
    assert max_abs(host(y), ref) <= F32_TOL
    assert max_abs(host(mean), x.mean(-1)) <= 1e-5
    assert max_abs(host(rstd), 1 / np.sqrt(x.var(-1) + 1e-6)) <= 1e-4
    w, b = randn(Cd), randn(Cd)
    (y2,) = M.layer_norm(dev(x), dev(w), dev(b), 1e-6, False)
    assert max_abs(host(y2), ref * w + b) <= F32_TOL


@pytest.mark.parametrize("B,T,NH,HS", [(2, 3, 4, 16), (1, 5, 24, 64), (2, 2, 2, 128), (1, 3, 3, 20)])
def test_rmsnorm_group(B, T, NH, HS):
    x, w = randn(B, T, NH * HS), 1 + 0.1 * randn(HS)
    ref = x.copy()
    ol.oracle().orc_rmsnorm_heads(fp(ref), fp(w), C.c_float(1e-6), B * T * NH, HS)
    assert max_abs(host(M.rms_norm_group(dev(x), dev(w), 1e-6, NH)), ref) <= F32_TOL
    (full,) = M.rms_norm(dev(x), dev(np.tile(w, NH)), 1e-6)
    ref2 = x.copy()
    ol.oracle().orc_rmsnorm_heads(fp(ref2), fp(np.tile(w, NH)), C.c_float(1e-6), B * T, NH * HS)
    assert max_abs(host(full), ref2) <= F32_TOL


def test_activations():
    x = np.concatenate([randn(5000) * 4, np.array([0, -30, 30, -88, 88, 1e-8], np.float32)])
    g, s = np.empty_like(x), np.empty_like(x)
    ol.oracle().orc_gelu_tanh(fp(x), fp(g), x.size)
    ol.oracle().orc_silu(fp(x), fp(s), x.size)
    assert max_abs(host(M.gelu_tanh(dev(x))), g) <= 1e-5
    assert max_abs(host(M.silu(dev(x))), s) <= 1e-5
    # the erf form, which the reference's extension calls `gelu` (modules.cpp:1795; module_tests/gelu.py:28 holds it to torch's
    # gelu(approximate="none")); 1e-5 separates it from the tanh form (up to ~5e-4 apart)
    e = np.empty_like(x)
    ol.oracle().orc_gelu(fp(x), fp(e), x.size)
    assert max_abs(host(M.gelu(dev(x))), e) <= 1e-5
    assert max_abs(e, torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="none").numpy()) <= 1e-6


@pytest.mark.parametrize("Mr,K,N", [(7, 40, 33), (1, 5, 3), (130, 320, 260), (64, 256, 128), (2, 1536, 64), (300, 64, 1536), (129, 17, 131)])
def test_linear_and_partial_linear(Mr, K, N):
    x, W, b = randn(Mr, K), randn(K, N) * 0.2, randn(N)
    ref = np.empty((Mr, N), np.float32)
    ol.oracle().orc_linear(fp(x), fp(W), fp(b), fp(ref), Mr, K, N)
    assert max_abs(host(M.linear(dev(x), dev(W), dev(b))), ref) <= F32_TOL
    if N >= 3:
        n0, n = N // 3, N // 3
        refp = np.empty((Mr, n), np.float32)
        ol.oracle().orc_partial_linear(fp(x), fp(W), fp(b), fp(refp), Mr, K, n, N, n0)
        assert max_abs(host(M.partial_linear(dev(x), dev(W), dev(b), n0, n)), refp) <= F32_TOL


@pytest.mark.parametrize("B,NH,T,L,HS", [(2, 3, 9, 13, 16), (1, 2, 130, 70, 64), (2, 2, 33, 257, 128), (1, 8, 128, 96, 64), (1, 1, 5, 5, 20)])
def test_multihead_attention(B, NH, T, L, HS):
    Q, K, V = randn(B, T, NH * HS), randn(B, L, NH * HS), randn(B, L, NH * HS)
    ref = np.empty_like(Q)
    ol.oracle().orc_attention(fp(Q), fp(K), fp(V), fp(ref), B, NH, T, L, HS)
    assert max_abs(host(M.mha(dev(Q), dev(K), dev(V), NH)), ref) <= F32_TOL


def test_attention_in_place_and_extreme_scores():
    from sd3_c_amd import lib as L_
    B, NH, T, HS = 1, 2, 70, 64
    Q, K, V = randn(B, T, NH * HS) * 6, randn(B, T, NH * HS) * 6, randn(B, T, NH * HS)  # logits of +-100: needs the max subtraction
    ref = np.empty_like(Q)
    ol.oracle().orc_attention(fp(Q), fp(K), fp(V), fp(ref), B, NH, T, T, HS)
    q, k, v = dev(Q), dev(K), dev(V)
    L_.call("sd3_multihead_attention", q.data_ptr(), k.data_ptr(), v.data_ptr(), q.data_ptr(), B, NH, T, T, HS, None)  # output aliases Q (modules.cpp:1430)
    assert np.isfinite(host(q)).all()
    assert max_abs(host(q), ref) <= F32_TOL


def test_embeddings():
    t = np.array([0.0, 0.37, 17.25, 512.5, 999.0], np.float32)
    ref = np.empty((5, 256), np.float32)
    ol.oracle().orc_timestep_embedding(fp(t), fp(ref), 5, 256)
    assert max_abs(host(M.sinusoidal_embedding(dev(t), 256)), ref) <= F32_TOL
    tab = np.empty((24 * 20, 64), np.float32)
    ol.oracle().orc_pos_embed_table(fp(tab), 64, 24, 20, 8)
    g = M.positional_embedding(64, 24, 20, 8)
    assert max_abs(host(g), tab) <= 1e-6
    sq = np.empty((24 * 24, 64), np.float32)
    ol.oracle().orc_pos_embed_table(fp(sq), 64, 24, 24, 8)
    crop = np.empty((10 * 7, 64), np.float32)
    ol.oracle().orc_pos_embed_crop(fp(sq), fp(crop), 24, 10, 7, 64)
    assert max_abs(host(M.crop_positional_embedding(dev(sq), 24, 10, 7, 64)), crop) == 0.0


@pytest.mark.parametrize("cfg", [(2, 4, 8, 8, 6, 2, 2, 0), (1, 3, 5, 7, 9, 3, 1, 1), (1, 2, 3, 8, 8, 3, 2, 1), (2, 16, 32, 16, 16, 2, 2, 0), (1, 1, 1, 5, 5, 5, 1, 2)])
def test_conv2d(cfg):
    B, Cin, Cout, ih, iw, k, s, p = cfg
    x, ker, b = randn(B, Cin, ih, iw), randn(Cout, Cin, k, k), randn(Cout)
    oh, ow = (ih + 2 * p - k) // s + 1, (iw + 2 * p - k) // s + 1
    ref = np.zeros((B, Cout, oh, ow), np.float32)
    ol.oracle().orc_conv2d(fp(x), fp(ref), fp(ker), fp(b), B, k, k, Cin, Cout, ih, iw, oh, ow, s, p)
    assert max_abs(host(M.conv2d(dev(x), dev(ker), dev(b), s, p)), ref) <= F32_TOL


def test_patch_embedding():
    B, Cin, H, W, Cd, p, pos_max, base = 2, 4, 16, 12, 64, 2, 24, 16
    lat, ker, b = randn(B, Cin, H, W), randn(Cd, Cin, p, p), randn(Cd)
    ref = np.empty((B, (H // p) * (W // p), Cd), np.float32)
    ol.oracle().orc_patch_embed(fp(lat), fp(ref), fp(ker), fp(b), B, H, W, Cin, Cd, p, pos_max, base)
    assert max_abs(host(M.patch_embedding(dev(lat), dev(ker), dev(b), Cd, p, pos_max, base)), ref) <= F32_TOL


@pytest.mark.parametrize("act,code", [("silu", 0), ("gelu_tanh", 1)])
def test_mlp(act, code):
    x, W1, b1, W2, b2 = randn(5, 48), randn(48, 100) * 0.2, randn(100), randn(100, 36) * 0.2, randn(36)
    h, ref = np.empty((5, 100), np.float32), np.empty((5, 36), np.float32)
    ol.oracle().orc_mlp(fp(x), fp(ref), fp(h), fp(W1), fp(b1), fp(W2), fp(b2), 5, 48, 100, 36, code)
    assert max_abs(host(M.mlp(dev(x), dev(W1), dev(b1), dev(W2), dev(b2), act)), ref) <= F32_TOL


def test_modulation_gating_concat_split():
    x, sh, sc = randn(2, 5, 24), randn(2, 24), randn(2, 24)
    ref = np.empty_like(x)
    ol.oracle().orc_modulate(fp(x), fp(ref), fp(sh), fp(sc), 2, 5, 24)
    assert max_abs(host(M.scale_and_shift(dev(x), dev(sh), dev(sc))), ref) <= 1e-6
    ol.oracle().orc_gate(fp(x), fp(ref), fp(sc), 2, 5, 24)
    assert max_abs(host(M.gating_mechanism(dev(x), dev(sc))), ref) <= 1e-6
    a, b = randn(2, 3, 8), randn(2, 5, 8)
    cat = M.concatenate_along_tokens(dev(a), dev(b))
    assert np.array_equal(host(cat), np.concatenate([a, b], 1))  # first argument's tokens come first
    s1, s2 = M.split_along_tokens(cat, 3)
    assert np.array_equal(host(s1), a) and np.array_equal(host(s2), b)


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 1 << 20])
def test_add(n):
    """modules.cpp:513-518; sizes around the vector width of the kernel; in place on the first operand as the block uses it."""
    a, b = randn(n) * 3, randn(n) * 1e-3
    ref = np.empty_like(a)
    ol.oracle().orc_add(fp(a), fp(b), fp(ref), C.c_long(n))
    assert np.array_equal(host(M.add(dev(a), dev(b))), ref)
    da = dev(a)
    from sd3_c_amd import lib as L_
    L_.call("sd3_add", da.data_ptr(), dev(b).data_ptr(), da.data_ptr(), n, None)
    assert np.array_equal(host(da), ref)


def test_empty_and_invalid_inputs():
    from sd3_c_amd import lib as L_
    e = torch.empty((0, 4, 8), device="cuda")
    assert M.layer_norm(e, None, None, 1e-6, False)[0].shape == (0, 4, 8)
    assert M.silu(torch.empty(0, device="cuda")).numel() == 0
    with pytest.raises(L_.Sd3Error):
        M.rms_norm_group(torch.zeros((1, 2, 10), device="cuda"), None, 1e-6, 3)  # 10 not divisible by 3
    with pytest.raises(L_.Sd3Error):
        M.mha(torch.zeros((1, 2, 2 * 200), device="cuda"), torch.zeros((1, 2, 400), device="cuda"), torch.zeros((1, 2, 400), device="cuda"), 2)  # head_dim 200
    with pytest.raises(L_.Sd3Error):
        L_.call("sd3_linear", None, None, None, None, 4, 4, 4, None)
    with pytest.raises(TypeError):
        M.silu(torch.zeros(4))  # host tensor
