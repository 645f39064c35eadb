"""Bit-for-bit comparison of the C restatement with the reference's own modules.cpp compiled in place
(oracle/_ref). Skipped where that library is not built (it needs the reference's sources)."""
import ctypes as C

import numpy as np
import pytest

import cases
import oracle_lib as ol
from oracle_lib import fp

import os

# decided from the file's presence alone: the compiled reference is loaded only when one of these CPU tests actually runs
pytestmark = pytest.mark.skipif(not os.path.exists(ol.REF_SO), reason="oracle/_ref/libsd3_ref.so not built (needs /root/reference)")
rng = np.random.default_rng(7)


def randn(*s):
    return rng.standard_normal(s, dtype=np.float32)


def test_primitives_bit_exact():
    o, r = ol.oracle(), ol.reference()
    x = randn(6, 96) * 2 + 0.5
    a, b = np.empty_like(x), np.empty_like(x)
    o.orc_layernorm(fp(x), fp(a), C.c_float(1e-6), 6, 96)
    r.ref_layernorm(fp(x), fp(b), C.c_float(1e-6), 1, 6, 96)
    assert np.array_equal(a, b)
    w = randn(32)
    a, b = x.copy(), x.copy()
    o.orc_rmsnorm_heads(fp(a), fp(w), C.c_float(1e-6), 18, 32)
    r.ref_rmsnorm_group(fp(b), fp(b), fp(w), C.c_float(1e-6), 3, 1, 6, 96)
    assert np.array_equal(a, b)
    v = randn(4096) * 4
    for of, rf in ((o.orc_gelu_tanh, r.ref_gelu_tanh), (o.orc_silu, r.ref_silu), (o.orc_gelu, r.ref_gelu)):
        a, b = np.empty_like(v), np.empty_like(v)
        of(fp(v), fp(a), 4096)
        rf(fp(v), fp(b), C.c_longlong(4096))
        assert np.array_equal(a, b)
    Q, K, V = randn(2, 9, 48), randn(2, 13, 48), randn(2, 13, 48)
    a, b = np.empty_like(Q), np.empty_like(Q)
    o.orc_attention(fp(Q), fp(K), fp(V), fp(a), 2, 3, 9, 13, 16)
    r.ref_multihead_attention(fp(Q), fp(K), fp(V), fp(b), 2, 3, 9, 13, 16)
    assert np.array_equal(a, b)
    t = (rng.random(5, dtype=np.float32) * 1000).astype(np.float32)
    a, b = np.empty((5, 256), np.float32), np.empty((5, 256), np.float32)
    o.orc_timestep_embedding(fp(t), fp(a), 5, 256)
    r.ref_sinusoidal_embedding(fp(t), fp(b), 5, 256)
    assert np.array_equal(a, b)
    a, b = np.empty((20 * 20, 64), np.float32), np.empty((20 * 20, 64), np.float32)
    o.orc_pos_embed_table(fp(a), 64, 20, 20, 8)
    r.ref_positional_embedding2D(fp(b), 64, 20, 20, 8)
    assert np.array_equal(a, b)
    lat, ker, bias = randn(2, 4, 16, 12), randn(64, 4, 2, 2), randn(64)
    a, b = np.zeros((2, 64, 8, 6), np.float32), np.zeros((2, 64, 8, 6), np.float32)
    o.orc_conv2d(fp(lat), fp(a), fp(ker), fp(bias), 2, 2, 2, 4, 64, 16, 12, 8, 6, 2, 0)
    r.ref_conv2d(fp(lat), fp(b), fp(ker), fp(bias), 2, 2, 2, 4, 64, 16, 12, 8, 6, 2, 0)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("name", list(cases.BLOCK_CASES))
def test_block_bit_exact(name):
    k = cases.block_case(name)
    args = (k["y"], k["c"], k["x"], k["params"], k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    co, xo = ol.orc_dit_block(*args)
    cr, xr = ol.ref_dit_block(*args)
    assert np.array_equal(xo, xr)
    if not k["discard_context"]:
        assert np.array_equal(co, cr)


@pytest.mark.parametrize("name", list(cases.DIT_CASES))
def test_dit_forward_bit_exact(name):
    k = cases.dit_case(name)
    args = (k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
    assert np.array_equal(ol.orc_dit_forward(*args), ol.ref_dit_forward(*args))
