"""Pins the CPU oracle (oracle/sd3_oracle.c) without the reference: library routines, float64 closed
forms, invariants, a float64 numpy block written from the op list, and the committed golden vectors
(outputs of the reference's own modules.cpp). CPU only."""
import ctypes as C
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import cases
import oracle_lib as ol
from oracle_lib import fp

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_outputs.npz"))
rng = np.random.default_rng(1234)


def randn(*shape):
    return rng.standard_normal(shape, dtype=np.float32)


def test_layernorm_vs_torch_and_moments():
    x = randn(3, 5, 96) * 3 + 1
    y = np.empty_like(x)
    ol.oracle().orc_layernorm(fp(x), fp(y), C.c_float(1e-6), 15, 96)
    ref = F.layer_norm(torch.from_numpy(x).double(), (96,), None, None, 1e-6).numpy()
    assert np.abs(y - ref).max() < 2e-6
    assert np.abs(y.mean(-1)).max() < 1e-6 and np.abs(y.var(-1) - 1).max() < 1e-4


def test_rmsnorm_heads_vs_torch():
    x = randn(2, 4, 3, 64)
    w = 1 + 0.1 * randn(64)
    y = x.copy()
    ol.oracle().orc_rmsnorm_heads(fp(y), fp(w), C.c_float(1e-6), 2 * 4 * 3, 64)
    ref = F.rms_norm(torch.from_numpy(x).double(), (64,), torch.from_numpy(w).double(), 1e-6).numpy()
    assert np.abs(y - ref).max() < 2e-6


def test_activations_vs_torch():
    x = randn(1000) * 3
    g, s, e = np.empty_like(x), np.empty_like(x), np.empty_like(x)
    ol.oracle().orc_gelu_tanh(fp(x), fp(g), 1000)
    ol.oracle().orc_silu(fp(x), fp(s), 1000)
    ol.oracle().orc_gelu(fp(x), fp(e), 1000)
    xd = torch.from_numpy(x).double()
    assert np.abs(g - F.gelu(xd, approximate="tanh").numpy()).max() < 1e-6
    assert np.abs(s - F.silu(xd).numpy()).max() < 1e-6
    # the erf form is what the reference's own test compares with (module_tests/gelu.py:28); the two forms differ by up to ~5e-4,
    # so this bound separates them
    assert np.abs(e - F.gelu(xd, approximate="none").numpy()).max() < 1e-6
    assert np.abs(e - g).max() > 1e-4


def test_linear_and_partial_linear_vs_float64():
    x, W, b = randn(7, 40), randn(40, 33), randn(33)
    y = np.empty((7, 33), np.float32)
    ol.oracle().orc_linear(fp(x), fp(W), fp(b), fp(y), 7, 40, 33)
    ref = x.astype(np.float64) @ W.astype(np.float64) + b
    assert np.abs(y - ref).max() < 2e-5
    yp = np.empty((7, 11), np.float32)
    ol.oracle().orc_partial_linear(fp(x), fp(W), fp(b), fp(yp), 7, 40, 11, 33, 11)
    assert np.abs(yp - ref[:, 11:22]).max() < 2e-5
    # a transposed weight must fail this check
    assert np.abs(y[:, :7] - (x[:, :7].astype(np.float64) @ W[:7, :7].T)).max() > 1e-2


def _attn64(Q, K, V, NH):
    B, T, Cd = Q.shape
    L = K.shape[1]
    HS = Cd // NH
    q = Q.astype(np.float64).reshape(B, T, NH, HS).transpose(0, 2, 1, 3)
    k = K.astype(np.float64).reshape(B, L, NH, HS).transpose(0, 2, 1, 3)
    v = V.astype(np.float64).reshape(B, L, NH, HS).transpose(0, 2, 1, 3)
    s = q @ k.transpose(0, 1, 3, 2) / np.sqrt(HS)
    s = np.exp(s - s.max(-1, keepdims=True))
    p = s / s.sum(-1, keepdims=True)
    return (p @ v).transpose(0, 2, 1, 3).reshape(B, T, Cd)


def test_attention_vs_float64_and_invariants():
    B, NH, T, L, HS = 2, 3, 9, 13, 16
    Q, K, V = randn(B, T, NH * HS), randn(B, L, NH * HS), randn(B, L, NH * HS)
    out = np.empty_like(Q)
    ol.oracle().orc_attention(fp(Q), fp(K), fp(V), fp(out), B, NH, T, L, HS)
    assert np.abs(out - _attn64(Q, K, V, NH)).max() < 2e-6
    # torch's own SDPA on the head-split view (what module_tests/attention.py compares against)
    sd = F.scaled_dot_product_attention(*(torch.from_numpy(a).view(B, -1, NH, HS).transpose(1, 2) for a in (Q, K, V)))
    assert np.abs(out - sd.transpose(1, 2).reshape(B, T, NH * HS).numpy()).max() < 2e-6
    # permuting the keys/values together leaves the result unchanged; V of ones returns ones
    perm = rng.permutation(L)
    out2 = np.empty_like(Q)
    Kp, Vp = np.ascontiguousarray(K[:, perm]), np.ascontiguousarray(V[:, perm])
    ol.oracle().orc_attention(fp(Q), fp(Kp), fp(Vp), fp(out2), B, NH, T, L, HS)
    assert np.abs(out - out2).max() < 2e-6
    ones = np.ones_like(V)
    ol.oracle().orc_attention(fp(Q), fp(K), fp(ones), fp(out2), B, NH, T, L, HS)
    assert np.abs(out2 - 1).max() < 1e-6
    # in place on Q, as the block calls it
    Qc = Q.copy()
    ol.oracle().orc_attention(fp(Qc), fp(K), fp(V), fp(Qc), B, NH, T, L, HS)
    assert np.array_equal(Qc, out)


def test_timestep_embedding_closed_form():
    t = np.array([0.0, 0.5, 17.25, 999.0], np.float32)
    out = np.empty((4, 256), np.float32)
    ol.oracle().orc_timestep_embedding(fp(t), fp(out), 4, 256)
    i = np.arange(128, dtype=np.float64)
    ang = t[:, None].astype(np.float64) * 10000.0 ** (-i / 128)
    assert np.abs(out[:, :128] - np.cos(ang)).max() < 2e-4  # float32 angle of up to 999 rad
    assert np.abs(out[:, 128:] - np.sin(ang)).max() < 2e-4
    assert np.abs(out[:2, :128] - np.cos(ang[:2])).max() < 1e-6


def test_pos_embed_closed_form_and_axis_order():
    Cd, size, base = 32, 12, 4
    tab = np.empty((size, size, Cd), np.float32)
    ol.oracle().orc_pos_embed_table(fp(tab), Cd, size, size, base)
    i = np.arange(Cd // 4, dtype=np.float64)
    freq = 1.0 / 10000.0 ** (4 * i / Cd)
    pos = np.arange(size, dtype=np.float64) * base / size
    # stored [a][b]: first two quarters encode the FAST index b, last two the slow index a
    exp = np.empty((size, size, Cd))
    exp[..., 0:8] = np.sin(pos[None, :, None] * freq)
    exp[..., 8:16] = np.cos(pos[None, :, None] * freq)
    exp[..., 16:24] = np.sin(pos[:, None, None] * freq)
    exp[..., 24:32] = np.cos(pos[:, None, None] * freq)
    assert np.abs(tab - exp).max() < 1e-7
    assert np.abs(tab - exp.transpose(1, 0, 2)).max() > 0.1  # the other axis order is a different table
    h, w = 6, 4
    crop = np.empty((h * w, Cd), np.float32)
    ol.oracle().orc_pos_embed_crop(fp(tab), fp(crop), size, h, w, Cd)
    assert np.array_equal(crop.reshape(h, w, Cd), tab[3:9, 4:8])


def test_conv2d_vs_torch():
    for (B, Cin, Cout, ih, iw, k, s, p) in [(2, 4, 8, 8, 6, 2, 2, 0), (1, 3, 5, 7, 9, 3, 1, 1), (1, 2, 3, 8, 8, 3, 2, 1)]:
        x, ker, b = randn(B, Cin, ih, iw), randn(Cout, Cin, k, k), randn(Cout)
        oh, ow = (ih + 2 * p - k) // s + 1, (iw + 2 * p - k) // s + 1
        out = np.zeros((B, Cout, oh, ow), np.float32)
        ol.oracle().orc_conv2d(fp(x), fp(out), fp(ker), fp(b), B, k, k, Cin, Cout, ih, iw, oh, ow, s, p)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(ker).double(), torch.from_numpy(b).double(), stride=s, padding=p).numpy()
        assert np.abs(out - ref).max() < 1e-5


def test_modulate_and_gate():
    x, sh, sc = randn(2, 3, 8), randn(2, 8), randn(2, 8)
    out = np.empty_like(x)
    ol.oracle().orc_modulate(fp(x), fp(out), fp(sh), fp(sc), 2, 3, 8)
    assert np.abs(out - (x * (1 + sc[:, None]) + sh[:, None])).max() < 1e-6
    ol.oracle().orc_gate(fp(x), fp(out), fp(sc), 2, 3, 8)
    assert np.abs(out - x * sc[:, None]).max() < 1e-6


# ---------------------------------------------------------------- float64 block written from the op list
def block64(y, c, x, P, NH, dual, qk, disc):
    f = lambda n: P[n].astype(np.float64)  # noqa: E731
    y, c, x = y.astype(np.float64), c.astype(np.float64), x.astype(np.float64)
    Cd = x.shape[-1]
    HS = Cd // NH

    def ln(a):
        m = a.mean(-1, keepdims=True)
        return (a - m) / np.sqrt(((a - m) ** 2).mean(-1, keepdims=True) + 1e-6)

    def rms(a, w):
        s = a.shape
        a = a.reshape(*s[:-1], NH, HS)
        return (a / np.sqrt((a ** 2).mean(-1, keepdims=True) + 1e-6) * w).reshape(s)

    def gelu(a):
        return 0.5 * a * (1 + np.tanh(np.sqrt(2 / np.pi) * (a + 0.044715 * a ** 3)))

    def qkv(a, pre):
        q, k, v = np.split(a @ f(pre + "to_qkv.weight") + f(pre + "to_qkv.bias"), 3, -1)
        if qk:
            q, k = rms(q, f(pre + "rmsnorm_query.weight")), rms(k, f(pre + "rmsnorm_key.weight"))
        return q, k, v

    cm = np.split(y @ f("context_ada_lnorm.linear.weight") + f("context_ada_lnorm.linear.bias"), 2 if disc else 6, -1)
    xm = np.split(y @ f("latent_ada_lnorm.linear.weight") + f("latent_ada_lnorm.linear.bias"), 9 if dual else 6, -1)
    cm = [m[:, None] for m in cm]
    xm = [m[:, None] for m in xm]
    c_shift, c_scale = (cm[1], cm[0]) if disc else (cm[0], cm[1])
    qc, kc, vc = qkv(ln(c) * (1 + c_scale) + c_shift, "context_")
    xn = ln(x)
    qx, kx, vx = qkv(xn * (1 + xm[1]) + xm[0], "latent_")
    Tc = c.shape[1]
    att = _attn64(np.concatenate([qc, qx], 1), np.concatenate([kc, kx], 1), np.concatenate([vc, vx], 1), NH)
    if not disc:
        c = c + cm[2] * (att[:, :Tc] @ f("context_attn_Wout.weight") + f("context_attn_Wout.bias"))
    x1 = x + xm[2] * (att[:, Tc:] @ f("latent_attn_Wout.weight") + f("latent_attn_Wout.bias"))
    if dual:
        q2, k2, v2 = qkv(xn * (1 + xm[7]) + xm[6], "latent_dual_")
        x1 = x1 + xm[8] * (_attn64(q2, k2, v2, NH) @ f("latent_dual_attn_Wout.weight") + f("latent_dual_attn_Wout.bias"))
    x = x1
    h = gelu((ln(x) * (1 + xm[4]) + xm[3]) @ f("latent_mlp.lin1.weight") + f("latent_mlp.lin1.bias"))
    x = x + xm[5] * (h @ f("latent_mlp.lin2.weight") + f("latent_mlp.lin2.bias"))
    if not disc:
        h = gelu((ln(c) * (1 + cm[4]) + cm[3]) @ f("context_mlp.lin1.weight") + f("context_mlp.lin1.bias"))
        c = c + cm[5] * (h @ f("context_mlp.lin2.weight") + f("context_mlp.lin2.bias"))
    return c, x


# ---------------------------------------------------------------- float64 forward written from the op list (modules.cpp:1660-1752)
def dit64(pooled, captions, latent, timesteps, P, cfg, progress=None):
    f = lambda n: P[n].astype(np.float64)  # noqa: E731
    silu = lambda a: a / (1 + np.exp(-a))  # noqa: E731
    pooled, captions, latent, t = (a.astype(np.float64) for a in (pooled, captions, latent, timesteps))
    B, Cin, H, W = latent.shape
    C, p = cfg.emb_dim, cfg.patch_size
    Hp, Wp = H // p, W // p
    # conditioning vector: [cos | sin] of t * 10000^(-i/128), two MLPs, sum, silu (modules.cpp:920-944, 1663-1675)
    freq = np.exp(-np.log(10000.0) * 2 * np.arange(128) / 256)
    temb = np.concatenate([np.cos(t[:, None] * freq), np.sin(t[:, None] * freq)], 1)
    mlp = lambda a, n: silu(a @ f(n + ".0.weight") + f(n + ".0.bias")) @ f(n + ".2.weight") + f(n + ".2.bias")  # noqa: E731
    y = silu(mlp(temb, "timestep_mlp") + mlp(pooled, "pooled_mlp"))
    c = captions @ f("captions_linear.weight") + f("captions_linear.bias")
    # patch embedding: p x p / stride p convolution, tokens in row-major patch order (modules.cpp:1037-1062, 1093-1117)
    patches = latent.reshape(B, Cin, Hp, p, Wp, p).transpose(0, 2, 4, 1, 3, 5).reshape(B, Hp * Wp, Cin * p * p)
    x = patches @ f("to_patch.conv.weight").reshape(C, Cin * p * p).T + f("to_patch.conv.bias")
    # position table (modules.cpp:946-995): entry [a][b] of the max x max table uses a for the "width" angle and b for the "height"
    # angle, [sin h | cos h | sin w | cos w]; the centre crop reads it as [row][col]
    mx, base = cfg.pos_embed_max_size, cfg.base_height // p
    fr = 1.0 / np.power(10000.0, 4.0 * np.arange(C // 4) / C)
    oh, ow = (mx - Hp) // 2, (mx - Wp) // 2
    pw = (np.arange(Hp) + oh)[:, None] * base / mx      # rows of the crop index the table's first ("width") axis
    ph = (np.arange(Wp) + ow)[:, None] * base / mx
    e_h = np.concatenate([np.sin(ph * fr), np.cos(ph * fr)], 1)   # (Wp, C/2)
    e_w = np.concatenate([np.sin(pw * fr), np.cos(pw * fr)], 1)   # (Hp, C/2)
    pos = np.concatenate([np.broadcast_to(e_h[None], (Hp, Wp, C // 2)), np.broadcast_to(e_w[:, None], (Hp, Wp, C // 2))], 2).reshape(Hp * Wp, C)
    x = x + pos.astype(np.float32).astype(np.float64)             # (the reference stores the table as float)
    for l in range(cfg.num_layers):
        pre = f"transformer.{l}."
        Pl = {n[len(pre):]: v for n, v in P.items() if n.startswith(pre)}
        c, x = block64(y, c, x, Pl, cfg.attn_heads, l in cfg.dual_attention_layers, cfg.use_qk_norm, l == cfg.num_layers - 1)
        if progress:
            progress(l)
    m = x.mean(-1, keepdims=True)
    xh = (x - m) / np.sqrt(((x - m) ** 2).mean(-1, keepdims=True) + 1e-5)
    scale, shift = np.split(y @ f("ada_ln_out.linear.weight") + f("ada_ln_out.linear.bias"), 2, -1)   # chunk 0 = scale, chunk 1 = shift
    tok = (xh * (1 + scale[:, None]) + shift[:, None]) @ f("linear_out.weight") + f("linear_out.bias")
    # tokens -> pixels: channel index of a token is (ph * p + pw) * C_in + ch (modules.cpp:1730-1752)
    return tok.reshape(B, Hp, Wp, p, p, Cin).transpose(0, 5, 1, 3, 2, 4).reshape(B, Cin, H, W)


@pytest.mark.parametrize("name", list(cases.DIT_CASES))
def test_float64_forward_written_from_the_op_list_vs_oracle_and_golden(name):
    """Pins dit64 (used by the GPU tests at sizes the CPU oracle cannot reach in a test run) to the oracle and to the compiled
    reference's output, conventions included: [cos|sin] order, position-table axes and crop, scale/shift swap, un-patchify order."""
    k = cases.dit_case(name)
    out64 = dit64(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
    out = ol.orc_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
    scale = max(1.0, np.abs(out64).max())
    assert np.abs(out - out64).max() < 2e-4 * scale
    assert np.abs(GOLDEN[name + ".out"] - out64).max() < 2e-4 * scale


@pytest.mark.parametrize("name", list(cases.BLOCK_CASES))
def test_block_vs_float64_numpy_and_golden(name):
    k = cases.block_case(name)
    c, x = ol.orc_dit_block(k["y"], k["c"], k["x"], k["params"], k["NH"], k["mlp_expand"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    c64, x64 = block64(k["y"], k["c"], k["x"], k["params"], k["NH"], k["use_dual"], k["use_qk_norm"], k["discard_context"])
    assert np.abs(x - x64).max() < 2e-4 * max(1, np.abs(x64).max())
    assert np.abs(c - c64).max() < 2e-4 * max(1, np.abs(c64).max())
    # the compiled reference's output on the same inputs
    assert np.abs(x - GOLDEN[name + ".x"]).max() <= 1e-5
    assert np.abs(c - GOLDEN[name + ".c"]).max() <= 1e-5
    if k["discard_context"]:
        assert np.array_equal(c, k["c"])  # the last block leaves the context stream untouched (modules.cpp:1457)


def test_block_zero_gates_is_identity():
    k = cases.block_case("block_dual_hs64")
    P = dict(k["params"])
    Cd = k["x"].shape[-1]
    for pre, nch in (("context_", 6), ("latent_", 9)):
        w, b = P[pre + "ada_lnorm.linear.weight"].copy(), P[pre + "ada_lnorm.linear.bias"].copy()
        for g in (2, 5, 8):
            if g < nch:
                w[:, g * Cd:(g + 1) * Cd] = 0
                b[g * Cd:(g + 1) * Cd] = 0
        P[pre + "ada_lnorm.linear.weight"], P[pre + "ada_lnorm.linear.bias"] = w, b
    c, x = ol.orc_dit_block(k["y"], k["c"], k["x"], P, k["NH"], k["mlp_expand"], True, True, False)
    assert np.array_equal(c, k["c"]) and np.array_equal(x, k["x"])


@pytest.mark.parametrize("name", list(cases.DIT_CASES))
def test_dit_forward_vs_golden(name):
    k = cases.dit_case(name)
    out = ol.orc_dit_forward(k["pooled"], k["captions"], k["latent"], k["timesteps"], k["params"], k["cfg"])
    assert out.shape == k["latent"].shape
    assert np.abs(out - GOLDEN[name + ".out"]).max() <= 1e-5
