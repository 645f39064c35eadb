"""ctypes bindings of the CPU checkers (test infrastructure only).

`oracle()` loads oracle/libsd3_oracle.so, this repo's C restatement of the reference's forward path.
`reference()` loads oracle/_ref/libsd3_ref.so, the reference's own modules.cpp compiled in place, or
returns None where that library was not built (it needs the reference sources and never travels).
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libsd3_oracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libsd3_ref.so")

FP = C.POINTER(C.c_float)

BLOCK_FIELDS = [  # argument order of dit_block, modules.cpp:1344-1358
    ("c_ada_w", "context_ada_lnorm.linear.weight"), ("c_ada_b", "context_ada_lnorm.linear.bias"),
    ("c_qkv_w", "context_to_qkv.weight"), ("c_qkv_b", "context_to_qkv.bias"),
    ("c_rms_q", "context_rmsnorm_query.weight"), ("c_rms_k", "context_rmsnorm_key.weight"),
    ("c_out_w", "context_attn_Wout.weight"), ("c_out_b", "context_attn_Wout.bias"),
    ("c_mlp_w1", "context_mlp.lin1.weight"), ("c_mlp_b1", "context_mlp.lin1.bias"),
    ("c_mlp_w2", "context_mlp.lin2.weight"), ("c_mlp_b2", "context_mlp.lin2.bias"),
    ("x_ada_w", "latent_ada_lnorm.linear.weight"), ("x_ada_b", "latent_ada_lnorm.linear.bias"),
    ("x_qkv_w", "latent_to_qkv.weight"), ("x_qkv_b", "latent_to_qkv.bias"),
    ("x_rms_q", "latent_rmsnorm_query.weight"), ("x_rms_k", "latent_rmsnorm_key.weight"),
    ("x_out_w", "latent_attn_Wout.weight"), ("x_out_b", "latent_attn_Wout.bias"),
    ("x2_qkv_w", "latent_dual_to_qkv.weight"), ("x2_qkv_b", "latent_dual_to_qkv.bias"),
    ("x2_rms_q", "latent_dual_rmsnorm_query.weight"), ("x2_rms_k", "latent_dual_rmsnorm_key.weight"),
    ("x2_out_w", "latent_dual_attn_Wout.weight"), ("x2_out_b", "latent_dual_attn_Wout.bias"),
    ("x_mlp_w1", "latent_mlp.lin1.weight"), ("x_mlp_b1", "latent_mlp.lin1.bias"),
    ("x_mlp_w2", "latent_mlp.lin2.weight"), ("x_mlp_b2", "latent_mlp.lin2.bias"),
]
TOP_FIELDS = [
    ("t_w0", "timestep_mlp.0.weight"), ("t_b0", "timestep_mlp.0.bias"), ("t_w2", "timestep_mlp.2.weight"), ("t_b2", "timestep_mlp.2.bias"),
    ("p_w0", "pooled_mlp.0.weight"), ("p_b0", "pooled_mlp.0.bias"), ("p_w2", "pooled_mlp.2.weight"), ("p_b2", "pooled_mlp.2.bias"),
    ("cap_w", "captions_linear.weight"), ("cap_b", "captions_linear.bias"),
    ("patch_w", "to_patch.conv.weight"), ("patch_b", "to_patch.conv.bias"),
    ("ada_out_w", "ada_ln_out.linear.weight"), ("ada_out_b", "ada_ln_out.linear.bias"),
    ("out_w", "linear_out.weight"), ("out_b", "linear_out.bias"),
]


class BlockWeights(C.Structure):
    _fields_ = [(f, FP) for f, _ in BLOCK_FIELDS]


class DitWeights(C.Structure):
    _fields_ = [(f, FP) for f, _ in TOP_FIELDS] + [("blocks", C.POINTER(BlockWeights))]


def fp(a):
    if a is None:
        return C.cast(None, FP)
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(FP)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def ensure_oracle_built():
    """Compile the C restatement if it is not there (gcc only, a second or two)."""
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
    return ORACLE_SO


_oracle = None


def oracle():
    global _oracle
    if _oracle is None:
        _oracle = C.CDLL(ensure_oracle_built())
        _oracle.orc_dit_block.restype = C.c_int
        _oracle.orc_dit_forward.restype = C.c_int
    return _oracle


_ref = False


def reference():
    global _ref
    if _ref is False:
        _ref = C.CDLL(REF_SO) if os.path.exists(REF_SO) else None
    return _ref


def block_weights(params, prefix=""):
    bw = BlockWeights()
    for field, name in BLOCK_FIELDS:
        setattr(bw, field, fp(params.get(prefix + name)))
    return bw


# ------------------------------------------------------------------ oracle wrappers (numpy in / numpy out)
def orc_dit_block(y, c, x, params, NH, mlp_expand, use_dual, use_qk_norm, discard_context, prefix=""):
    """Returns (c_out, x_out); inputs untouched."""
    c, x, y = f32(c).copy(), f32(x).copy(), f32(y)
    B, Tc, Cd = c.shape
    Tx = x.shape[1]
    bw = block_weights(params, prefix)
    rc = oracle().orc_dit_block(fp(y), fp(c), fp(x), C.byref(bw), B, Tc, Tx, Cd, NH, mlp_expand, int(use_dual), int(use_qk_norm), int(discard_context))
    assert rc == 0
    return c, x


def orc_dit_forward(pooled, captions, latent, timesteps, params, cfg):
    pooled, captions, latent, timesteps = f32(pooled), f32(captions), f32(latent), f32(timesteps)
    B, Cin, H, W = latent.shape
    Tc = captions.shape[1]
    blocks = (BlockWeights * cfg.num_layers)(*[block_weights(params, f"transformer.{l}.") for l in range(cfg.num_layers)])
    dw = DitWeights()
    for field, name in TOP_FIELDS:
        setattr(dw, field, fp(params.get(name)))
    dw.blocks = C.cast(blocks, C.POINTER(BlockWeights))
    mask = (C.c_ubyte * cfg.num_layers)(*[1 if l in cfg.dual_attention_layers else 0 for l in range(cfg.num_layers)])
    out = np.empty_like(latent)
    rc = oracle().orc_dit_forward(fp(pooled), fp(captions), fp(latent), fp(timesteps), fp(out), C.byref(dw), mask, B, Tc, H, W, cfg.num_layers,
                                  cfg.pooled_dim, cfg.captions_dim, Cin, cfg.emb_dim, cfg.attn_heads, cfg.mlp_expand, cfg.patch_size,
                                  cfg.pos_embed_max_size, cfg.base_height, int(cfg.use_qk_norm))
    assert rc == 0
    return out


# ------------------------------------------------------------------ compiled-reference wrappers
def _param_arrays(params):
    names = list(params.keys())
    n = len(names)
    c_names = (C.c_char_p * n)(*[s.encode() for s in names])
    c_ptrs = (FP * n)(*[fp(params[s]) for s in names])
    c_numel = (C.c_longlong * n)(*[params[s].size for s in names])
    return n, c_names, c_ptrs, c_numel


def ref_dit_block(y, c, x, params, NH, mlp_expand, use_dual, use_qk_norm, discard_context):
    c, x, y = f32(c).copy(), f32(x).copy(), f32(y).copy()
    B, Tc, Cd = c.shape
    Tx = x.shape[1]
    n, names, ptrs, numel = _param_arrays(params)
    reference().ref_dit_block(fp(y), fp(c), fp(x), n, names, ptrs, numel, B, Tc, Tx, Cd, NH, mlp_expand, int(use_dual), int(use_qk_norm), int(discard_context))
    return c, x


def ref_dit_forward(pooled, captions, latent, timesteps, params, cfg):
    pooled, captions, latent, timesteps = f32(pooled).copy(), f32(captions).copy(), f32(latent).copy(), f32(timesteps).copy()
    B, Cin, H, W = latent.shape
    Tc = captions.shape[1]
    n, names, ptrs, numel = _param_arrays(params)
    dual = (C.c_int * max(1, len(cfg.dual_attention_layers)))(*cfg.dual_attention_layers)
    out = np.empty_like(latent)
    reference().ref_dit_forward(fp(pooled), fp(captions), fp(latent), fp(timesteps), fp(out), n, names, ptrs, numel, B, Tc, H, W, cfg.num_layers,
                                len(cfg.dual_attention_layers), dual, cfg.pooled_dim, cfg.captions_dim, Cin, cfg.emb_dim, cfg.attn_heads,
                                cfg.mlp_expand, cfg.patch_size, cfg.pos_embed_max_size, cfg.base_height, int(cfg.use_qk_norm))
    return out
