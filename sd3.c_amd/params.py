"""Parameter inventory in the reference's layout, and synthetic initialisation.

Names are the PyTorch `named_parameters()` names of the reference's model (module_tests/modules.py:205-425)
as the C++ looks them up (modules.cpp:1558-1575, 1665-1728). Every 2-D weight is stored transposed,
`(C_in, C_out)` row-major, exactly as the reference's drivers pass it (module_tests/DiT.py:26-31); the
patch convolution weight stays `(C, C_in, p, p)`.
"""
from collections import OrderedDict

import numpy as np

from .config import DiTConfig


def block_param_shapes(C: int, mlp_expand: int, use_dual: bool, use_qk_norm: bool, discard_context: bool, head_dim: int) -> "OrderedDict[str, tuple]":
    s = OrderedDict()
    cch = 2 if discard_context else 6
    xch = 9 if use_dual else 6
    s["context_ada_lnorm.linear.weight"] = (C, cch * C)
    s["context_ada_lnorm.linear.bias"] = (cch * C,)
    s["context_to_qkv.weight"] = (C, 3 * C)
    s["context_to_qkv.bias"] = (3 * C,)
    if use_qk_norm:
        s["context_rmsnorm_key.weight"] = (head_dim,)
        s["context_rmsnorm_query.weight"] = (head_dim,)
    if not discard_context:
        s["context_attn_Wout.weight"] = (C, C)
        s["context_attn_Wout.bias"] = (C,)
        s["context_mlp.lin1.weight"] = (C, mlp_expand * C)
        s["context_mlp.lin1.bias"] = (mlp_expand * C,)
        s["context_mlp.lin2.weight"] = (mlp_expand * C, C)
        s["context_mlp.lin2.bias"] = (C,)
    s["latent_ada_lnorm.linear.weight"] = (C, xch * C)
    s["latent_ada_lnorm.linear.bias"] = (xch * C,)
    s["latent_to_qkv.weight"] = (C, 3 * C)
    s["latent_to_qkv.bias"] = (3 * C,)
    if use_qk_norm:
        s["latent_rmsnorm_key.weight"] = (head_dim,)
        s["latent_rmsnorm_query.weight"] = (head_dim,)
    s["latent_attn_Wout.weight"] = (C, C)
    s["latent_attn_Wout.bias"] = (C,)
    s["latent_mlp.lin1.weight"] = (C, mlp_expand * C)
    s["latent_mlp.lin1.bias"] = (mlp_expand * C,)
    s["latent_mlp.lin2.weight"] = (mlp_expand * C, C)
    s["latent_mlp.lin2.bias"] = (C,)
    if use_dual:
        s["latent_dual_to_qkv.weight"] = (C, 3 * C)
        s["latent_dual_to_qkv.bias"] = (3 * C,)
        if use_qk_norm:
            s["latent_dual_rmsnorm_key.weight"] = (head_dim,)
            s["latent_dual_rmsnorm_query.weight"] = (head_dim,)
        s["latent_dual_attn_Wout.weight"] = (C, C)
        s["latent_dual_attn_Wout.bias"] = (C,)
    return s


def dit_param_shapes(cfg: DiTConfig) -> "OrderedDict[str, tuple]":
    C, p = cfg.emb_dim, cfg.patch_size
    s = OrderedDict()
    s["timestep_mlp.0.weight"] = (256, C)
    s["timestep_mlp.0.bias"] = (C,)
    s["timestep_mlp.2.weight"] = (C, C)
    s["timestep_mlp.2.bias"] = (C,)
    s["pooled_mlp.0.weight"] = (cfg.pooled_dim, C)
    s["pooled_mlp.0.bias"] = (C,)
    s["pooled_mlp.2.weight"] = (C, C)
    s["pooled_mlp.2.bias"] = (C,)
    s["captions_linear.weight"] = (cfg.captions_dim, C)
    s["captions_linear.bias"] = (C,)
    s["to_patch.conv.weight"] = (C, cfg.in_channels, p, p)
    s["to_patch.conv.bias"] = (C,)
    for l in range(cfg.num_layers):
        last = l == cfg.num_layers - 1
        blk = block_param_shapes(C, cfg.mlp_expand, l in cfg.dual_attention_layers, cfg.use_qk_norm, last, cfg.head_dim)
        for k, v in blk.items():
            s[f"transformer.{l}.{k}"] = v
    s["ada_ln_out.linear.weight"] = (C, 2 * C)
    s["ada_ln_out.linear.bias"] = (2 * C,)
    s["linear_out.weight"] = (C, p * p * cfg.in_channels)
    s["linear_out.bias"] = (p * p * cfg.in_channels,)
    return s


def synthetic_params_numpy(shapes, seed: int, weight_std: float = 0.02, bias_std: float = 0.0, rms_jitter: float = 0.02):
    """Seeded fp32 parameters: matrices ~N(0, weight_std), biases ~N(0, bias_std) (0 -> zeros),
    per-head RMSNorm weights 1 + N(0, rms_jitter). One Philox stream per call, names drawn in dict order."""
    rng = np.random.Generator(np.random.Philox(seed))
    out = OrderedDict()
    for name, shape in shapes.items():
        if "rmsnorm" in name:
            a = 1.0 + rms_jitter * rng.standard_normal(shape, dtype=np.float32)
        elif name.endswith(".bias"):
            a = bias_std * rng.standard_normal(shape, dtype=np.float32) if bias_std else np.zeros(shape, np.float32)
        else:
            a = weight_std * rng.standard_normal(shape, dtype=np.float32)
        out[name] = np.ascontiguousarray(a, dtype=np.float32)
    return out
