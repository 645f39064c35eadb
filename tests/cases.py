"""Seeded test cases shared by the golden-vector generator and the parity tests.

Inputs and weights are regenerated from the seed (numpy Philox), so fixtures only store outputs."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from conftest import load_package  # noqa: E402

pkg = load_package()
from sd3_c_amd.config import DiTConfig  # noqa: E402
from sd3_c_amd.params import block_param_shapes, dit_param_shapes, synthetic_params_numpy  # noqa: E402

# name: (B, Tc, Tx, C, NH, mlp_expand, use_dual, use_qk_norm, discard_context)
BLOCK_CASES = {
    "block_dual_hs16": (2, 5, 12, 64, 4, 2, True, True, False),
    "block_dual_hs64": (1, 7, 16, 128, 2, 4, True, True, False),
    "block_plain_hs64": (2, 3, 9, 128, 2, 4, False, True, False),
    "block_discard_hs64": (1, 7, 16, 128, 2, 4, False, True, True),
    "block_noqknorm_hs32": (1, 4, 10, 64, 2, 2, True, False, False),
}

# name: (cfg, B, Tc, H, W)
DIT_CASES = {
    "dit_small": (DiTConfig(num_layers=3, dual_attention_layers=(0,), pooled_dim=48, captions_dim=40, in_channels=4, emb_dim=64, attn_heads=2,
                            mlp_expand=4, patch_size=2, pos_embed_max_size=24, base_height=16, use_qk_norm=True), 2, 7, 16, 12),
    "dit_hs64": (DiTConfig(num_layers=2, dual_attention_layers=(0,), pooled_dim=64, captions_dim=64, in_channels=16, emb_dim=128, attn_heads=2,
                           mlp_expand=4, patch_size=2, pos_embed_max_size=20, base_height=16, use_qk_norm=True), 2, 6, 16, 16),
}


# The configuration of the reference's own full-model check (module_tests/DiT.py:8-21): too slow for the CPU oracle
# inside a test run, so its golden output is only compared with the GPU fp32 path.
DIT_REFERENCE_TEST = ("dit_reference_test", DiTConfig(num_layers=3, dual_attention_layers=(0,), pooled_dim=2048, captions_dim=2048, in_channels=16,
                                                      emb_dim=256, attn_heads=2, mlp_expand=4, patch_size=2, pos_embed_max_size=96, base_height=64,
                                                      use_qk_norm=True), 2, 154, 64, 64)


def dit_reference_test_case():
    name, cfg, B, Tc, H, W = DIT_REFERENCE_TEST
    rng = np.random.Generator(np.random.Philox(_seed(name)))
    params = synthetic_params_numpy(dit_param_shapes(cfg), _seed(name) + 1, 0.05, 0.05)
    latent = rng.standard_normal((B, cfg.in_channels, H, W), dtype=np.float32)
    captions = rng.standard_normal((B, Tc, cfg.captions_dim), dtype=np.float32)
    pooled = rng.standard_normal((B, cfg.pooled_dim), dtype=np.float32)
    timesteps = rng.random((B,), dtype=np.float32)  # the reference draws timesteps from U[0,1) (module_tests/DiT.py:38)
    return dict(cfg=cfg, latent=latent, captions=captions, pooled=pooled, timesteps=timesteps, params=params)


def _seed(name):
    return 0x5D3 + sum(ord(ch) * (i + 1) for i, ch in enumerate(name))


def block_case(name, weight_std=0.1, bias_std=0.1):
    B, Tc, Tx, C, NH, me, dual, qk, disc = BLOCK_CASES[name]
    rng = np.random.Generator(np.random.Philox(_seed(name)))
    params = synthetic_params_numpy(block_param_shapes(C, me, dual, qk, disc, C // NH), _seed(name) + 1, weight_std, bias_std)
    y = rng.standard_normal((B, C), dtype=np.float32)
    c = rng.standard_normal((B, Tc, C), dtype=np.float32)
    x = rng.standard_normal((B, Tx, C), dtype=np.float32)
    return dict(y=y, c=c, x=x, params=params, NH=NH, mlp_expand=me, use_dual=dual, use_qk_norm=qk, discard_context=disc)


def dit_case(name, weight_std=0.1, bias_std=0.1):
    cfg, B, Tc, H, W = DIT_CASES[name]
    rng = np.random.Generator(np.random.Philox(_seed(name)))
    params = synthetic_params_numpy(dit_param_shapes(cfg), _seed(name) + 1, weight_std, bias_std)
    latent = rng.standard_normal((B, cfg.in_channels, H, W), dtype=np.float32)
    captions = rng.standard_normal((B, Tc, cfg.captions_dim), dtype=np.float32)
    pooled = rng.standard_normal((B, cfg.pooled_dim), dtype=np.float32)
    timesteps = (rng.random((B,), dtype=np.float32) * 1000.0).astype(np.float32)
    return dict(cfg=cfg, latent=latent, captions=captions, pooled=pooled, timesteps=timesteps, params=params)
