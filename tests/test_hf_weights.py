"""CPU only: Hugging Face state-dict names <-> the reference's parameter names and layout (sd3.c_amd/hf_weights.py).
The correspondence follows the reference's own copy loop (module_tests/modules.py:532-612); these tests pin the layout
rules (row thirds of the fused q|k|v weights, transposition to (C_in, C_out), which blocks lack which entries) with
hand-built tensors, not with the converter's own inverse alone."""
import numpy as np
import pytest

from conftest import load_package

load_package()
from sd3_c_amd import hf_weights as H  # noqa: E402
from sd3_c_amd.config import DiTConfig, sd35_medium  # noqa: E402
from sd3_c_amd.params import dit_param_shapes, synthetic_params_numpy  # noqa: E402


def tiny_cfg():
    return DiTConfig(num_layers=3, dual_attention_layers=(0,), in_channels=4, emb_dim=32, pooled_dim=24, captions_dim=40, patch_size=2,
                     attn_heads=2, mlp_expand=4, pos_embed_max_size=8, base_height=8, use_qk_norm=True)


def test_round_trip_through_hf_names_is_the_identity():
    cfg = tiny_cfg()
    params = synthetic_params_numpy(dit_param_shapes(cfg), seed=3, bias_std=0.1)
    hf = H.to_hf_state_dict(params, cfg)
    back = H.convert_state_dict(hf, cfg)
    assert list(back.keys()) == list(params.keys())
    for k in params:
        assert back[k].dtype == np.float32 and back[k].flags["C_CONTIGUOUS"]
        assert np.array_equal(back[k], params[k]), k


def test_layout_rules_with_hand_built_tensors():
    cfg = tiny_cfg()
    C = cfg.emb_dim
    params = synthetic_params_numpy(dit_param_shapes(cfg), seed=4)
    hf = H.to_hf_state_dict(params, cfg)
    # nn.Linear layout on the Hugging Face side: (C_out, C_in); q, k, v are separate layers there
    q = np.arange(C * C, dtype=np.float32).reshape(C, C)          # to_q.weight[o, i] = o*C + i
    k, v = q + 10000, q + 20000
    hf["transformer_blocks.1.attn.to_q.weight"], hf["transformer_blocks.1.attn.to_k.weight"], hf["transformer_blocks.1.attn.to_v.weight"] = q, k, v
    hf["transformer_blocks.1.attn.to_q.bias"] = np.full(C, 1, np.float32)
    hf["transformer_blocks.1.attn.to_k.bias"] = np.full(C, 2, np.float32)
    hf["transformer_blocks.1.attn.to_v.bias"] = np.full(C, 3, np.float32)
    w1 = np.arange(4 * C * C, dtype=np.float32).reshape(4 * C, C)  # ff.net.0.proj.weight (4C, C)
    hf["transformer_blocks.1.ff.net.0.proj.weight"] = w1
    conv = np.arange(C * cfg.in_channels * 4, dtype=np.float32).reshape(C, cfg.in_channels, 2, 2)
    hf["pos_embed.proj.weight"] = conv
    hf["transformer_blocks.0.attn2.norm_q.weight"] = np.full(C // cfg.attn_heads, 7, np.float32)
    hf["transformer_blocks.2.attn.norm_added_k.weight"] = np.full(C // cfg.attn_heads, 9, np.float32)
    out = H.convert_state_dict(hf, cfg)
    W = out["transformer.1.latent_to_qkv.weight"]                  # reference layout (C_in, 3C): y = x @ W
    assert W.shape == (C, 3 * C)
    assert W[5, 7] == q[7, 5] and W[5, C + 7] == k[7, 5] and W[5, 2 * C + 7] == v[7, 5]
    assert np.array_equal(out["transformer.1.latent_to_qkv.bias"], np.repeat([1, 2, 3], C).astype(np.float32))
    assert np.array_equal(out["transformer.1.latent_mlp.lin1.weight"], w1.T)
    assert np.array_equal(out["to_patch.conv.weight"], conv)       # the convolution weight is not transposed
    assert np.all(out["transformer.0.latent_dual_rmsnorm_query.weight"] == 7)
    assert np.all(out["transformer.2.context_rmsnorm_key.weight"] == 9)
    # a linear layer applied both ways gives the same numbers
    x = np.random.default_rng(0).standard_normal((3, C)).astype(np.float32)
    hf_y = np.concatenate([x @ q.T + 1, x @ k.T + 2, x @ v.T + 3], axis=1)
    np.testing.assert_allclose(x @ W + out["transformer.1.latent_to_qkv.bias"], hf_y, rtol=1e-6)


def test_which_blocks_have_which_entries():
    cfg = tiny_cfg()
    plan = H.name_plan(cfg)
    hf_names = {n for _, names in plan.values() for n in names}
    last = cfg.num_layers - 1
    assert f"transformer_blocks.{last}.attn.to_add_out.weight" not in hf_names      # the last block drops its context output
    assert f"transformer_blocks.{last}.ff_context.net.2.weight" not in hf_names
    assert f"transformer_blocks.{last}.attn.add_q_proj.weight" in hf_names          # ... but still projects the context to q,k,v
    assert "transformer_blocks.0.attn2.to_q.weight" in hf_names and "transformer_blocks.1.attn2.to_q.weight" not in hf_names
    shapes = dit_param_shapes(cfg)
    assert shapes[f"transformer.{last}.context_ada_lnorm.linear.weight"] == (cfg.emb_dim, 2 * cfg.emb_dim)
    assert shapes["transformer.0.latent_ada_lnorm.linear.weight"] == (cfg.emb_dim, 9 * cfg.emb_dim)


def test_sd35_medium_plan_covers_the_inventory_and_counts_parameters():
    cfg = sd35_medium()
    plan, shapes = H.name_plan(cfg), dit_param_shapes(cfg)
    assert list(plan.keys()) == list(shapes.keys())
    n = sum(int(np.prod(s)) for s in shapes.values())
    assert 2.2e9 < n < 2.3e9   # 2.24 B parameters (the position table is a buffer, not a parameter)
    assert len({x for _, names in plan.values() for x in names}) == sum(len(names) for _, names in plan.values())  # no HF entry used twice


def test_errors_name_the_problem():
    cfg = tiny_cfg()
    hf = H.to_hf_state_dict(synthetic_params_numpy(dit_param_shapes(cfg), seed=5), cfg)
    missing = dict(hf)
    del missing["transformer_blocks.2.norm1_context.linear.bias"]
    with pytest.raises(KeyError, match="norm1_context.linear.bias"):
        H.convert_state_dict(missing, cfg)
    extra = dict(hf)
    extra["transformer_blocks.2.ff_context.net.2.weight"] = np.zeros((2, 2), np.float32)
    with pytest.raises(ValueError, match="map to nothing"):
        H.convert_state_dict(extra, cfg)
    assert "transformer.0.latent_to_qkv.weight" in H.convert_state_dict(extra, cfg, strict=False)
    wrong = dict(hf)
    wrong["proj_out.weight"] = np.zeros((3, 3), np.float32)
    with pytest.raises(ValueError, match="linear_out.weight"):
        H.convert_state_dict(wrong, cfg)
    ok = dict(hf)
    ok["pos_embed.pos_embed"] = np.zeros((1, 64, cfg.emb_dim), np.float32)   # the stored position table is ignored
    H.convert_state_dict(ok, cfg)


def test_safetensors_files_sharded_and_in_half_precision(tmp_path):
    torch = pytest.importorskip("torch")
    st = pytest.importorskip("safetensors.torch")
    cfg = tiny_cfg()
    params = synthetic_params_numpy(dit_param_shapes(cfg), seed=6, bias_std=0.1)
    hf = {k: torch.from_numpy(v).to(torch.bfloat16) for k, v in H.to_hf_state_dict(params, cfg).items()}
    keys = sorted(hf)
    half = len(keys) // 2
    st.save_file({k: hf[k] for k in keys[:half]}, str(tmp_path / "diffusion_pytorch_model-00001-of-00002.safetensors"))
    st.save_file({k: hf[k] for k in keys[half:]}, str(tmp_path / "diffusion_pytorch_model-00002-of-00002.safetensors"))
    got = H.load_safetensors(str(tmp_path), cfg)
    for k, v in params.items():
        want = torch.from_numpy(v).to(torch.bfloat16).float().numpy()
        assert np.array_equal(got[k], want), k
