"""Real weights: Hugging Face `SD3Transformer2DModel` state-dict names (stabilityai/stable-diffusion-3.5-medium,
`transformer/diffusion_pytorch_model*.safetensors`) <-> the reference's parameter names and layout.

The reference spells the correspondence out where it copies its own model into the Hugging Face one to compare
them (module_tests/modules.py:532-612): `attn.to_q/to_k/to_v` are the row thirds of `latent_to_qkv`,
`attn.add_{q,k,v}_proj` those of `context_to_qkv`, `attn2.*` the `latent_dual_*` layers, `norm1(.context).linear` the
`*_ada_lnorm.linear` layers, `ff(.context).net.0.proj / net.2` the MLPs, plus the embedders and the output layers.
The per-head RMSNorm weights (`attn.norm_q`, `attn.norm_k`, `attn.norm_added_q`, `attn.norm_added_k`, `attn2.norm_q`,
`attn2.norm_k`) are not in that listing (it runs without qk-norm); their targets are the `*_rmsnorm_query/key` vectors of
module_tests/modules.py:224-247. Chunk orders agree on both sides (shift, scale, gate, ... for the 6- and 9-chunk
modulations; scale, shift for the two 2-chunk ones), so rows are copied without permutation.

Layout rule of the reference's drivers (module_tests/DiT.py:26-31): every 2-D parameter is handed over transposed,
`(C_in, C_out)` row-major; everything else as it is. Hugging Face stores `nn.Linear.weight` as `(C_out, C_in)`.

Nothing here touches the GPU; arrays are numpy float32 on return.
"""
import json
import os
from collections import OrderedDict

import numpy as np

from .config import DiTConfig
from .params import dit_param_shapes

# state-dict entries of the Hugging Face model that have no counterpart: the precomputed position table (this library
# computes and caches the cropped table itself)
IGNORED_HF_KEYS = ("pos_embed.pos_embed",)


def name_plan(cfg: DiTConfig) -> "OrderedDict[str, tuple]":
    """reference name -> (kind, [hf names]). kind 'linear': concatenate the hf weights along rows (outputs), then
    transpose to (C_in, C_out); 'vector': concatenate; 'asis': copy."""
    plan = OrderedDict()

    def lin(ref, *hf):
        plan[ref + ".weight"] = ("linear", [h + ".weight" for h in hf])
        plan[ref + ".bias"] = ("vector", [h + ".bias" for h in hf])

    lin("timestep_mlp.0", "time_text_embed.timestep_embedder.linear_1")
    lin("timestep_mlp.2", "time_text_embed.timestep_embedder.linear_2")
    lin("pooled_mlp.0", "time_text_embed.text_embedder.linear_1")
    lin("pooled_mlp.2", "time_text_embed.text_embedder.linear_2")
    lin("captions_linear", "context_embedder")
    plan["to_patch.conv.weight"] = ("asis", ["pos_embed.proj.weight"])
    plan["to_patch.conv.bias"] = ("asis", ["pos_embed.proj.bias"])
    for l in range(cfg.num_layers):
        r, h = f"transformer.{l}.", f"transformer_blocks.{l}."
        last = l == cfg.num_layers - 1
        dual = l in cfg.dual_attention_layers
        lin(r + "context_ada_lnorm.linear", h + "norm1_context.linear")
        lin(r + "context_to_qkv", h + "attn.add_q_proj", h + "attn.add_k_proj", h + "attn.add_v_proj")
        if cfg.use_qk_norm:
            plan[r + "context_rmsnorm_key.weight"] = ("asis", [h + "attn.norm_added_k.weight"])
            plan[r + "context_rmsnorm_query.weight"] = ("asis", [h + "attn.norm_added_q.weight"])
        if not last:
            lin(r + "context_attn_Wout", h + "attn.to_add_out")
            lin(r + "context_mlp.lin1", h + "ff_context.net.0.proj")
            lin(r + "context_mlp.lin2", h + "ff_context.net.2")
        lin(r + "latent_ada_lnorm.linear", h + "norm1.linear")
        lin(r + "latent_to_qkv", h + "attn.to_q", h + "attn.to_k", h + "attn.to_v")
        if cfg.use_qk_norm:
            plan[r + "latent_rmsnorm_key.weight"] = ("asis", [h + "attn.norm_k.weight"])
            plan[r + "latent_rmsnorm_query.weight"] = ("asis", [h + "attn.norm_q.weight"])
        lin(r + "latent_attn_Wout", h + "attn.to_out.0")
        lin(r + "latent_mlp.lin1", h + "ff.net.0.proj")
        lin(r + "latent_mlp.lin2", h + "ff.net.2")
        if dual:
            lin(r + "latent_dual_to_qkv", h + "attn2.to_q", h + "attn2.to_k", h + "attn2.to_v")
            if cfg.use_qk_norm:
                plan[r + "latent_dual_rmsnorm_key.weight"] = ("asis", [h + "attn2.norm_k.weight"])
                plan[r + "latent_dual_rmsnorm_query.weight"] = ("asis", [h + "attn2.norm_q.weight"])
            lin(r + "latent_dual_attn_Wout", h + "attn2.to_out.0")
    lin("ada_ln_out.linear", "norm_out.linear")
    lin("linear_out", "proj_out")
    return plan


def _as_f32(a):
    if hasattr(a, "detach"):  # torch tensor (bf16 / fp16 files cannot go through numpy directly)
        a = a.detach().float().cpu().numpy()
    return np.asarray(a, dtype=np.float32)


def convert_state_dict(hf, cfg: DiTConfig, strict: bool = True) -> "OrderedDict[str, np.ndarray]":
    """Hugging Face state dict (name -> array or torch tensor) -> reference-named float32 arrays in the reference layout.
    Raises KeyError naming the first missing entry, ValueError on a shape that does not fit `cfg`, and, with strict,
    ValueError on entries that nothing maps to."""
    shapes = dit_param_shapes(cfg)
    plan = name_plan(cfg)
    assert list(plan.keys()) == list(shapes.keys()), "name plan and parameter inventory disagree"
    out = OrderedDict()
    used = set()
    for ref, (kind, names) in plan.items():
        parts = []
        for n in names:
            if n not in hf:
                raise KeyError(f"{n} (needed for {ref}) is missing from the Hugging Face state dict")
            parts.append(_as_f32(hf[n]))
            used.add(n)
        if kind == "linear":
            a = np.concatenate(parts, axis=0).T
        elif kind == "vector":
            a = np.concatenate(parts, axis=0)
        else:
            a = parts[0]
        if tuple(a.shape) != tuple(shapes[ref]):
            raise ValueError(f"{ref}: got shape {tuple(a.shape)} from {names}, the configuration needs {tuple(shapes[ref])}")
        out[ref] = np.ascontiguousarray(a, dtype=np.float32)
    if strict:
        extra = [k for k in hf.keys() if k not in used and k not in IGNORED_HF_KEYS]
        if extra:
            raise ValueError(f"{len(extra)} entries of the Hugging Face state dict map to nothing, e.g. {extra[:3]}")
    return out


def to_hf_state_dict(params, cfg: DiTConfig) -> "OrderedDict[str, np.ndarray]":
    """The inverse: reference-named arrays -> Hugging Face names and layout (what module_tests/modules.py:532-612 does
    tensor by tensor). Used for round-trip tests and for exporting."""
    out = OrderedDict()
    for ref, (kind, names) in name_plan(cfg).items():
        a = np.asarray(params[ref], dtype=np.float32)
        if kind == "linear":
            a = a.T
        pieces = np.split(a, len(names), axis=0) if len(names) > 1 else [a]
        for n, p in zip(names, pieces):
            out[n] = np.ascontiguousarray(p)
    return out


def load_safetensors(path, cfg: DiTConfig, strict: bool = True) -> "OrderedDict[str, np.ndarray]":
    """Reads one .safetensors file, a list of shards, or a directory holding `*.safetensors` (with or without the
    `*.safetensors.index.json` that lists the shards) and converts it. Only the safetensors reader is used: nothing in the
    files is executed."""
    from safetensors import safe_open

    if isinstance(path, (list, tuple)):
        files = list(path)
    elif os.path.isdir(path):
        index = [f for f in sorted(os.listdir(path)) if f.endswith(".safetensors.index.json")]
        if index:
            with open(os.path.join(path, index[0])) as f:
                files = sorted({os.path.join(path, v) for v in json.load(f)["weight_map"].values()})
        else:
            files = [os.path.join(path, f) for f in sorted(os.listdir(path)) if f.endswith(".safetensors")]
    else:
        files = [path]
    if not files:
        raise FileNotFoundError(f"no .safetensors file under {path}")
    hf = {}
    for fn in files:
        with safe_open(fn, framework="pt") as f:
            for k in f.keys():
                hf[k] = f.get_tensor(k)
    return convert_state_dict(hf, cfg, strict)
