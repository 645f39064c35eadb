"""Stand-in for the reference's torch extension `custom_modules` (PYBIND11_MODULE, modules.cpp:1789-1815), forward entry
points only, so that scripts written like the reference's drivers run against this library unchanged:

    import sys; sys.path.insert(0, "<repo>/sd3.c_amd"); import custom_modules as F
    x_out = F.DiT(pooled, captions, latent, timesteps, params, num_layers, set(dual_layers), pooled_dim, captions_dim,
                  in_channels, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm)

The reference's `Dit_block` and `DiT` take host tensors and compute on the CPU (module_tests/DiT.py:33-47,
module_tests/dit_block.py:40-46); here the same calls copy their arguments to the GPU, run the path named by the module-level
`PRECISION` ("fp32", the default: the one held to the reference's 1e-4 / 1e-5 comparisons; set `F.PRECISION = "bf16"` for the
bf16 MFMA throughput path, relative L2 <= 1e-2) and copy the results back, keeping the in-place contract of the block:
`context_embeddings` and `latent_vector` are overwritten and returned. `DiT_block_cuda` takes device tensors as in
module_tests/dit_block.py:60-66. There is no CPU fallback: without a GPU every call raises.

The backward functions and `softmax*` of the extension are not on the forward path and are not provided.
"""
import os
import sys

import torch

_here = os.path.dirname(os.path.abspath(__file__))
if "sd3_c_amd" not in sys.modules:  # the package directory name has a dot in it: load it under an importable name
    import importlib.util

    _spec = importlib.util.spec_from_file_location("sd3_c_amd", os.path.join(_here, "__init__.py"), submodule_search_locations=[_here])
    _mod = importlib.util.module_from_spec(_spec)
    sys.modules["sd3_c_amd"] = _mod
    _spec.loader.exec_module(_mod)
from sd3_c_amd import modules as _M  # noqa: E402

_DEV = "cuda"
PRECISION = "fp32"  # "fp32" | "bf16": the arithmetic of Dit_block / DiT_block_cuda / DiT (the reference's signatures have no slot for it)


def _up(t):
    return t.detach().to(device=_DEV, dtype=torch.float32).contiguous()


_uploaded = {}  # name -> (tensor of the caller, its version counter, the device copy)


def _params_up(params):
    """Device copies of a parameter map. The reference's entry points receive the whole map on every call; a tensor that is the same
    object (or the same memory) with the same torch version counter as in the previous call keeps its device copy, so a sampling
    loop uploads the weights once and the context behind `Dit_block` / `DiT` keeps what it derived from them. Tensors that are on
    the GPU already, in float32 and contiguous, are passed through. `release()` drops the copies."""
    out = {}
    for name, t in params.items():
        old = _uploaded.get(name)
        if old is not None and (old[0] is t or (old[0].data_ptr() == t.data_ptr() and old[0].shape == t.shape and old[0].dtype == t.dtype)) \
                and old[1] == t._version:
            out[name] = old[2]
            continue
        d = _up(t)
        _uploaded[name] = (t, t._version, d)
        out[name] = d
    for name in [n for n in _uploaded if n not in params]:
        del _uploaded[name]
    return out


def release():
    """Frees what the module keeps between calls: the device copies of the last parameter map and the contexts behind `Dit_block` /
    `DiT` (their bf16 weight copies and workspaces)."""
    _uploaded.clear()
    _M.release_shared_contexts()


def _host_op(fn):
    """Operator-level entry points: host tensors in, host tensor out, like the reference's CPU functions."""
    def wrapped(*args):
        dev_args = [_up(a) if isinstance(a, torch.Tensor) else a for a in args]
        out = fn(*dev_args)
        torch.cuda.synchronize()
        if isinstance(out, (list, tuple)):
            return [o.cpu() if isinstance(o, torch.Tensor) else o for o in out]
        return out.cpu() if isinstance(out, torch.Tensor) else out
    wrapped.__name__ = fn.__name__
    wrapped.__doc__ = fn.__doc__
    return wrapped


layer_norm = _host_op(lambda input, weight=None, bias=None, eps=1e-5, save_for_backward=False: _M.layer_norm(input, weight, bias, eps, save_for_backward))
rms_norm = _host_op(lambda input, weight, eps, save_for_backward=False: _M.rms_norm(input, weight, eps, save_for_backward))
gelu = _host_op(_M.gelu)            # modules.cpp:1795 binds `gelu` to the erf form (modules.cpp:280-285)
gelu_tanh = _host_op(_M.gelu_tanh)  # the block MLPs' activation (modules.cpp:293); not exported by the reference's extension, kept under its own name
silu = _host_op(_M.silu)
linear = _host_op(_M.linear)
conv2d = _host_op(_M.conv2d)
sinusoidal_embedding = _host_op(_M.sinusoidal_embedding)
mha = _host_op(_M.mha)
mlp = _host_op(_M.mlp)


def positional_embedding(emb_dim, height, width, base_size):
    """modules.cpp:997 positional_embedding2D_forward"""
    out = _M.positional_embedding(emb_dim, height, width, base_size, device=_DEV)
    torch.cuda.synchronize()
    return out.cpu()


def Dit_block(temp_embeddings, context_embeddings, latent_vector, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm,
              discard_context, precision=None):
    """modules.cpp:1508 DiT_block_forward on host tensors: context_embeddings and latent_vector are updated in place and returned.
    `precision` (not in the reference's list) overrides the module-level PRECISION for this call."""
    y, c, x = _up(temp_embeddings), _up(context_embeddings), _up(latent_vector)
    c, x = _M.Dit_block(y, c, x, _params_up(params), B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm, discard_context,
                        precision=precision or PRECISION)
    context_embeddings.copy_(c.to(context_embeddings.device))
    latent_vector.copy_(x.to(latent_vector.device))
    return [context_embeddings, latent_vector]


def DiT_block_cuda(temp_embeddings, context_embeddings, latent_vector, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention,
                   use_qk_norm, discard_context, precision=None):
    """modules.cpp:1783 DiT_block_forward_cuda: device tensors, updated in place and returned."""
    return _M.Dit_block(temp_embeddings, context_embeddings, latent_vector, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention,
                        use_qk_norm, discard_context, precision=precision or PRECISION)


def DiT(pooled_captions, captions, latent_vector, timesteps, params, num_layers, dual_attention_layers, pooled_dim, captions_dim, C_in, emb_dim, attn_heads,
        mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision=None):
    """modules.cpp:1605 DiT_forward on host (or device) tensors: returns a new (B, C_in, H, W) tensor on the latent's device."""
    out = _M.DiT(_up(pooled_captions), _up(captions), _up(latent_vector), _up(timesteps), _params_up(params), num_layers, dual_attention_layers,
                 pooled_dim, captions_dim, C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm,
                 precision=precision or PRECISION)
    return out.to(latent_vector.device)
