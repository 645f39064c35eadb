"""Host-side mirror of the reference's `custom_modules` extension (modules.cpp:1789-1815), running on the GPU.

Same function names, argument order and in-place behaviour as the reference's Python-visible functions, for torch
tensors that live on the MI355X. torch is only used to hold device memory and to name the current stream; every
operation is one or more launches of this repo's HIP kernels through the C ABI. Extra keyword: `precision`
("fp32" = fp32 MFMA path matching the CPU reference to 1e-4, "bf16" = bf16 MFMA path)."""
import ctypes as C

import torch

from . import lib as L

_PREC = {"fp32": L.PREC_F32, "f32": L.PREC_F32, "bf16": L.PREC_BF16, "bf16+fp8": L.PREC_BF16_FP8, "bf16+fp8-tensor": L.PREC_BF16_FP8_TENSOR}


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, name, dtype=torch.float32):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a tensor on the GPU")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


# ------------------------------------------------------------------ per-op functions (reference names)
def layer_norm(input, weight=None, bias=None, eps=1e-5, save_for_backward=True):
    """modules.cpp:51 LayerNorm_forward -> [output, mean, rstd] (the last two only when save_for_backward)."""
    x = _dev(input, "input")
    B, T, Cd = x.shape
    y = torch.empty_like(x)
    mean = torch.empty((B, T), device=x.device) if save_for_backward else None
    rstd = torch.empty((B, T), device=x.device) if save_for_backward else None
    L.call("sd3_layernorm", _p(x), _p(y), _p(mean), _p(rstd), _p(weight), _p(bias), eps, B, T, Cd, _stream())
    return [y, mean, rstd] if save_for_backward else [y]


def rms_norm(input, weight, eps, save_for_backward=False):
    """modules.cpp:200 RMSNorm_forward."""
    x = _dev(input, "input")
    B, T, Cd = x.shape
    y = torch.empty_like(x)
    rms = torch.empty((B, T), device=x.device) if save_for_backward else None
    L.call("sd3_rmsnorm", _p(x), _p(y), _p(weight), _p(rms), eps, B, T, Cd, _stream())
    return [y, rms] if save_for_backward else [y]


def rms_norm_group(input, weight, eps, groups):
    """modules.cpp:192 rmsnorm_group, out of place."""
    x = _dev(input, "input")
    B, T, Cd = x.shape
    y = torch.empty_like(x)
    L.call("sd3_rmsnorm_group", _p(x), _p(y), _p(weight), _p(None), eps, groups, B, T, Cd, _stream())
    return y


def gelu(input):
    """modules.cpp:302 GELU_forward: the erf form (modules.cpp:280-285), what the extension exports as `gelu`."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    L.call("sd3_gelu", _p(x), _p(y), x.numel(), _stream())
    return y


def gelu_tanh(input):
    """modules.cpp:293 gelu_tanh (the activation of the block MLPs)."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    L.call("sd3_gelu_tanh", _p(x), _p(y), x.numel(), _stream())
    return y


def silu(input):
    """modules.cpp:360 SiLU_forward."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    L.call("sd3_silu", _p(x), _p(y), x.numel(), _stream())
    return y


def add(input, other):
    """modules.cpp:513 add: element-wise sum (the residual adds of the block, modules.cpp:1462, 1485-1486)."""
    a, b = _dev(input, "input"), _dev(other, "other")
    if a.shape != b.shape:
        raise ValueError("add: shapes differ")
    out = torch.empty_like(a)
    L.call("sd3_add", _p(a), _p(b), _p(out), a.numel(), _stream())
    return out


def linear(input, weight, bias):
    """modules.cpp:538 Linear_forward: weight is (C_in, C_out)."""
    x, W, b = _dev(input, "input"), _dev(weight, "weight"), _dev(bias, "bias")
    Cin, Cout = W.shape
    rows = x.numel() // Cin
    y = torch.empty(x.shape[:-1] + (Cout,), device=x.device)
    L.call("sd3_linear", _p(x), _p(W), _p(b), _p(y), rows, Cin, Cout, _stream())
    return y


def partial_linear(input, weight, bias, n0, N):
    """modules.cpp:492 partial_linear: columns [n0, n0+N) of a (K, Nmax) weight."""
    x, W, b = _dev(input, "input"), _dev(weight, "weight"), _dev(bias, "bias")
    K, Nmax = W.shape
    rows = x.numel() // K
    y = torch.empty(x.shape[:-1] + (N,), device=x.device)
    L.call("sd3_partial_linear", _p(x), _p(W), _p(b), _p(y), rows, K, N, Nmax, n0, _stream())
    return y


def conv2d(input, kernel, bias, stride, padding):
    """modules.cpp:1065 conv2d_forward."""
    x, k, b = _dev(input, "input"), _dev(kernel, "kernel"), _dev(bias, "bias")
    B, Cin, ih, iw = x.shape
    Cout, _, kh, kw = k.shape
    oh, ow = (ih + 2 * padding - kh) // stride + 1, (iw + 2 * padding - kw) // stride + 1
    y = torch.empty((B, Cout, oh, ow), device=x.device)
    L.call("sd3_conv2d", _p(x), _p(y), _p(k), _p(b), B, kh, kw, Cin, Cout, ih, iw, oh, ow, stride, padding, _stream())
    return y


def sinusoidal_embedding(timesteps, emb_dim):
    """modules.cpp:920 sinusoidal_embedding."""
    t = _dev(timesteps, "timesteps")
    out = torch.empty((t.shape[0], emb_dim), device=t.device)
    L.call("sd3_sinusoidal_embedding", _p(t), _p(out), t.shape[0], emb_dim, _stream())
    return out


def positional_embedding(emb_dim, height, width, base_size, device="cuda"):
    """modules.cpp:997 positional_embedding2D_forward -> (height*width, emb_dim)."""
    out = torch.empty((height * width, emb_dim), device=device)
    L.call("sd3_positional_embedding2D", _p(out), emb_dim, height, width, base_size, _stream())
    return out


def crop_positional_embedding(pos_embed, pos_embed_max_size, new_height, new_width, emb_dim):
    """modules.cpp:977 crop_positional_embedding2D."""
    out = torch.empty((new_height * new_width, emb_dim), device=pos_embed.device)
    L.call("sd3_crop_positional_embedding2D", _p(_dev(pos_embed, "pos_embed")), _p(out), pos_embed_max_size, new_height, new_width, emb_dim, _stream())
    return out


def patch_embedding(latent, kernel, bias, emb_dim, patch_size, pos_embed_max_size, base_height):
    """modules.cpp:1093 PatchEmbedding -> (B, Tx, emb_dim)."""
    x = _dev(latent, "latent")
    B, Cin, H, W = x.shape
    hp, wp = (H - patch_size) // patch_size + 1, (W - patch_size) // patch_size + 1
    out = torch.empty((B, hp * wp, emb_dim), device=x.device)
    L.call("sd3_patch_embedding", _p(x), _p(out), _p(_dev(kernel, "kernel")), _p(_dev(bias, "bias")), B, H, W, Cin, emb_dim, patch_size,
           pos_embed_max_size, base_height, _stream())
    return out


def mha(query, key, value, num_heads):
    """modules.cpp:901 mha: (B,T,C) x (B,L,C) -> (B,T,C)."""
    q, k, v = _dev(query, "query"), _dev(key, "key"), _dev(value, "value")
    B, T, Cd = q.shape
    Lk = k.shape[1]
    if Cd % num_heads:
        raise ValueError("C must be divisible by num_heads")
    out = torch.empty_like(q)
    L.call("sd3_multihead_attention", _p(q), _p(k), _p(v), _p(out), B, num_heads, T, Lk, Cd // num_heads, _stream())
    return out


def mlp(input, W1, b1, W2, b2, activation, B=None, C_in=None, C_hid=None, C_out=None):
    """modules.cpp:1167 MLP: act(x @ W1 + b1) @ W2 + b2, argument list of the reference's binding (the four sizes may be left out: they
    follow from the weights). `activation` by the reference's names, "GELU" / "gelu" (the tanh form) or "silu" / "SILU" / "SiLU", or
    "gelu_tanh". (The reference's binding sets the activation to SiLU whatever the name, modules.cpp:1190-1192; here the name is
    honoured, as in the raw-pointer mlp of modules.cpp:1120 that the forward path uses.)"""
    x = _dev(input, "input")
    Cin, Chid = W1.shape
    Cout = W2.shape[1]
    rows = x.numel() // Cin
    for given, actual, what in ((B, rows, "B"), (C_in, Cin, "C_in"), (C_hid, Chid, "C_hid"), (C_out, Cout, "C_out")):
        if given is not None and int(given) != actual:
            raise ValueError(f"mlp: {what}={given} does not match the tensors ({actual})")
    h = torch.empty((rows, Chid), device=x.device)
    out = torch.empty(x.shape[:-1] + (Cout,), device=x.device)
    names = {"silu": L.ACT_SILU, "SILU": L.ACT_SILU, "SiLU": L.ACT_SILU, "gelu_tanh": L.ACT_GELU_TANH, "GELU": L.ACT_GELU_TANH, "gelu": L.ACT_GELU_TANH}
    if activation not in names:
        raise ValueError(f"mlp: unknown activation {activation!r}")
    act = names[activation]
    L.call("sd3_mlp", _p(x), _p(out), _p(h), _p(_dev(W1, "W1")), _p(_dev(b1, "b1")), _p(_dev(W2, "W2")), _p(_dev(b2, "b2")), rows, Cin, Chid, Cout, act,
           _stream())
    return out


def scale_and_shift(input, shift, scale):
    x = _dev(input, "input")
    B, T, Cd = x.shape
    out = torch.empty_like(x)
    L.call("sd3_scale_and_shift", _p(x), _p(out), _p(_dev(shift, "shift")), _p(_dev(scale, "scale")), B, T, Cd, _stream())
    return out


def gating_mechanism(input, gate):
    x = _dev(input, "input")
    B, T, Cd = x.shape
    out = torch.empty_like(x)
    L.call("sd3_gating_mechanism", _p(x), _p(out), _p(_dev(gate, "gate")), B, T, Cd, _stream())
    return out


def concatenate_along_tokens(x, y):
    x, y = _dev(x, "x"), _dev(y, "y")
    B, Tx, Cd = x.shape
    Ty = y.shape[1]
    out = torch.empty((B, Tx + Ty, Cd), device=x.device)
    L.call("sd3_concatenate_along_tokens", _p(x), _p(y), _p(out), B, Tx, Ty, Cd, _stream())
    return out


def split_along_tokens(input, T1):
    x = _dev(input, "input")
    B, T, Cd = x.shape
    a, b = torch.empty((B, T1, Cd), device=x.device), torch.empty((B, T - T1, Cd), device=x.device)
    L.call("sd3_split_along_tokens", _p(x), _p(a), _p(b), B, T1, T - T1, Cd, _stream())
    return a, b


# ------------------------------------------------------------------ context + model-level entry points
class Context:
    """Owns an sd3_ctx: the bound `name -> tensor` parameter map (modules.cpp:1512,1609), the bf16 copies and the workspace.
    Keeps references to the bound tensors so that their addresses stay valid."""

    def __init__(self, device=None):
        self._h = C.c_void_p()
        dev = torch.cuda.current_device() if device is None else torch.device(device).index or 0
        L.call("sd3_ctx_create", C.byref(self._h), dev)
        self._keep = {}

    def bind(self, params):
        """Adds `params` to the bound map. A name that is already bound to the same tensor (same storage address and size, unchanged
        torch version counter) costs nothing and keeps the library's derived copies; a tensor that torch has modified in place
        since it was bound has its copies dropped; anything else is bound anew."""
        keep = self._keep
        for name, t in params.items():
            old = keep.get(name)
            if old is not None:
                ot, over = old
                if ot is t or (ot.data_ptr() == t.data_ptr() and ot.numel() == t.numel()):
                    if t._version != over:  # same memory, new contents
                        L.call("sd3_weights_forget", self._h, _p(t))
                        keep[name] = (t, t._version)
                    elif ot is not t:
                        keep[name] = (t, over)
                    continue
            _dev(t, name)
            L.call("sd3_weights_bind", self._h, name.encode(), _p(t), t.numel())
            keep[name] = (t, t._version)  # the reference keeps the address alive (and out of the allocator's hands) while bound

    def set_params(self, params):
        """Makes the bound map equal to `params` (the reference's entry points receive the whole map on every call, modules.cpp:1512,
        1609): names that are not in it are unbound, the rest goes through `bind`, so an unchanged map keeps every derived copy."""
        for name in [n for n in self._keep if n not in params]:
            L.call("sd3_weights_unbind", self._h, name.encode())
            del self._keep[name]
        self.bind(params)

    def copies_built(self):
        """Derived weight copies (bf16 / fp8 / transposed) built by this context so far."""
        n = C.c_longlong(0)
        L.call("sd3_weights_copies_built", self._h, C.byref(n))
        return n.value

    def clear(self):
        L.call("sd3_weights_clear", self._h)
        self._keep = {}

    def refresh(self, precision="bf16"):
        """Call after changing bound weights in place: drops the derived bf16 copies."""
        L.call("sd3_weights_prepare", self._h, _PREC[precision])

    def block(self, y, c, x, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm, discard_context, precision="fp32", prefix=""):
        L.call("sd3_ctx_set_stream", self._h, _stream())
        L.call("sd3_dit_block", self._h, _p(_dev(y, "y")), _p(_dev(c, "c")), _p(_dev(x, "x")), prefix.encode(), B, Tc, Tx, emb_dim, attn_heads,
               mlp_expand, int(use_dual_attention), int(use_qk_norm), int(discard_context), _PREC[precision])
        return [c, x]

    def block_static(self, y, c, x, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm, discard_context, precision="fp32",
                     prefix=""):
        """`block` without any device allocation: intermediates go to the library's fixed scratch array (64 MiB per device); a block that
        needs more is refused. With "bf16" the weight copies must exist already (one earlier `block` call builds them)."""
        L.call("sd3_ctx_set_stream", self._h, _stream())
        L.call("sd3_dit_block_static", self._h, _p(_dev(y, "y")), _p(_dev(c, "c")), _p(_dev(x, "x")), prefix.encode(), B, Tc, Tx, emb_dim, attn_heads,
               mlp_expand, int(use_dual_attention), int(use_qk_norm), int(discard_context), _PREC[precision])
        return [c, x]

    def forward(self, pooled_captions, captions, latent_vector, timesteps, num_layers, dual_attention_layers, pooled_dim, captions_dim, C_in, emb_dim,
                attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision="fp32", out=None):
        lat = _dev(latent_vector, "latent_vector")
        B, _, H, W = lat.shape
        Tc = captions.shape[1]
        if out is None:
            out = torch.empty_like(lat)
        dual = sorted(int(i) for i in dual_attention_layers)
        arr = (C.c_int * max(1, len(dual)))(*dual)
        L.call("sd3_ctx_set_stream", self._h, _stream())
        L.call("sd3_dit_forward", self._h, _p(_dev(pooled_captions, "pooled_captions")), _p(_dev(captions, "captions")), _p(lat),
               _p(_dev(timesteps, "timesteps")), _p(out), B, Tc, H, W, num_layers, C.cast(arr, C.c_void_p), len(dual), pooled_dim, captions_dim, C_in,
               emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, int(use_qk_norm), _PREC[precision])
        return out

    def forward_cfg_euler(self, pooled_captions, captions, latent_vector, timesteps, guidance, dsigma, num_layers, dual_attention_layers, pooled_dim,
                          captions_dim, C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision="fp32",
                          out=None):
        """The forward on a batch [n unconditional ; n conditional] followed, in its last kernel, by classifier-free guidance and
        one Euler step: returns latent[:n] + dsigma * (v_u + guidance * (v_c - v_u)), shape (n, C_in, H, W)."""
        lat = _dev(latent_vector, "latent_vector")
        B, _, H, W = lat.shape
        Tc = captions.shape[1]
        if out is None:
            out = torch.empty((B // 2,) + tuple(lat.shape[1:]), device=lat.device)
        dual = sorted(int(i) for i in dual_attention_layers)
        arr = (C.c_int * max(1, len(dual)))(*dual)
        L.call("sd3_ctx_set_stream", self._h, _stream())
        L.call("sd3_dit_forward_cfg_euler", self._h, _p(_dev(pooled_captions, "pooled_captions")), _p(_dev(captions, "captions")), _p(lat),
               _p(_dev(timesteps, "timesteps")), _p(_dev(out, "out")), B, Tc, H, W, num_layers, C.cast(arr, C.c_void_p), len(dual), pooled_dim, captions_dim,
               C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, int(use_qk_norm), _PREC[precision], float(guidance),
               float(dsigma))
        return out

    def synchronize(self):
        L.call("sd3_ctx_synchronize", self._h)

    PROFILE_CLASSES = ("gemm", "attention", "layernorm_modulate", "adaln_linear", "gemm_fp8", "fp8_quantize")

    def profile_begin(self):
        L.call("sd3_profile_begin", self._h)

    def profile_end(self):
        """-> {class: (ms, work, launches)}; work is FLOP for gemm/attention and bytes for the memory-bound classes."""
        n = len(self.PROFILE_CLASSES)
        ms, work, cnt = (C.c_double * n)(), (C.c_double * n)(), (C.c_longlong * n)()
        L.call("sd3_profile_end", self._h, C.cast(ms, C.c_void_p), C.cast(work, C.c_void_p), C.cast(cnt, C.c_void_p))
        return {k: (ms[i], work[i], cnt[i]) for i, k in enumerate(self.PROFILE_CLASSES)}

    def close(self):
        if self._h:
            L.load().sd3_ctx_destroy(self._h)
            self._h = C.c_void_p()
            self._keep = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_shared = {}  # device index -> the Context behind the reference-shaped entry points below


def shared_context(device):
    """The one context per device that `Dit_block`, `DiT_block_cuda` and `DiT` run in. The reference's entry points take the parameter
    map on every call and keep nothing between calls; here the context stays alive, each call hands its map to `set_params`, and a
    map that has not changed re-uses the bf16 weight copies and the workspace of the previous call. The context keeps the last
    map's tensors alive until the next call replaces them or `release_shared_contexts()` is called."""
    idx = torch.device(device).index
    idx = torch.cuda.current_device() if idx is None else idx
    ctx = _shared.get(idx)
    if ctx is None:
        ctx = _shared[idx] = Context(idx)
    return ctx


def release_shared_contexts():
    """Destroys the contexts behind `Dit_block` / `DiT` (bf16 copies, workspaces, references to the last parameter maps)."""
    for ctx in _shared.values():
        ctx.close()
    _shared.clear()


def Dit_block(temp_embeddings, context_embeddings, latent_vector, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm,
              discard_context, precision="fp32"):
    """modules.cpp:1508 DiT_block_forward: mutates and returns [context_embeddings, latent_vector]. Enqueued on torch's current
    stream; like the reference's GPU entry it does not wait for the result (cuda/dit.cu:1060)."""
    ctx = shared_context(latent_vector.device)
    ctx.set_params(params)
    return ctx.block(temp_embeddings, context_embeddings, latent_vector, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm,
                     discard_context, precision)


def DiT_block_cuda(*args, **kwargs):
    """modules.cpp:1783 DiT_block_forward_cuda: the reference's GPU entry has the same argument list as Dit_block."""
    return Dit_block(*args, **kwargs)


def DiT(pooled_captions, captions, latent_vector, timesteps, params, num_layers, dual_attention_layers, pooled_dim, captions_dim, C_in, emb_dim,
        attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision="fp32"):
    """modules.cpp:1605 DiT_forward: returns a new (B, C_in, H, W) tensor; inputs are left untouched. Enqueued on torch's current
    stream, in the shared per-device context (see `shared_context`)."""
    ctx = shared_context(latent_vector.device)
    ctx.set_params(params)
    return ctx.forward(pooled_captions, captions, latent_vector, timesteps, num_layers, dual_attention_layers, pooled_dim, captions_dim, C_in, emb_dim,
                       attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision)


class Denoiser:
    """The denoiser step with weights bound once (what a sampling loop or a benchmark holds on to)."""

    def __init__(self, params, cfg, precision="bf16"):
        self.cfg, self.precision = cfg, precision
        self.ctx = Context(next(iter(params.values())).device)
        self.ctx.bind(params)

    def __call__(self, pooled_captions, captions, latent_vector, timesteps, out=None):
        c = self.cfg
        return self.ctx.forward(pooled_captions, captions, latent_vector, timesteps, c.num_layers, c.dual_attention_layers, c.pooled_dim, c.captions_dim,
                                c.in_channels, c.emb_dim, c.attn_heads, c.mlp_expand, c.patch_size, c.pos_embed_max_size, c.base_height, c.use_qk_norm,
                                self.precision, out)

    def cfg_euler_step(self, pooled_captions, captions, latent_pair, timesteps, guidance, dsigma, out=None):
        """One sampler step: `latent_pair` is the current latents repeated for the [unconditional ; conditional] halves."""
        c = self.cfg
        return self.ctx.forward_cfg_euler(pooled_captions, captions, latent_pair, timesteps, guidance, dsigma, c.num_layers, c.dual_attention_layers,
                                          c.pooled_dim, c.captions_dim, c.in_channels, c.emb_dim, c.attn_heads, c.mlp_expand, c.patch_size,
                                          c.pos_embed_max_size, c.base_height, c.use_qk_norm, self.precision, out)
