"""ctypes binding of libsd3_hip.so (the C ABI declared in include/sd3_hip.h).

The library is built in-tree by `sd3.c_amd/build.py` (hipcc, gfx950). There is no fallback: if it is missing or a
call fails, an exception is raised."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsd3_hip.so")

PREC_F32, PREC_BF16, PREC_BF16_FP8, PREC_BF16_FP8_TENSOR = 0, 1, 2, 3
ACT_SILU, ACT_GELU_TANH = 0, 1

vp, ci, cf, cll, cs = C.c_void_p, C.c_int, C.c_float, C.c_longlong, C.c_char_p

# name -> argument types (all return int status), in the order of include/sd3_hip.h
SIGNATURES = {
    "sd3_layernorm": [vp, vp, vp, vp, vp, vp, cf, ci, ci, ci, vp],
    "sd3_rmsnorm": [vp, vp, vp, vp, cf, ci, ci, ci, vp],
    "sd3_rmsnorm_group": [vp, vp, vp, vp, cf, ci, ci, ci, ci, vp],
    "sd3_gelu": [vp, vp, cll, vp],
    "sd3_gelu_tanh": [vp, vp, cll, vp],
    "sd3_silu": [vp, vp, cll, vp],
    "sd3_linear": [vp, vp, vp, vp, ci, ci, ci, vp],
    "sd3_partial_linear": [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp],
    "sd3_add": [vp, vp, vp, cll, vp],
    "sd3_multihead_attention": [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp],
    "sd3_sinusoidal_embedding": [vp, vp, ci, ci, vp],
    "sd3_positional_embedding2D": [vp, ci, ci, ci, ci, vp],
    "sd3_crop_positional_embedding2D": [vp, vp, ci, ci, ci, ci, vp],
    "sd3_conv2d": [vp, vp, vp, vp] + [ci] * 11 + [vp],
    "sd3_patch_embedding": [vp, vp, vp, vp] + [ci] * 8 + [vp],
    "sd3_mlp": [vp] * 7 + [ci] * 5 + [vp],
    "sd3_scale_and_shift": [vp, vp, vp, vp, ci, ci, ci, vp],
    "sd3_gating_mechanism": [vp, vp, vp, ci, ci, ci, vp],
    "sd3_concatenate_along_tokens": [vp, vp, vp, ci, ci, ci, ci, vp],
    "sd3_split_along_tokens": [vp, vp, vp, ci, ci, ci, ci, vp],
    "sd3_dit_block_w": [vp, vp, vp, vp, vp] + [ci] * 10,
    "sd3_ctx_create": [C.POINTER(vp), ci],
    "sd3_ctx_destroy": [vp],
    "sd3_ctx_set_stream": [vp, vp],
    "sd3_ctx_synchronize": [vp],
    "sd3_weights_bind": [vp, cs, vp, cll],
    "sd3_weights_unbind": [vp, cs],
    "sd3_weights_forget": [vp, vp],
    "sd3_weights_clear": [vp],
    "sd3_weights_copies_built": [vp, C.POINTER(cll)],
    "sd3_weights_prepare": [vp, ci],
    "sd3_dit_block": [vp, vp, vp, vp, cs] + [ci] * 10,
    "sd3_dit_block_static": [vp, vp, vp, vp, cs] + [ci] * 10,
    "sd3_dit_forward": [vp] * 6 + [ci] * 5 + [vp] + [ci] * 12,
    "sd3_dit_forward_cfg_euler": [vp] * 6 + [ci] * 5 + [vp] + [ci] * 12 + [cf, cf],
    "sd3_profile_begin": [vp],
    "sd3_profile_end": [vp, vp, vp, vp],
    "sd3_flash_attention_bf16": [vp] * 8 + [ci] * 5 + [vp],
    "sd3_flash_attention_bf16_split": [vp] * 4 + [ci] * 6 + [vp, cll, vp],
    "sd3_pack_weight_bf16": [vp, vp, ci, ci, vp],
    "sd3_gemm_bf16": [vp, vp, vp, vp, ci, ci, ci, ci, vp],
    "sd3_gemm_bf16_grouped": [vp, ci, ci, ci, vp],
    "sd3_quantize_weight_fp8": [vp, vp, vp, ci, ci, ci, vp],
    "sd3_quantize_rows_fp8": [vp, vp, vp, ci, ci, ci, vp],
    "sd3_gemm_fp8": [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp],
    "sd3_cast_f32_to_bf16": [vp, vp, cll, vp],
    "sd3_gemm_bf16_force_tile": [ci],
    "sd3_tune": [cs, ci],
    "sd3_probe_mfma_bf16": [ci, ci, vp],
}


class GemmBf16Problem(C.Structure):
    """sd3_gemm_bf16_problem of include/sd3_hip.h"""
    _fields_ = [("A", vp), ("wpacked", vp), ("bias", vp), ("out", vp), ("M", ci), ("N", ci), ("K", ci), ("gate", vp), ("gate_ld", ci), ("resid", vp),
                ("table", vp), ("rows_per_batch", ci), ("rms_q", vp), ("rms_k", vp)]


class Sd3Error(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"sd3 status {status}: {message}")
        self.status = status


_lib = None


def load():
    """Loads the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is missing: build it with `python sd3.c_amd/build.py` (there is no CPU fallback)")
        # torch ships its own copy of the HIP runtime under the same SONAME (libamdhip64.so.7). Two copies in one process
        # do not share devices or streams, so torch -- which holds the tensors this library is handed -- is loaded first
        # and the library then binds to the runtime torch brought in.
        import torch  # noqa: F401
        lib = C.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = ci
        lib.sd3_last_error.restype = cs
        lib.sd3_last_error.argtypes = []
        lib.sd3_version.restype = ci
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        raise Sd3Error(status, load().sd3_last_error().decode(errors="replace"))


def call(name, *args):
    check(getattr(load(), name)(*args))
