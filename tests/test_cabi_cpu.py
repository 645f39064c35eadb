"""No GPU needed: the C-ABI library loads, exports every entry point that include/sd3_hip.h declares, reports errors
through status codes (never exits), and the host-side bookkeeping (parameter inventory, FLOP counts) is right."""
import ctypes as C
import os
import re
import subprocess

import pytest

from conftest import ROOT, load_package

pkg = load_package()
from sd3_c_amd import lib as L  # noqa: E402
from sd3_c_amd.config import sd35_medium, reference_dit_test  # noqa: E402
from sd3_c_amd.params import dit_param_shapes, block_param_shapes  # noqa: E402

HEADER = os.path.join(ROOT, "include", "sd3_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sd3_[a-zA-Z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load()
    names = declared_functions()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/sd3_hip.h but not exported by libsd3_hip.so"
    # and the Python binding covers them all (plus nothing that is not declared)
    bound = set(L.SIGNATURES) | {"sd3_last_error", "sd3_version"}
    assert set(names) == bound


def test_header_is_plain_c():
    src = '#include "sd3_hip.h"\nint main(void){ sd3_block_weights w; (void)w; return sd3_version() < 0; }\n'
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), "-x", "c", "-"], input=src, text=True,
                       capture_output=True)
    assert r.returncode == 0, r.stderr


def test_reference_named_cpp_overloads_compile():
    src = ('#include "modules_api.hpp"\nvoid f(float* p){ linear(p,p,p,p,1,2,3); rmsnorm_group(p,p,p,nullptr,1e-6f,2,1,1,4); mlp(p,p,p,p,p,p,p,1,1,1,1,silu); '
           'scale_and_shift(p,p,p,p,1,1,1); multihead_attention(p,p,p,p,1,1,1,1,1); }\n')
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "sd3.c_amd", "csrc"), "-x", "c++", "-"], input=src, text=True,
                       capture_output=True)
    assert r.returncode == 0, r.stderr


def test_cpp_callers_of_the_boundary_are_built_and_link():
    """tests/cpp: the C++ program over modules_api.hpp and the reference-side torch binding (run on the GPU by
    tests/test_gpu_cpp_boundary.py); here: they exist, resolve their libraries, and the binding imports and exports its two entry points."""
    import sys
    cpp = os.path.join(ROOT, "tests", "cpp")
    if not (os.path.exists(os.path.join(cpp, "host_block")) and os.path.exists(os.path.join(cpp, "sd3_ref_binding.so"))):
        r = subprocess.run(["make", "-C", cpp], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run(["ldd", os.path.join(cpp, "host_block")], capture_output=True, text=True)
    assert "libsd3_hip.so =>" in r.stdout and "not found" not in r.stdout, r.stdout
    import torch  # noqa: F401  (the binding links against torch's libraries)
    sys.path.insert(0, cpp)
    import sd3_ref_binding
    assert callable(sd3_ref_binding.DiT_block_cuda) and callable(sd3_ref_binding.DiT_cuda)


def test_argument_errors_are_status_codes_not_exits():
    lib = L.load()
    assert lib.sd3_version() >= 1
    none = C.c_void_p(0)
    assert lib.sd3_linear(none, none, none, none, 4, 4, 4, none) == 1  # SD3_ERR_INVALID_ARG
    assert b"null pointer" in lib.sd3_last_error()
    assert lib.sd3_linear(none, none, none, none, 0, 4, 4, none) == 0  # empty batch: nothing to do
    assert lib.sd3_linear(none, none, none, none, 4, -1, 4, none) == 1
    assert lib.sd3_rmsnorm_group(none, none, none, none, 1e-6, 3, 1, 2, 10, none) == 1  # 10 % 3
    assert b"divisible" in lib.sd3_last_error()
    assert lib.sd3_gelu_tanh(none, none, -5, none) == 1
    assert lib.sd3_conv2d(none, none, none, none, 1, 2, 2, 4, 8, 8, 8, 5, 5, 2, 0, none) == 1  # wrong output size
    assert lib.sd3_weights_bind(none, b"x", none, 4) == 1
    assert lib.sd3_dit_block(none, none, none, none, b"", 1, 1, 1, 64, 1, 4, 0, 0, 0, 0) == 1
    with pytest.raises(L.Sd3Error):
        L.call("sd3_silu", None, None, 8, None)


def test_tuning_switches_are_checked():
    lib = L.load()
    assert lib.sd3_tune(b"gemm_bf16_tile", 192) == 0 and lib.sd3_tune(b"gemm_bf16_tile", 0) == 0
    assert lib.sd3_tune(b"gemm_bf16_tile", 100) == 1
    assert lib.sd3_tune(b"attention_context_splits", 1) == 1 and lib.sd3_tune(b"attention_context_splits", -1) == 0
    assert lib.sd3_tune(b"gemm_bf16_row_split", 1) == 0
    assert lib.sd3_tune(b"no_such_switch", 1) == 1 and b"unknown setting" in lib.sd3_last_error()
    assert lib.sd3_tune(None, 1) == 1


def test_context_creation_without_a_gpu_fails_cleanly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    with pytest.raises(L.Sd3Error) as e:
        L.call("sd3_ctx_create", C.byref(h), 0)
    assert e.value.status == 4 and not h.value


def test_parameter_inventory_matches_sd35_medium():
    shapes = dit_param_shapes(sd35_medium())
    total = sum(int(__import__("numpy").prod(s)) for s in shapes.values())
    assert abs(total - 2.242e9) / 2.242e9 < 2e-3  # 2.242e9 parameters
    ada = sum(int(__import__("numpy").prod(s)) for n, s in shapes.items() if "ada_l" in n and n.endswith("weight"))
    assert abs(ada - 7.67e8) / 7.67e8 < 5e-3     # of which adaLN modulation projections
    assert shapes["transformer.0.latent_ada_lnorm.linear.weight"] == (1536, 9 * 1536)     # dual block: 9 chunks
    assert shapes["transformer.13.latent_ada_lnorm.linear.weight"] == (1536, 6 * 1536)
    assert shapes["transformer.23.context_ada_lnorm.linear.weight"] == (1536, 2 * 1536)   # last block: context pre-only
    assert "transformer.23.context_mlp.lin1.weight" not in shapes and "transformer.13.latent_dual_to_qkv.weight" not in shapes
    assert shapes["to_patch.conv.weight"] == (1536, 16, 2, 2) and shapes["linear_out.weight"] == (1536, 64)
    small = dit_param_shapes(reference_dit_test())
    assert small["captions_linear.weight"] == (2048, 256) and small["timestep_mlp.0.weight"] == (256, 256)
    blk = block_param_shapes(768, 2, True, True, False, 64)
    assert blk["latent_mlp.lin1.weight"] == (768, 1536) and blk["context_rmsnorm_key.weight"] == (64,)


def test_flop_model_matches_the_published_work_table():
    import sys
    sys.path.insert(0, ROOT)
    import bench
    g, a, e = bench.forward_flops(sd35_medium(), 2, 154, 4096)
    assert abs(g - 1.3551e13) / 1.3551e13 < 1e-3 and abs(a - 8.007e12) / 8.007e12 < 1e-3
    g, a, e = bench.forward_flops(sd35_medium(), 2, 154, 1024)
    assert abs(g + a + e - 4.276e12) / 4.276e12 < 2e-3


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr
