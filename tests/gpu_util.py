"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from conftest import load_package

pkg = load_package()
from sd3_c_amd import modules as M  # noqa: E402

F32_TOL = 1e-4  # max abs error of the fp32 GPU path against the CPU reference arithmetic (the fp32 parity bar of this build)
BF16_REL_L2 = 1e-2  # relative L2 of the bf16 path against the fp32 path


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_params(params):
    return {k: dev(v) for k, v in params.items()}


def host(t):
    torch.cuda.synchronize()
    return t.detach().float().cpu().numpy()


def max_abs(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max()) if a.size else 0.0


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
