"""The forward halves of the reference's own unit scripts (module_tests/*.py), run against the stand-in for its extension with the
same calls, shapes, seeds and library oracles; where a script only prints its difference, the bound here is the fp32 one of this
library (1e-4 max-abs; 1e-5 where the reference asserts that)."""
import os
import sys

import pytest
import torch
import torch.nn.functional as TF

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "sd3.c_amd"))
import custom_modules as F2  # noqa: E402


def test_ln_py():
    """module_tests/ln.py:57-67, 45: B,T,C = 2,3,4, affine, eps 1e-5, the call that also returns mean and rstd."""
    B, T, C = 2, 3, 4
    torch.manual_seed(1)
    x, w, b = torch.randn(B, T, C), torch.randn(C), torch.randn(C)
    out2, mean, rstd = F2.layer_norm(x, w, b, 1e-5, True)
    assert (out2 - TF.layer_norm(x, (C,), w, b, 1e-5)).abs().max().item() <= 1e-5
    assert (mean.reshape(B, T) - x.mean(-1)).abs().max().item() <= 1e-6
    assert (rstd.reshape(B, T) - (x.var(-1, unbiased=False) + 1e-5) ** -0.5).abs().max().item() <= 1e-4


def test_rmsnorm_py():
    """module_tests/rmsnorm.py:9, 22-29."""
    B, T, C = 2, 3, 4
    torch.manual_seed(1)
    x, w = torch.randn(B, T, C), torch.randn((C,))
    out2, rms = F2.rms_norm(x, w, 1e-5, True)
    assert (out2 - TF.rms_norm(x, (C,), w, 1e-5)).abs().max().item() <= 1e-5


def test_gelu_py_and_silu_py():
    """module_tests/gelu.py:20-28 (the erf form, at the script's 1e-5) and module_tests/silu.py:20-25."""
    torch.manual_seed(1)
    x = torch.randn(2, 3, 4)
    assert (F2.gelu(x) - TF.gelu(x, approximate="none")).abs().max().item() <= 1e-5
    x = torch.randn(2, 3, 128)
    assert (F2.silu(x) - TF.silu(x)).abs().max().item() <= 1e-5


def test_linear_py():
    """module_tests/linear.py:25-34: (2, 4, 512) @ (512, 128) + bias."""
    torch.manual_seed(1)
    x, W, b = torch.randn(2, 4, 512), torch.randn((512, 128)), torch.randn(128)
    out = F2.linear(x, W, b)
    assert out.shape == (2, 4, 128)
    assert (out - (x @ W + b)).abs().max().item() <= 1e-4 * max(1.0, (x @ W).abs().max().item() / 16)


@pytest.mark.parametrize("B,C_in,C_out,H,W,kernel_size,stride,padding", [
    (2, 1, 1, 32, 32, (2, 3), 1, 0), (2, 3, 1, 32, 32, (4, 2), 1, 0), (2, 1, 1, 32, 32, (3, 3), 1, 3), (2, 1, 2, 6, 6, (3, 3), 2, 1),
    (2, 16, 32, 128, 128, (3, 5), 2, 2)])
def test_conv2d_py(B, C_in, C_out, H, W, kernel_size, stride, padding):
    """module_tests/conv2d.py:42-56: the five configurations, non-square kernels, stride and padding included."""
    torch.manual_seed(2)
    x, kernel, bias = torch.randn((B, C_in, H, W)), torch.randn((C_out, C_in, *kernel_size)), torch.randn((C_out,))
    out = TF.conv2d(x, kernel, bias, stride, padding)
    out2 = F2.conv2d(x, kernel, bias, stride, padding)
    assert out2.shape == out.shape
    assert (out - out2).abs().max().item() <= 1e-4 * max(1.0, out.abs().max().item() / 16)


def test_sinusoidal_embeddings_py():
    """module_tests/sinusoidal_embeddings.py:7-45: timestep embedding of 16 timesteps at width 256 against the script's float32 formula
    ([cos | sin] of t * exp(-ln(10000) i / 128)), and the 96 x 96 position table with base size 64 against its float64 one."""
    B, C, H, W, base_size = 16, 256, 96, 96, 64
    torch.manual_seed(3)
    t = torch.rand((B,))
    half = C // 2
    freq = torch.exp(-9.2103403719761836 * torch.arange(half, dtype=torch.float32) / half)
    temb = torch.cat([torch.cos(t[:, None] * freq), torch.sin(t[:, None] * freq)], dim=1)
    assert (temb - F2.sinusoidal_embedding(t, C)).abs().max().item() <= 1e-5
    # the script's table (its meshgrid with indexing="xy"): row i * H + j holds [sin | cos] of h[j] and then [sin | cos] of w[i]
    div = 1.0 / (10000.0 ** (torch.arange(C // 4, dtype=torch.float64) / (C / 4.0)))
    hh = torch.arange(H, dtype=torch.float64) / (H / base_size)
    ww = torch.arange(W, dtype=torch.float64) / (W / base_size)
    fast = torch.cat([torch.sin(hh[:, None] * div), torch.cos(hh[:, None] * div)], 1)   # (H, C/2), index j
    slow = torch.cat([torch.sin(ww[:, None] * div), torch.cos(ww[:, None] * div)], 1)   # (W, C/2), index i
    pe = torch.cat([fast[None].expand(W, H, C // 2), slow[:, None].expand(W, H, C // 2)], 2).reshape(W * H, C).to(torch.float32)
    pe2 = F2.positional_embedding(C, H, W, base_size)
    assert pe2.shape == (H * W, C)
    assert (pe - pe2).abs().max().item() <= 1e-5


def test_attention_py():
    """module_tests/attention.py:52-66: F2.mha against nn.MultiheadAttention with identity projections, B,T,L,C = 2,128,96,512, 8 heads
    (the script names its query length T and key length L)."""
    B, T, L, C, num_heads = 2, 128, 96, 512, 8
    torch.manual_seed(1)
    Q, K, V = torch.randn((B, T, C)), torch.randn((B, L, C)), torch.randn((B, L, C))
    mha = torch.nn.MultiheadAttention(C, num_heads, 0.0, batch_first=True)
    mha.in_proj_weight.data = torch.cat([torch.eye(C), torch.eye(C), torch.eye(C)], 0)
    mha.in_proj_bias.data.zero_()
    mha.out_proj.weight.data = torch.eye(C)
    mha.out_proj.bias.data.zero_()
    with torch.no_grad():
        out1, _ = mha(Q, K, V, need_weights=False)
    out2 = F2.mha(Q, K, V, num_heads)
    assert (out1 - out2).abs().max().item() <= 1e-4


@pytest.mark.parametrize("activation", ["SiLU", "GELU"])
def test_mlp_py(activation):
    """module_tests/mlp.py:7-26: 16 rows, 256 -> 1024 -> 256, the binding's ten-argument call with the activation by name."""
    B, C_in, C_hid, C_out = 16, 256, 1024, 256
    torch.manual_seed(4)
    lin1, lin2 = torch.nn.Linear(C_in, C_hid), torch.nn.Linear(C_hid, C_out)
    act = torch.nn.SiLU() if activation == "SiLU" else torch.nn.GELU(approximate="tanh")
    x = torch.randn((B, C_in))
    with torch.no_grad():
        y_true = lin2(act(lin1(x)))
    y = F2.mlp(x, lin1.weight.data.T.contiguous(), lin1.bias.data, lin2.weight.data.T.contiguous(), lin2.bias.data, activation, B, C_in, C_hid, C_out)
    assert y.shape == (B, C_out)
    assert (y - y_true).abs().max().item() <= 1e-4
