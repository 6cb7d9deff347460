"""The 1x1 projection as channel-first GEMMs (deconver_amd.layers.pointwise_linear) against
``conv1d`` in float64: the map the reference's ``Linear`` computes (layers/linear.py:53-58)."""

import pytest
import torch
import torch.nn.functional as F

from deconver_amd.layers import Linear, _wgrad_chunks, _wgrad_plan, pointwise_linear

pytestmark = pytest.mark.gpu


def _rel(a, ref):
    return float((a.double().cpu() - ref).abs().max() / ref.abs().max())


@pytest.mark.parametrize("B,cin,cout,n,bias", [
    (2, 32, 128, 64 * 64 * 16, True),    # 16 chunks of the voxel axis in the weight gradient
    (1, 128, 32, 32 * 32 * 32, False),   # 16 chunks
    (3, 16, 64, 7 * 9 * 11, True),       # odd voxel count: one chunk
    (2, 8, 8, 4096, True),               # two chunks
])
def test_pointwise_linear_matches_conv1d(B, cin, cout, n, bias):
    g = torch.Generator().manual_seed(0)
    x0 = torch.randn(B, cin, n, generator=g)
    w0 = torch.randn(cout, cin, 1, generator=g) / cin ** 0.5
    b0 = torch.randn(cout, generator=g) if bias else None
    gy0 = torch.randn(B, cout, n, generator=g)
    x = x0.cuda().bfloat16().requires_grad_(True)
    w = w0.cuda().bfloat16().requires_grad_(True)
    b = b0.cuda().requires_grad_(True) if bias else None
    y = pointwise_linear(x, w, b)
    assert y.dtype == torch.bfloat16 and y.shape == (B, cout, n) and y.is_contiguous()
    y.backward(gy0.cuda().bfloat16())
    xr = x.detach().double().cpu().requires_grad_(True)
    wr = w.detach().double().cpu().requires_grad_(True)
    br = b0.double().requires_grad_(True) if bias else None
    yr = F.conv1d(xr, wr, br)
    yr.backward(gy0.bfloat16().double())
    assert _rel(y.detach(), yr.detach()) < 1e-2
    assert _rel(x.grad, xr.grad) < 1e-2
    assert _rel(w.grad, wr.grad) < 1e-2
    if bias:
        assert b.grad.dtype == torch.float32 and _rel(b.grad, br.grad) < 1e-2


def test_chunk_rule():
    assert _wgrad_chunks(2, 64 ** 3) == 64 and _wgrad_chunks(2, 128 ** 3) == 64
    assert _wgrad_chunks(2, 32 ** 3) == 16 and _wgrad_chunks(3, 7 * 9 * 11) == 1
    assert _wgrad_chunks(8, 256 * 256) == 16 and _wgrad_chunks(1, 2048) == 1
    bf16, f32 = torch.bfloat16, torch.float32
    assert [_wgrad_plan(2, s ** 3, bf16) for s in (16, 32, 64, 128)] == [1, 16, 32, 64]
    assert [_wgrad_plan(8, s ** 2, f32) for s in (64, 128, 256, 512)] == [1, 1, 1, 16]
    assert _wgrad_plan(2, 64 ** 3, f32) == 64 and _wgrad_plan(3, 7 * 9 * 11, bf16) == 1


def test_linear_module_under_autocast_keeps_float32_parameter_gradients():
    torch.manual_seed(0)
    lin = Linear(16, 48).cuda()
    x = torch.randn(2, 16, 8, 8, 64, device="cuda", requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = lin(x)
    assert y.dtype == torch.bfloat16 and y.shape == (2, 48, 8, 8, 64)
    y.float().pow(2).sum().backward()
    assert lin.linear.weight.grad.dtype == torch.float32 and lin.linear.weight.grad.shape == (48, 16, 1)
    assert lin.linear.bias.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
    # float32 tensors outside autocast take the same GEMM route in float32: the library
    # convolution's result to float32 rounding
    y32 = lin(x.detach())
    ref = F.conv1d(x.detach().double().flatten(2), lin.linear.weight.double(), lin.linear.bias.double()).view_as(y32)
    assert y32.dtype == torch.float32
    assert float((y32.double() - ref).abs().max() / ref.abs().max()) <= 1e-5
