"""Row normalisation (ndc_rownorm_forward / ndc_rownorm_backward, the InstanceNorm of the
Deconver blocks) against torch's instance norm in float64 on the same inputs.

CPU tests run the host build of the library (same splitting and formulas, sequential); GPU tests
run the HIP kernels through the C ABI and through the module.  Bars: float32 1e-5 of the largest
entry (the statistics are float32 sums over up to millions of elements), bfloat16 2e-2."""

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import deconver_amd as dc
from deconver_amd import _lib, norm, ops
from tests.helpers import hostcheck_library


def _reference(x, gy, eps):
    x64 = x.double().requires_grad_(True)
    y = F.instance_norm(x64.unsqueeze(0), eps=eps)[0]
    (gx,) = torch.autograd.grad(y, x64, gy.double())
    return y.detach(), gx


def _rel(a, b):
    return float((a.double() - b).abs().max() / b.abs().max().clamp_min(1e-30))


def _run(lib, x, gy, eps):
    y, stats = ops.rownorm_forward(lib, x, eps)
    gx = ops.rownorm_backward(lib, gy, y, stats)
    # with an addend: the same plus that tensor (one rounding of the sum)
    extra = torch.flip(gy, (1,))
    gx2 = ops.rownorm_backward(lib, gy, y, stats, addend=extra)
    tol = 1e-6 if x.dtype == torch.float32 else 1e-2
    torch.testing.assert_close(gx2.float(), gx.float() + extra.float(), rtol=tol, atol=tol * float(gy.abs().max()))
    return y, stats, gx


# (rows, n): one part; several parts with a ragged last one; not a multiple of the vector width
SHAPES = [(3, 7), (5, 64), (2, 8192 * 3 + 8), (1, 2048 * 9 + 3), (4, 20000),
          # around the split's thresholds (parts of at least 8 192 elements, multiples of 2 048)
          (1, 8191), (1, 8192), (2, 16383), (1, 16384), (1, 16385), (1, 2 * 8192 + 2048 + 8), (3, 5)]


@pytest.mark.parametrize("rows,n", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_host_build_matches_instance_norm(rows, n, dtype):
    lib = hostcheck_library()
    gen = torch.Generator().manual_seed(rows * 1000 + n)
    x = (torch.randn(rows, n, generator=gen) * 1.7 + 3.0).to(dtype)
    gy = torch.randn(rows, n, generator=gen).to(dtype)
    y, stats, gx = _run(lib, x, gy, 1e-5)
    y_ref, gx_ref = _reference(x, gy, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert _rel(y, y_ref) <= tol
    assert _rel(gx, gx_ref) <= tol
    xd = x.double()
    torch.testing.assert_close(stats[:, 0].double(), xd.mean(1), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(stats[:, 1].double(), (xd.var(1, unbiased=False) + 1e-5).rsqrt(), rtol=1e-4, atol=0)


def test_large_offset_does_not_cancel():
    """mean / std = 1000: the shifted sums keep the variance; a plain E[x^2] - mean^2 in
    float32 would lose it."""
    lib = hostcheck_library()
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(2, 30000, generator=gen) + 1000.0
    y, stats = ops.rownorm_forward(lib, x, 1e-5)
    y_ref = F.instance_norm(x.double().unsqueeze(0), eps=1e-5)[0]
    assert _rel(y, y_ref) <= 1e-3          # x itself carries 6e-5 of rounding at this offset
    torch.testing.assert_close(stats[:, 1].double(), (x.double().var(1, unbiased=False) + 1e-5).rsqrt(),
                               rtol=1e-4, atol=0)


def test_constant_rows_and_bad_arguments():
    lib = hostcheck_library()
    x = torch.full((2, 100), 3.5)
    y, stats = ops.rownorm_forward(lib, x, 1e-5)
    assert bool((y == 0).all()) and torch.allclose(stats[:, 0], torch.tensor(3.5))
    assert lib.rownorm_workspace_bytes(128, 128 ** 3) == 128 * 32 * 8
    assert lib.rownorm_workspace_bytes(4096, 4096) == 4096 * 8
    ws = torch.empty(64)
    with pytest.raises(_lib.NdcError):     # workspace too small
        lib.rownorm_forward(x.data_ptr(), y.data_ptr(), stats.data_ptr(), 2, 100, _lib.NDC_F32, 1e-5,
                            ws.data_ptr(), 8, None)
    with pytest.raises(_lib.NdcError):     # in place
        lib.rownorm_forward(x.data_ptr(), x.data_ptr(), stats.data_ptr(), 2, 100, _lib.NDC_F32, 1e-5,
                            ws.data_ptr(), 256, None)
    with pytest.raises(_lib.NdcError):     # unknown dtype
        lib.rownorm_forward(x.data_ptr(), y.data_ptr(), stats.data_ptr(), 2, 100, 7, 1e-5,
                            ws.data_ptr(), 256, None)
    with pytest.raises(_lib.NdcError):
        lib.rownorm_forward(None, y.data_ptr(), stats.data_ptr(), 2, 100, _lib.NDC_F32, 1e-5,
                            ws.data_ptr(), 256, None)


def test_modules_are_the_torch_modules_off_the_gpu():
    """Same class hierarchy, constructor and state dict; on the CPU, with affine parameters or
    with running statistics the parent's forward runs."""
    for cls, parent, shape in ((dc.InstanceNorm2d, nn.InstanceNorm2d, (2, 3, 5, 6)),
                               (dc.InstanceNorm3d, nn.InstanceNorm3d, (2, 3, 4, 5, 6)),
                               (dc.InstanceNorm1d, nn.InstanceNorm1d, (2, 3, 9))):
        x = torch.randn(*shape)
        m, ref = cls(3), parent(3)
        assert isinstance(m, parent) and m.state_dict().keys() == ref.state_dict().keys()
        assert torch.equal(m(x), ref(x))
        m2 = cls(3, affine=True, track_running_stats=True)
        assert set(m2.state_dict()) == set(parent(3, affine=True, track_running_stats=True).state_dict())
    assert norm.native_norm(nn.InstanceNorm3d) is dc.InstanceNorm3d
    assert norm.native_norm((nn.InstanceNorm2d, {"eps": 1e-3}))[0] is dc.InstanceNorm2d
    assert norm.native_norm(nn.BatchNorm2d) is nn.BatchNorm2d
    assert norm.native_norm(dc.LayerNorm) is dc.LayerNorm
    net = dc.Deconver(in_channels=1, out_channels=1, spatial_dims=2, encoder_depth=(1, 1), encoder_width=(4, 8),
                      strides=(1, 2), decoder_depth=(1,), kernel_size=(3, 3), ratio=2, norm=nn.InstanceNorm2d)
    blk = net.encoder.blocks[0].block.blocks[0]
    assert isinstance(blk.norm1, dc.InstanceNorm2d) and isinstance(blk.norm2, nn.InstanceNorm2d)


GPU_SHAPES = [((2, 3, 5, 7), 1e-5), ((2, 64, 32, 32, 32), 1e-5), ((1, 5, 33, 17, 9), 1e-3),
              ((2, 4, 128, 128, 64), 1e-5), ((3, 130, 8, 8, 8), 1e-5)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape,eps", GPU_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hip_module_matches_instance_norm(shape, eps, dtype):
    gen = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=gen) * 1.3 + 0.7).to(dtype)
    gy = torch.randn(*shape, generator=gen).to(dtype)
    y_ref, gx_ref = _reference(x.flatten(0, 1).flatten(1), gy.flatten(0, 1).flatten(1), eps)
    xg = x.cuda().requires_grad_(True)
    m = getattr(dc, f"InstanceNorm{len(shape) - 2}d")(shape[1], eps=eps)
    y = m(xg)
    (gx,) = torch.autograd.grad(y, xg, gy.cuda())
    assert y.dtype == dtype and y.shape == x.shape and gx.shape == x.shape
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert _rel(y.cpu().flatten(0, 1).flatten(1), y_ref) <= tol
    assert _rel(gx.cpu().flatten(0, 1).flatten(1), gx_ref) <= tol
    # and against torch's own kernels on the same device tensor
    x2 = x.cuda().requires_grad_(True)
    y2 = F.instance_norm(x2, eps=eps)
    (gx2,) = torch.autograd.grad(y2, x2, gy.cuda())
    assert _rel(y.cpu(), y2.double().cpu()) <= tol and _rel(gx.cpu(), gx2.double().cpu()) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_with_skip_sums_the_two_gradients(dtype):
    """x + f(norm(x)) through ``with_skip``: the gradient of x is the norm's plus the residual
    branch's, as autograd would have summed them."""
    torch.manual_seed(7)
    shape = (2, 6, 16, 8, 40)
    x = torch.randn(*shape, device="cuda").to(dtype).requires_grad_(True)
    w = torch.randn(*shape, device="cuda").to(dtype)
    g = torch.randn(*shape, device="cuda").to(dtype)
    m = dc.InstanceNorm3d(6)
    y, xs = m.with_skip(x)
    (gx,) = torch.autograd.grad(xs + y * w, x, g)
    x64 = x.detach().double().requires_grad_(True)
    ref = x64 + F.instance_norm(x64) * w.double()
    (gx_ref,) = torch.autograd.grad(ref, x64, g.double())
    assert _rel(gx.cpu(), gx_ref.cpu()) <= (1e-5 if dtype == torch.float32 else 2e-2)
    # only one of the two outputs used
    y, xs = m.with_skip(x)
    (ga,) = torch.autograd.grad(y * w, x, g)
    (gb,) = torch.autograd.grad(m(x) * w, x, g)
    assert torch.equal(ga, gb)
    y, xs = m.with_skip(x)
    (gc,) = torch.autograd.grad(xs * w, x, g)
    assert torch.equal(gc, (g * w))


@pytest.mark.gpu
def test_hip_rownorm_is_reproducible_and_handles_views():
    x = torch.randn(2, 6, 16, 16, 16, device="cuda")
    a = dc.instance_norm(x)
    b = dc.instance_norm(x)
    assert torch.equal(a, b)
    xt = x.transpose(2, 4)               # not contiguous: copied first
    ref = F.instance_norm(xt.double())
    assert _rel(dc.instance_norm(xt).cpu(), ref.cpu()) <= 1e-5


@pytest.mark.gpu
def test_full_size_rows_of_the_3d_network():
    """The first level of the 3-D network (B 2, 64 channels, 128^3, bf16: 128 rows of 2 M
    elements, cut into 32 parts each) through size-independent properties: normalised rows have
    zero mean and unit variance, the gradient is orthogonal to the constant and to the
    normalised row (the two directions the norm removes), and sampled rows agree with float64."""
    torch.manual_seed(11)
    B, C, n = 2, 64, 128 ** 3
    lib = _lib.get_library()
    x = (torch.randn(B * C, n, device="cuda") * 0.8 + 0.3).bfloat16()
    gy = torch.randn(B * C, n, device="cuda").bfloat16()
    assert lib.rownorm_workspace_bytes(B * C, n) == B * C * 32 * 8
    y, stats = ops.rownorm_forward(lib, x, 1e-5)
    gx = ops.rownorm_backward(lib, gy, y, stats)
    yf, gf = y.float(), gx.float()
    assert float(yf.mean(1).abs().max()) <= 2e-3           # bf16 rounding of y leaves ~1e-4
    assert float((yf.var(1, unbiased=False) - 1).abs().max()) <= 5e-3
    scale = float(gf.abs().mean())
    assert float(gf.mean(1).abs().max()) <= 2e-3 * scale
    assert float((gf * yf).mean(1).abs().max()) <= 5e-3 * scale
    for row in (0, 77, 127):
        y_ref, gx_ref = _reference(x[row:row + 1].cpu(), gy[row:row + 1].cpu(), 1e-5)
        assert _rel(y[row:row + 1].cpu(), y_ref) <= 2e-2
        assert _rel(gx[row:row + 1].cpu(), gx_ref) <= 2e-2
        torch.testing.assert_close(stats[row, 0].double().cpu(), x[row].double().mean().cpu(), rtol=1e-4, atol=1e-5)
