"""Normalisation over the channel axis of a channel-first tensor (ndc_chnorm_forward /
ndc_chnorm_backward: the reference's LayerNorm, layers/norm.py:25-34) against ``nn.LayerNorm``
applied with the channel axis moved last, in float64 on the same inputs.

CPU tests run the host build of the library; GPU tests the HIP kernels, through the C ABI and
through the module.  Bars: float32 1e-5 of the largest entry, bfloat16 2e-2."""

import pytest
import torch
import torch.nn.functional as F

import deconver_amd as dc
from deconver_amd import _lib, ops
from tests.helpers import hostcheck_library


def _rel(a, b):
    return float((a.detach().double() - b.detach().double()).abs().max() / b.detach().double().abs().max().clamp_min(1e-30))


def _reference(x, gy, w, b, eps):
    x64 = x.double().requires_grad_(True)
    w64 = None if w is None else w.double().requires_grad_(True)
    b64 = None if b is None else b.double().requires_grad_(True)
    y = F.layer_norm(x64.movedim(1, -1), (x.shape[1],), w64, b64, eps).movedim(-1, 1)
    leaves = [t for t in (x64, w64, b64) if t is not None]
    grads = torch.autograd.grad(y, leaves, gy.double())
    gx = grads[0]
    gw = grads[1] if w is not None else None
    gb = grads[-1] if b is not None else None
    return y.detach(), gx, gw, gb


def _check(lib, shape, dtype, affine, device="cpu"):
    gen = torch.Generator().manual_seed(sum(shape) + affine)
    x = (torch.randn(*shape, generator=gen) * 1.5 + 0.8).to(dtype).to(device)
    gy = torch.randn(*shape, generator=gen).to(dtype).to(device)
    w = (torch.rand(shape[1], generator=gen) + 0.5).to(device) if affine else None
    b = (torch.rand(shape[1], generator=gen) - 0.5).to(device) if affine else None
    y, stats = ops.chnorm_forward(lib, x, w, b, 1e-5)
    gx, gw, gb = ops.chnorm_backward(lib, gy, x, stats, w)
    y_ref, gx_ref, gw_ref, gb_ref = _reference(x, gy, w, b, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert _rel(y, y_ref) <= tol and _rel(gx, gx_ref) <= tol
    xd = x.double()
    torch.testing.assert_close(stats[:, 0].double(), xd.mean(1), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(stats[:, 1].double(), (xd.var(1, unbiased=False) + 1e-5).rsqrt(), rtol=1e-4, atol=0)
    if affine:
        # the affine gradients are float32 sums of unrounded terms over batch and voxels
        assert gw.dtype == torch.float32 and _rel(gw, gw_ref) <= max(tol, 1e-4)
        assert _rel(gb, gb_ref) <= max(tol, 1e-4)
    else:
        # without weights the same sums are still those of g * xhat and g
        assert _rel(gb, gy.double().sum((0, 2))) <= max(tol, 1e-4)
    gx2, none_w, none_b = ops.chnorm_backward(lib, gy, x, stats, w, need_affine_grads=False)
    assert none_w is None and none_b is None and torch.equal(gx, gx2)


# (B, C, n): one vector per thread and several; rows that are not whole 16-byte vectors; one channel
SHAPES = [(2, 3, 8), (1, 5, 64), (2, 4, 2048 + 8), (1, 7, 1027), (3, 1, 16), (2, 16, 300)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("affine", [True, False])
def test_host_build_matches_layer_norm(shape, dtype, affine):
    if shape[1] == 1:
        pytest.skip("one channel: the output is the bias and the gradient vanishes; see below")
    _check(hostcheck_library(), shape, dtype, affine)


def test_one_channel_and_bad_arguments():
    lib = hostcheck_library()
    x = torch.randn(3, 1, 16)
    b = torch.tensor([0.25])
    y, stats = ops.chnorm_forward(lib, x, torch.ones(1), b, 1e-5)
    assert torch.allclose(y, torch.full_like(y, 0.25)) and torch.allclose(stats[:, 0], x[:, 0])
    assert lib.chnorm_parts(2, 128 ** 3, _lib.NDC_BF16) == 2 * (128 ** 3 // 8 // 256) * 4   # 16-byte accesses
    assert lib.chnorm_parts(2, 4096, _lib.NDC_BF16) == 2 * (4096 // 256) * 4                # a small grid: one voxel per thread
    assert lib.chnorm_parts(1, 7, _lib.NDC_F32) == 4
    with pytest.raises(_lib.NdcError):   # in place
        lib.chnorm_forward(x.data_ptr(), None, None, x.data_ptr(), stats.data_ptr(), 3, 1, 16, _lib.NDC_F32, 1e-5, None)
    with pytest.raises(_lib.NdcError):
        lib.chnorm_forward(x.data_ptr(), None, None, y.data_ptr(), stats.data_ptr(), 3, 1, 16, 5, 1e-5, None)
    with pytest.raises(_lib.NdcError):
        lib.chnorm_forward(None, None, None, y.data_ptr(), stats.data_ptr(), 3, 1, 16, _lib.NDC_F32, 1e-5, None)
    with pytest.raises(ValueError):
        ops.chnorm_forward(lib, x, torch.ones(2), None, 1e-5)


def test_module_is_the_reference_form_off_the_gpu():
    """On the CPU ``LayerNorm`` is the reference's movedim form around ``nn.LayerNorm``; the
    state dict is ``norm.weight`` / ``norm.bias``."""
    torch.manual_seed(0)
    ln = dc.LayerNorm(6)
    x = torch.randn(2, 6, 5, 7)
    assert torch.equal(ln(x), ln.norm(x.movedim(1, -1)).movedim(-1, 1))
    assert set(ln.state_dict()) == {"norm.weight", "norm.bias"}


GPU_SHAPES = [(2, 8, 6, 10), (2, 64, 8, 12, 16), (1, 5, 7, 9), (2, 32, 64, 64), (1, 130, 4, 6, 8),
              (2, 16, 64, 64, 64)]   # the last one large enough for 16-byte accesses


@pytest.mark.gpu
@pytest.mark.parametrize("shape", GPU_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("affine", [True, False])
def test_hip_kernels_match_layer_norm(shape, dtype, affine):
    flat = (shape[0], shape[1], int(torch.tensor(shape[2:]).prod()))
    _check(_lib.get_library(), flat, dtype, affine, device="cuda")


@pytest.mark.gpu
@pytest.mark.parametrize("regime", ["float32", "bfloat16", "bf16 autocast"])
@pytest.mark.parametrize("shape", [(2, 8, 6, 10), (2, 64, 16, 24, 48), (1, 5, 7, 9), (2, 16, 64, 64, 64)])
def test_module_matches_the_reference_form_on_the_gpu(regime, shape):
    """``dc.LayerNorm`` on the GPU against the reference's movedim form around the same
    ``nn.LayerNorm`` (PyTorch's kernels): values, input gradient and parameter gradients; under
    autocast both are float32, as PyTorch's autocast rules make layer norm."""
    import contextlib
    torch.manual_seed(sum(shape))
    ln = dc.LayerNorm(shape[1]).cuda()
    with torch.no_grad():
        ln.norm.weight.uniform_(0.5, 1.5)
        ln.norm.bias.uniform_(-0.5, 0.5)
    dtype = torch.bfloat16 if regime == "bfloat16" else torch.float32
    if regime == "bfloat16":
        ln = ln.bfloat16()
    x = torch.randn(*shape, device="cuda").to(dtype).requires_grad_(True)
    g = torch.randn(*shape, device="cuda")
    ctx = (lambda: torch.autocast("cuda", dtype=torch.bfloat16)) if regime == "bf16 autocast" else contextlib.nullcontext
    with ctx():
        y = ln(x)
        ref = ln.norm(x.movedim(1, -1)).movedim(-1, 1)
    assert y.shape == x.shape and y.dtype == ref.dtype
    on_kernels = shape[0] * int(torch.tensor(shape[2:]).prod()) >= 32768   # smaller grids keep the reference form
    assert y.is_contiguous() == on_kernels
    params = (x, ln.norm.weight, ln.norm.bias)
    got = torch.autograd.grad(y, params, g.to(y.dtype))
    want = torch.autograd.grad(ref, params, g.to(y.dtype))
    tol = 2e-2 if regime == "bfloat16" else 1e-5
    assert _rel(y, ref) <= tol
    for a, r in zip(got, want):
        assert a.dtype == r.dtype and _rel(a, r) <= max(tol, 1e-4)


@pytest.mark.gpu
def test_default_norm_block_on_the_gpu_matches_its_float64_general_route():
    """A Deconver block with the reference's default norm (LayerNorm) under bf16 autocast
    against the same block in float64 on the CPU."""
    torch.manual_seed(6)
    blk = dc.DeconverBlock(16, kernel_size=(3, 3, 3), ratio=4)
    assert isinstance(blk.norm1, dc.LayerNorm)
    x = torch.rand(2, 16, 24, 32, 32)      # enough voxels for the module to take the kernels
    ref = blk.double()(x.double())
    blk = blk.float().cuda()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = blk(x.cuda())
    assert _rel(y.cpu(), ref) <= 2e-2
