"""InstanceNorm for the Deconver networks on the HIP row-normalisation kernels.

The reference's blocks take their norm as a class (``norm1`` / ``norm2``, deconver.py:52-64)
and its segmentation networks pass ``nn.InstanceNorm2d`` / ``nn.InstanceNorm3d``: no affine
parameters, no running statistics.  On a channel-first tensor that is a normalisation of
``B * C`` contiguous rows.  PyTorch runs it as a batch norm with one workgroup per row, which
at the 3-D network's first level is 128 workgroups walking 2M elements each; the kernels behind
``ndc_rownorm_forward`` / ``ndc_rownorm_backward`` cut every row over many workgroups.

``InstanceNorm{1,2,3}d`` here are subclasses of the ``torch.nn`` modules with the same
constructor, parameters and state dict.  GPU tensors in float32 / bfloat16 without affine
parameters and running statistics take the kernels (a missing library raises, as for the NDC
update: there is no silent PyTorch path for them); anything else -- CPU tensors, float64,
affine or tracked statistics -- runs the parent's forward.
"""

from __future__ import annotations

import torch
from torch import Tensor, nn

from . import _lib, ops

__all__ = ["InstanceNorm1d", "InstanceNorm2d", "InstanceNorm3d", "instance_norm", "native_norm"]


class _RowNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, eps: float) -> Tensor:
        lib = _lib.get_library()
        x = x.contiguous()
        rows = x.shape[0] * x.shape[1]
        with torch.cuda.device(x.device):
            y, stats = ops.rownorm_forward(lib, x.view(rows, -1), eps)
        ctx.save_for_backward(y, stats)
        ctx.shape = x.shape
        return y.view(x.shape)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy: Tensor):
        y, stats = ctx.saved_tensors
        lib = _lib.get_library()
        gy = gy.contiguous().view(y.shape)
        with torch.cuda.device(y.device):
            gx = ops.rownorm_backward(lib, gy, y, stats)
        return gx.view(ctx.shape), None


class _RowNormSkip(torch.autograd.Function):
    """``(norm(x), x)``: the norm and the tensor it was taken of, for a pre-norm residual block
    ``x + f(norm(x))``.  In backward the gradient that arrives for the second output (the
    residual branch's) is summed into the norm's own input gradient by the kernel that writes
    it, instead of by a separate addition."""

    @staticmethod
    def forward(ctx, x: Tensor, eps: float):
        lib = _lib.get_library()
        xc = x.contiguous()
        rows = xc.shape[0] * xc.shape[1]
        with torch.cuda.device(xc.device):
            y, stats = ops.rownorm_forward(lib, xc.view(rows, -1), eps)
        ctx.save_for_backward(y, stats)
        ctx.shape = xc.shape
        ctx.set_materialize_grads(False)     # an unused output's gradient arrives as None
        return y.view(xc.shape), x.view_as(x)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy, gskip):
        y, stats = ctx.saved_tensors
        if gy is None:
            return gskip, None
        gy = gy.contiguous().view(y.shape)
        if gskip is not None:
            gskip = gskip.to(gy.dtype).contiguous().view(y.shape)
        with torch.cuda.device(y.device):
            gx = ops.rownorm_backward(_lib.get_library(), gy, y, stats, addend=gskip)
        return gx.view(ctx.shape), None


def hip_norm_applies(x: Tensor) -> bool:
    return (x.is_cuda and x.dim() >= 3 and x.dtype in (torch.float32, torch.bfloat16) and x.numel() > 0
            and x[0, 0].numel() > 1)


def instance_norm(x: Tensor, eps: float = 1e-5) -> Tensor:
    """``F.instance_norm(x, eps=eps)`` (no affine parameters, statistics of the input) on the
    HIP kernels; ``x`` is ``(B, C, *S)`` on the GPU, float32 or bfloat16."""
    if not hip_norm_applies(x):
        raise ValueError("instance_norm runs on GPU tensors (B, C, *S) in float32 or bfloat16")
    shape = x.shape
    return _RowNorm.apply(x, float(eps)).view(shape)


class _HipInstanceNorm:
    def _on_hip(self, x: Tensor) -> bool:
        return not (self.affine or self.track_running_stats or not hip_norm_applies(x)
                    or x.dim() == self._get_no_batch_dim())

    def forward(self, x: Tensor) -> Tensor:
        if not self._on_hip(x):
            return super().forward(x)
        self._check_input_dim(x)
        return instance_norm(x, self.eps)

    def with_skip(self, x: Tensor):
        """``(self(x), x)`` for a residual block ``x + f(self(x))``: use the second tensor as
        the residual term and the two gradients of ``x`` are summed inside the norm's backward
        kernel (on the HIP route; elsewhere it is ``x`` itself)."""
        if not self._on_hip(x) or not x.requires_grad:
            return self(x), x
        self._check_input_dim(x)
        return _RowNormSkip.apply(x, float(self.eps))


class InstanceNorm1d(_HipInstanceNorm, nn.InstanceNorm1d):
    pass


class InstanceNorm2d(_HipInstanceNorm, nn.InstanceNorm2d):
    pass


class InstanceNorm3d(_HipInstanceNorm, nn.InstanceNorm3d):
    pass


_NATIVE = {nn.InstanceNorm1d: InstanceNorm1d, nn.InstanceNorm2d: InstanceNorm2d,
           nn.InstanceNorm3d: InstanceNorm3d}


def native_norm(spec):
    """A norm spec (class or ``(class, kwargs)``) with ``torch.nn``'s InstanceNorm classes
    replaced by the subclasses above; everything else unchanged."""
    if isinstance(spec, (tuple, list)) and spec:
        return (native_norm(spec[0]), *spec[1:])
    try:
        return _NATIVE.get(spec, spec)
    except TypeError:      # unhashable spec
        return spec
