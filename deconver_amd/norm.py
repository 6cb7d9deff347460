"""InstanceNorm for the Deconver networks on the HIP row-normalisation kernels.

The reference's blocks take their norm as a class (``norm1`` / ``norm2``, deconver.py:52-64)
and its segmentation networks pass ``nn.InstanceNorm2d`` / ``nn.InstanceNorm3d``: no affine
parameters, no running statistics.  On a channel-first tensor that is a normalisation of
``B * C`` contiguous rows.  PyTorch runs it as a batch norm with one workgroup per row, which
at the 3-D network's first level is 128 workgroups walking 2M elements each; the kernels behind
``ndc_rownorm_forward`` / ``ndc_rownorm_backward`` cut every row over many workgroups.

``InstanceNorm{1,2,3}d`` here are subclasses of the ``torch.nn`` modules with the same
constructor, parameters and state dict.  GPU tensors in float32 / bfloat16 without affine
parameters and running statistics take the kernels; anything else runs the parent's forward.
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
    def forward(self, x: Tensor) -> Tensor:
        if (self.affine or self.track_running_stats or not hip_norm_applies(x)
                or not _lib.library_available()):
            return super().forward(x)
        self._check_input_dim(x)
        if x.dim() == self._get_no_batch_dim():
            return super().forward(x)
        return instance_norm(x, self.eps)


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
