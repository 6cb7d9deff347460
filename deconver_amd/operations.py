"""PyTorch operations of the layer's GENERAL path (everything the HIP update does not cover:
``update_filter=True``, convolution keyword arguments, CPU tensors, float64, diagnostics).

Same call signatures and results as ``deconver/deconvolution/operations.py`` of the
reference (``conv``, ``sconv``, ``t``, ``flip``, ``norm2``, ``relative_error``,
``softmax``, ``kl_divergence``); written from the operator definitions, not from its code.
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch
import torch.nn.functional as F
from torch import Tensor

_CONVND = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}


def conv(input: Tensor, weight: Tensor, groups: int = 1, **kwargs) -> Tensor:
    """Per-sample grouped cross-correlation.

    ``input`` is ``(N, Cin, *S)`` and ``weight`` ``(N, Cout, Cin // groups, *k)``: sample
    ``n`` is filtered with ``weight[n]``.  All samples run as ONE convolution by stacking
    them along the channel axis and multiplying the group count by ``N``
    (operations.py:12-31 of the reference).
    """
    n, nd = input.shape[0], input.dim() - 2
    stacked = input.reshape(1, n * input.shape[1], *input.shape[2:])
    filters = weight.reshape(n * weight.shape[1], *weight.shape[2:])
    out = _CONVND[nd](stacked, filters, groups=n * groups, **kwargs)
    return out.reshape(n, -1, *out.shape[2:])


def sconv(input1: Tensor, input2: Tensor, **kwargs) -> Tensor:
    """Per-sample correlation of every channel of ``input1`` with every channel of ``input2``.

    ``input1`` is ``(N, C1, *S)``, ``input2`` ``(N, C2, *S)``; the result ``(N, C1, C2, *k)``
    holds, for a padding of ``k // 2``, ``sum_p input1[n,a,p+tau-pad] * input2[n,b,p]``
    (operations.py:43-49 of the reference, which vmaps a convolution whose "kernel" is the
    whole second volume).  Here the sample axis is folded into the group axis instead.
    """
    n, c1, nd = input1.shape[0], input1.shape[1], input1.dim() - 2
    c2 = input2.shape[1]
    lhs = input1.transpose(0, 1)                                    # (C1, N, *S): C1 "images"
    rhs = input2.reshape(n * c2, 1, *input2.shape[2:])              # N groups of C2 "filters"
    out = _CONVND[nd](lhs, rhs, groups=n, **kwargs)                 # (C1, N*C2, *k)
    out = out.reshape(c1, n, c2, *out.shape[2:])
    return out.permute(1, 0, 2, *range(3, 3 + nd))


def t(x: Tensor) -> Tensor:
    """Swap the output/input channel axes of a batched filter ``(N, out, in, *k)``."""
    return x.transpose(1, 2)


def flip(h: Tensor) -> Tensor:
    """Reverse the spatial axes of a batched filter ``(N, out, in, *k)``."""
    return torch.flip(h, dims=tuple(range(3 - h.ndim, 0)))


def softmax(x: Tensor, dim: int | Sequence[int]) -> Tensor:
    """Softmax taken jointly over one or several dimensions."""
    dims = [dim] if isinstance(dim, int) else list(dim)
    dims = [d % x.ndim for d in dims]
    if len(dims) == 1:
        return F.softmax(x, dim=dims[0])
    keep = [d for d in range(x.ndim) if d not in dims]
    order = keep + dims
    inverse = [order.index(d) for d in range(x.ndim)]
    moved = x.permute(order)
    flat = moved.flatten(start_dim=len(keep))
    return F.softmax(flat, dim=-1).view(moved.shape).permute(inverse)


def norm2(x: Tensor, w: Optional[Tensor] = None) -> Tensor:
    """Per-sample (optionally weighted) Euclidean norm of a ``(B, ...)`` tensor."""
    sq = x.flatten(1).square()
    if w is not None:
        sq = sq * w.flatten(1)
    return sq.sum(dim=1).sqrt()


def relative_error(x: Tensor, y: Tensor, w: Optional[Tensor] = None, eps: float = 1e-16) -> Tensor:
    """Per-sample ``(|x - y| + eps) / (|x| + eps)`` in the (weighted) Euclidean norm."""
    return (norm2(x - y, w) + eps) / (norm2(x, w) + eps)


def kl_divergence(x: Tensor, y: Tensor, eps: float = 1e-16) -> Tensor:
    """Per-sample mean generalised KL divergence ``x log(x/y) - x + y`` of clamped inputs."""
    x = x.clamp(min=eps)
    y = y.clamp(min=eps)
    return (x * torch.log(x / y) - x + y).flatten(1).mean(-1)
