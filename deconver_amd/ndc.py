"""The NDC layer (``Deconv``, alias ``NDC``) and its learned initialiser.

API-compatible with ``deconver/deconvolution/deconv.py`` of the reference -- constructor
arguments, public attributes, the overridable methods ``update_s / update_h / update /
context / iterative_update``, ``fit / reconstruct / loss / normalize_h /
fast_path_applicable``, and the state-dict keys ``init.h0``,
``init.linear.linear.weight``, ``init.linear.linear.bias`` -- so that reference checkpoints
load with ``strict=True``.

Execution
---------
``forward`` asks ``fast_path_applicable(x)`` and then runs one of two routes:

HIP route
    One autograd node per iteration, on ``libdeconver_ndc.so``
    (``functional.projected_update``, which holds the projection too, then
    ``functional.deconv_update``).  Taken for GPU tensors in float32 or bfloat16 (bfloat16 also
    under autocast, which the reference declines at deconv.py:139-147) when the layer is in
    its default regime: source updates only, odd kernel, no extra convolution arguments, no
    overridden update methods.  The projection runs as a bias-free 1x1 GEMM; its bias and
    the ReLU are applied by the kernels while loading.
general route
    The layer written out in PyTorch ops (``operations.py``): filter updates, verbose
    diagnostics, convolution keyword arguments, CPU tensors, float64.
"""

from __future__ import annotations

import contextlib
import functools
import math
from typing import Any, Optional, Sequence

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import operations as ops_general
from . import ops
from ._lib import get_library
from .functional import deconv_update, hip_kernels_apply, projected_update
from .layers import Linear

__all__ = ["Initializer", "Deconv", "NDC"]

_HIP_DTYPES = (torch.float32, torch.bfloat16)
_ROUTED_METHODS = ("update_s", "update", "iterative_update")


class Initializer(nn.Module):
    """``x -> (relu(W x + b), relu(h0) broadcast over the batch)`` (deconv.py:20-45).

    ``h0`` is created before the projection, which fixes the order in which a seeded
    generator is consumed.
    """

    def __init__(self, channels: int, source_channels: int, kernel_size: Sequence[int],
                 groups: int) -> None:
        super().__init__()
        if groups is None:
            groups = channels
        assert channels % groups == 0, "`channels` must be divisible by groups"
        self.h0 = nn.Parameter(
            nn.init.kaiming_uniform_(torch.empty(channels, source_channels, *kernel_size),
                                     a=math.sqrt(5)))
        self.linear = Linear(channels, groups * source_channels)

    def forward(self, x: Tensor) -> tuple[Tensor, Tensor]:
        batched_h = self.h0.expand(x.shape[0], *self.h0.shape)
        return F.relu(self.linear(x)), F.relu(batched_h)


def _fold_groups(groups: int, x: Tensor) -> Tensor:
    """``b (g c) ... -> (b g) c ...``: every (sample, group) becomes its own problem."""
    return x.reshape(x.shape[0] * groups, x.shape[1] // groups, *x.shape[2:])


def _unfold_groups(groups: int, x: Tensor) -> Tensor:
    """``(b g) c ... -> b (g c) ...``"""
    return x.reshape(x.shape[0] // groups, groups * x.shape[1], *x.shape[2:])


class Deconv(nn.Module):
    """Fits a non-negative source ``s`` with ``x ~ conv(s, h)`` by multiplicative updates
    that start from a learned initialisation; returns ``s`` of shape ``(B, G*sc, *S)``."""

    def __init__(self, channels: int, kernel_size=Sequence[int],
                 source_channels: Optional[int] = None, ratio: float = 1, groups: int = -1,
                 update_source=True, update_filter=False, eps: float = 1e-16,
                 num_iters: int = 1, num_grad_iters: Optional[int] = None,
                 verbose: bool = False, **kwargs) -> None:
        super().__init__()
        groups = channels if groups == -1 else groups
        assert channels % groups == 0, "`channels` must be divisible by groups"
        if source_channels is None:
            source_channels = channels * ratio / groups
        self.channels, self.groups = channels, groups
        self.source_channels = round(source_channels)
        self.filter_channels = channels // groups
        self.kernel_size = kernel_size
        self.update_source, self.update_filter = update_source, update_filter
        self.num_iters = num_iters
        self.num_grad_iters = num_iters if num_grad_iters is None else num_grad_iters
        self.eps, self.verbose = eps, verbose
        self.init = Initializer(channels, self.source_channels, kernel_size, groups)

        same_pad = tuple(k // 2 for k in kernel_size)
        self._conv_kwargs = dict(kwargs)
        self.conv = functools.partial(ops_general.conv, padding=same_pad, **kwargs)
        self.sconv = functools.partial(ops_general.sconv, padding=same_pad, **kwargs)
        self.split_channels = functools.partial(_fold_groups, groups)
        self.merge_channels = functools.partial(_unfold_groups, groups)

    # ------------------------------------------------------------------ route choice

    def _regime_allows_hip(self) -> bool:
        """Input-independent part of the route choice (deconv.py:122-135)."""
        if self.update_filter or not self.update_source or self.verbose or self._conv_kwargs:
            return False
        if self.num_iters < 1 or any(k % 2 == 0 for k in self.kernel_size):
            return False
        if not self._hip_is_ahead():
            return False
        # a subclass that overrides a method the HIP route would bypass gets the general route
        if any(getattr(type(self), name) is not getattr(Deconv, name) for name in _ROUTED_METHODS):
            return False
        return type(self.init).forward is Initializer.forward

    def _hip_is_ahead(self) -> bool:
        """Whether the HIP kernels are the faster route for this filter geometry.

        The kernels are built for the depthwise / few-channels-per-group stencils the network
        uses.  With many filter and source channels per group the update is GEMM-shaped work
        that the library convolutions of the general route do better: on an MI355X (16
        channels, 24^3, batch 2, forward + backward) the HIP route is 1.1x-9x ahead up to
        the bounds below and 0.35x-0.65x behind past them.  The reference keeps its fused
        route to a similar envelope (``kernels.py:137-163``) and falls back wherever it is
        not measurably ahead.
        """
        taps = math.prod(self.kernel_size)
        per_source = self.source_channels * taps
        return per_source <= 3000 and self.filter_channels * per_source <= 30000

    def _differentiates(self, x: Tensor) -> bool:
        """Whether autograd will record this call (so a backward may follow)."""
        return torch.is_grad_enabled() and (
            x.requires_grad or any(p.requires_grad for p in self.parameters()))

    @staticmethod
    def _hip_dtype(x: Tensor) -> Optional[torch.dtype]:
        """Activation dtype the HIP route would store ``x`` in, or None if there is none."""
        if not x.is_cuda:
            return None
        try:
            if torch.is_autocast_enabled(x.device.type):
                dtype = torch.get_autocast_dtype(x.device.type)
                return dtype if dtype == torch.bfloat16 else None
        except (TypeError, RuntimeError):  # pragma: no cover - device types without autocast
            pass
        return x.dtype if x.dtype in _HIP_DTYPES else None

    def fast_path_applicable(self, x: Optional[Tensor] = None) -> bool:
        """Whether ``forward(x)`` (or, with ``x=None``, the configuration alone) takes the
        HIP route.  Raises if the route applies but the HIP library has not been built."""
        if not self._regime_allows_hip():
            return False
        if x is None:
            return True
        dtype = self._hip_dtype(x)
        if dtype is None or x.dim() - 2 != len(self.kernel_size):
            return False
        # forward-only calls: with many source channels per group the library convolutions
        # are ahead (0.44x-0.94x measured); once a backward follows the HIP route wins again
        if self.source_channels >= 16 and self.filter_channels >= 4 and not self._differentiates(x):
            return False
        return hip_kernels_apply(x, self.filter_channels, self.source_channels,
                                 self.kernel_size, dtype)

    # ------------------------------------------------------------------ HIP route

    def _fit_fast(self, x: Tensor, rectified_input: bool = False) -> tuple[Tensor, Tensor]:
        dtype = self._hip_dtype(x)
        x = x.contiguous().to(dtype)
        proj = self.init.linear.linear
        h = F.relu(self.init.h0).float()
        # bias-free projection; bias and ReLU are folded into the first update's loads, so
        # neither relu(Linear(x)) nor the biased projection ever exists in memory.  Projection
        # and first update are one autograd node: both read x, and the node's backward
        # accumulates the projection's input gradient onto the update's
        weight = proj.weight.squeeze(-1) if proj.weight.dim() == 3 else proj.weight
        bias = None if proj.bias is None else proj.bias.float()
        kwargs = dict(groups=self.groups, m=self.filter_channels, sc=self.source_channels,
                      eps=self.eps)
        if self.num_iters > 1:   # one filter table for all iterations (a single one makes its own)
            with torch.no_grad(), torch.cuda.device(x.device):
                kwargs["taps"] = ops.prepare_taps(
                    get_library(), x, h.detach().contiguous(), groups=self.groups,
                    m=self.filter_channels, sc=self.source_channels)
        s = None
        for it in range(1, self.num_iters + 1):
            with self.context(it):
                if it == 1:
                    s = projected_update(x, weight, h, bias, rectified_input=rectified_input, **kwargs)
                else:
                    s = deconv_update(x, s, h, None, relu_input=False, **kwargs)
        return s, h

    # ------------------------------------------------------------------ general route

    def normalize_h(self, h: Tensor) -> Tensor:
        """Scale every (sample, input-channel) slice of the filter to unit sum."""
        reduce_over = [d for d in range(h.ndim) if d not in (0, 2)]
        return (h + self.eps) / (h.sum(reduce_over, keepdim=True) + self.eps)

    def update_s(self, x: Tensor, s: Tensor, h: Tensor) -> Tensor:
        """``s <- s * (A x + eps) / (A K s + eps)`` with ``K = conv(., h)``, ``A = K^T``."""
        adjoint = ops_general.t(ops_general.flip(h))
        return s * (self.conv(x, adjoint) + self.eps) / (
            self.conv(self.conv(s, h), adjoint) + self.eps)

    def update_h(self, x: Tensor, s: Tensor, h: Tensor) -> Tensor:
        """The same multiplicative rule for the filter, with the roles of s and h swapped."""
        ratio = (self.sconv(s, x) + self.eps) / (self.sconv(s, self.conv(s, h)) + self.eps)
        return h * ops_general.t(ratio)

    def update(self, x: Tensor, s: Tensor, h: Tensor) -> tuple[Tensor, Tensor]:
        s = self.update_s(x, s, h) if self.update_source else s
        h = self.update_h(x, s, h) if self.update_filter else h
        return s, h

    def context(self, it: int) -> Any:
        """Iterations ``1 .. num_iters - num_grad_iters`` run without autograd."""
        truncated = it <= self.num_iters - self.num_grad_iters
        return torch.no_grad() if truncated else contextlib.nullcontext()

    def iterative_update(self, x: Tensor, s: Tensor, h: Tensor) -> tuple[Tensor, Tensor]:
        for it in range(1, self.num_iters + 1):
            with self.context(it):
                if self.verbose:
                    print(f"iter {it}: loss = {self.loss(x, s, h)}")
                s, h = self.update(x, s, h)
        return s, h

    def _fit_general(self, x: Tensor) -> tuple[Tensor, Tensor]:
        s, h = self.init(x)
        grouped = self.groups != 1
        if grouped:
            x, s, h = (self.split_channels(v) for v in (x, s, h))
        s, h = self.iterative_update(x, s, h)
        if grouped:
            s, h = self.merge_channels(s), self.merge_channels(h)
        return s, h

    # ------------------------------------------------------------------ interface

    def fit(self, x: Tensor) -> tuple[Tensor, Tensor]:
        """``(s, h)`` with ``h`` in its batched form ``(B, C, sc, *k)``, contiguous."""
        if not self.fast_path_applicable(x):
            return self._fit_general(x)
        s, h = self._fit_fast(x)
        return s, h.expand(x.shape[0], *h.shape).contiguous()

    def reconstruct(self, s: Tensor, h: Tensor) -> Tensor:
        """``conv(s, h)`` for merged-channel ``s`` and batched ``h``."""
        if self.groups == 1:
            return self.conv(s, h)
        return self.merge_channels(self.conv(self.split_channels(s), self.split_channels(h)))

    def loss(self, x: Tensor, s: Tensor, h: Tensor) -> Tensor:
        """Relative reconstruction error; takes channel-split tensors, as
        ``iterative_update`` passes them."""
        return ops_general.relative_error(x, self.conv(s, h))

    def forward(self, x: Tensor, rectified_input: bool = False) -> Tensor:
        """The layer's sources.  ``rectified_input`` (not in the reference; see
        ``takes_rectified_input``): ``x`` is a rectifier's output whose producer leaves that
        rectifier's backward to this layer."""
        if rectified_input and not self.takes_rectified_input(x):
            # the producer has already dropped its rectifier's backward: refusing is the only
            # answer that cannot return a wrong gradient
            raise RuntimeError("Deconv.forward(rectified_input=True) on a call that takes_rectified_input() declines")
        if self.fast_path_applicable(x):
            return self._fit_fast(x, rectified_input)[0]
        return self._fit_general(x)[0]

    def takes_rectified_input(self, x: Tensor) -> bool:
        """Whether ``forward(x, rectified_input=True)`` returns the gradient of ``x`` already
        zero where ``x`` is: the HIP route with a single update, whose one node forms that
        gradient in a GEMM.  A caller that rectifies ``x`` may then skip the rectifier's own
        backward pass; otherwise it must not."""
        if self.num_iters != 1 or not self.fast_path_applicable(x) or self._hip_dtype(x) != torch.bfloat16:
            return False
        # ... and that GEMM is the library's own, which masks in its epilogue (elsewhere the
        # mask would be a pass of its own again)
        n = math.prod(x.shape[2:])
        return get_library().pointwise_gemm_supported(self.groups * self.source_channels, self.channels, n,
                                                      ops.dtype_tag(torch.bfloat16))


NDC = Deconv
