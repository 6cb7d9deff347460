"""Autograd node of one NDC source update, running on the HIP kernels.

Mirrors ``deconver/deconvolution/functional.py:97-207`` of the reference
(``DeconvUpdate`` / ``deconv_update``): same arguments, same returned gradients
``(gx, gz, gh, gb, None x5)``, same refusal of double backward.  It saves the reference's
``(x, z, t1, h, bias)`` plus, unless ``save_ratio(False)`` was called, the forward's
``s/(A(t1)+eps)`` and ``(A(x)+eps)/(A(t1)+eps)``: two tensors of the size of the output
kept until backward, which then does not gather ``A(x)`` and ``A(t1)`` a second time.
The arithmetic is in ``libdeconver_ndc.so``; there is no PyTorch implementation behind
this node.
"""

from __future__ import annotations

import os
from typing import Optional

import torch
from torch import Tensor

from . import _lib, ops

__all__ = ["deconv_update", "projected_update", "hip_kernels_apply", "DeconvUpdate", "ProjectedUpdate",
           "save_ratio", "matrix_kernels"]

_SAVE_RATIO = os.environ.get("DECONVER_NDC_SAVE_RATIO", "1") != "0"


def save_ratio(enabled: Optional[bool] = None) -> bool:
    """Get or set whether training keeps the forward's denominator and ratio for backward.

    On (the default; environment ``DECONVER_NDC_SAVE_RATIO=0`` turns it off): each update
    node holds two more tensors of the size of its output until backward, and backward is
    shorter.  Off: backward re-gathers them from ``x`` and ``t1`` as the reference does.
    """
    global _SAVE_RATIO
    if enabled is not None:
        _SAVE_RATIO = bool(enabled)
    return _SAVE_RATIO


def matrix_kernels(enabled: Optional[bool] = None) -> bool:
    """Get or set whether bf16 3x3x3 updates may run on the kernels that use the 4x4x4 matrix
    instruction (the process default, ``ndc_matrix_kernels``).  Off by default (environment
    ``DECONVER_NDC_MATRIX=1`` turns it on when the library is loaded): the path is specified
    without matrix instructions.  Same results to the bf16 tolerance, less time per step.
    An update node reads the setting once, in its forward, and names the family in its forward
    and backward calls (``ndc_geom.path``), so a change takes effect from the next forward."""
    return _lib.get_library().matrix_kernels(enabled)


def hip_kernels_apply(x: Tensor, m: int, sc: int, kernel_size, dtype=None) -> bool:
    """Whether the HIP update can run for this input and filter geometry.

    Counterpart of ``fused_kernels_apply`` (``functional.py:34-47``): device tensors only,
    no active functorch transform, float32 or bfloat16 storage, rank 1-3, odd kernel.
    """
    try:
        functorch = torch._C._are_functorch_transforms_active()
    except AttributeError:  # pragma: no cover
        functorch = False
    dtype = x.dtype if dtype is None else dtype
    if functorch or not x.is_cuda or dtype not in (torch.float32, torch.bfloat16):
        return False
    if not 1 <= len(kernel_size) <= 3 or x.dim() - 2 != len(kernel_size):
        return False
    if any(k % 2 == 0 for k in kernel_size):
        return False
    lib = _lib.get_library()  # raises when the library is missing: no silent fallback
    g = _lib.make_geom(x.shape[0], x.shape[1] // m, m, sc, x.shape[2:], kernel_size,
                       ops.dtype_tag(dtype), True, 0.0)
    return lib.check_geometry(g) == 0


def _node_forward(ctx, needs, x, z, h, bias, groups, m, sc, eps, relu_input, taps):
    """Forward of an update node: runs the kernels, records on ``ctx`` what backward needs
    besides tensors and returns ``(out, tensors to save)``.  ``needs``: whether a gradient is
    wanted for ``(x, z, h, bias)``."""
    if not x.is_cuda:
        raise RuntimeError("deconv_update runs on the GPU only (HIP kernels); "
                           "CPU tensors take the layer's general PyTorch path")
    lib = _lib.get_library()
    # channels-last tensors (torch.channels_last / channels_last_3d) come in through the
    # library's tiled transposition, and the results go back out the same way, in the
    # layout of the tensor they belong to
    ctx.cl = (ops.is_channels_last(x), ops.is_channels_last(z))
    with torch.cuda.device(x.device):
        x = ops.to_channel_first(lib, x)
        z = ops.to_channel_first(lib, z)
    hc = h.contiguous()
    need_t1 = any(needs)
    keep = need_t1 and _SAVE_RATIO
    # The kernel family is read once, here, and named in both calls of this node: backward
    # runs on an autograd thread, possibly after the process default has changed.
    path = _lib.PATH_AUTO
    if lib.fused_supported(ops.make_geom_for(x, hc, groups, m, sc, eps, relu_input)):
        path = _lib.PATH_FUSED_MATRIX if lib.matrix_kernels() else _lib.PATH_FUSED_VECTOR
    if keep:
        # only where the backward kernels for this geometry read them
        keep = lib.backward_uses_saved(
            ops.make_geom_for(x, hc, groups, m, sc, eps, relu_input, path))
    with torch.cuda.device(x.device):
        if taps is None:
            # packed once here, used by the forward kernel and again by the backward's
            taps = ops.prepare_taps(lib, x, hc, groups=groups, m=m, sc=sc)
        res = ops.update_forward(lib, x, z, hc, bias, groups=groups, m=m, sc=sc, eps=eps,
                                 relu_input=relu_input, need_t1=need_t1, save_ratio=keep,
                                 taps=taps, path=path)
    out, t1 = res[0], res[1]
    s_over_den, ratio = res[2] if keep else (None, None)
    ctx.cfg = (groups, m, sc, eps, relu_input)
    ctx.path = path
    ctx.taps = taps if need_t1 else None   # a function of h alone; h is saved
    if ctx.cl[1]:
        with torch.cuda.device(x.device):
            out = ops.to_channels_last(lib, out)
    return out, (x, z, t1, hc, bias, s_over_den, ratio)


def _node_backward(ctx, saved, gout, need_x, need_z, need_h, need_b):
    """``(gx, gz, gh, gb)`` of an update node from the tensors its forward saved."""
    # The gradients come from kernels autograd cannot see through, so a second
    # differentiation would silently drop terms: refuse it, as the reference does.
    if torch.is_grad_enabled():
        raise RuntimeError(
            "double backward through the fused Deconv update is not supported; "
            "construct the layer with a convolution keyword argument (e.g. stride=1) "
            "to force the general path, which is plain PyTorch and doubly differentiable")
    x, z, t1, h, bias, s_over_den, ratio = saved
    groups, m, sc, eps, relu_input = ctx.cfg
    if t1 is None:
        raise RuntimeError("backward called on an update that was run without gradients")
    lib = _lib.get_library()
    if gout.dtype != z.dtype:
        gout = gout.to(z.dtype)
    with torch.cuda.device(x.device):
        gout = ops.to_channel_first(lib, gout)
        gx, gz, gh, gb = ops.update_backward(
            lib, x, z, t1, h, bias, gout, groups=groups, m=m, sc=sc, eps=eps,
            relu_input=relu_input, need_x=need_x, need_z=need_z, need_h=need_h,
            need_b=need_b and bias is not None, path=ctx.path,
            saved=None if s_over_den is None else (s_over_den, ratio), taps=ctx.taps)
        if ctx.cl[0] and gx is not None:
            gx = ops.to_channels_last(lib, gx)
        if ctx.cl[1] and gz is not None:
            gz = ops.to_channels_last(lib, gz)
    return gx, gz, gh, gb


class DeconvUpdate(torch.autograd.Function):
    """``out = relu(z + b) * (A(x) + eps) / (A(K(relu(z + b))) + eps)``."""

    @staticmethod
    def forward(ctx, x, z, h, bias, groups, m, sc, eps, relu_input, taps=None):
        out, saved = _node_forward(ctx, ctx.needs_input_grad[:4], x, z, h, bias, groups, m, sc,
                                   eps, relu_input, taps)
        ctx.save_for_backward(*saved)
        return out

    @staticmethod
    def backward(ctx, gout):
        gx, gz, gh, gb = _node_backward(ctx, ctx.saved_tensors, gout, *ctx.needs_input_grad[:4])
        return gx, gz, gh, gb, None, None, None, None, None, None


class ProjectedUpdate(torch.autograd.Function):
    """The layer's first update together with the 1x1 projection that makes its source
    (deconv.py:157-165 with layers/linear.py:53-58 of the reference):
    ``z = W x`` per sample, then ``DeconvUpdate`` on ``(x, z)`` with the projection's bias and
    the ReLU applied where the kernels load ``z``.

    One node instead of two because ``x`` feeds both the projection and the update: as two
    nodes their input gradients are two tensors that autograd adds in a pass of its own;
    here the projection's input-gradient GEMM accumulates onto the update's ``gx``
    (``gx += W^T gz``, one rounding instead of two in bfloat16).  The GEMMs are the ones of
    ``layers.pointwise_linear``: one batched launch over the samples on the channel-first
    tensors, the weight gradient summed in float32."""

    @staticmethod
    def forward(ctx, x, weight, h, bias, groups, m, sc, eps, taps=None, rectified_input=False):
        from .layers import project
        # (kept in its own dtype where the GEMMs pack it themselves, cast once otherwise)
        w = weight.detach()
        if not ops.pointwise_gemm_applies(_lib.get_library(), x.flatten(2), w.shape[0]):
            w = w.to(x.dtype)
        z = project(w, x.flatten(2)).view(x.shape[0], w.shape[0], *x.shape[2:])
        need_x, need_w, need_h, need_b = ctx.needs_input_grad[:4]
        out, saved = _node_forward(ctx, (need_x, need_x or need_w, need_h, need_b), x, z, h,
                                   bias, groups, m, sc, eps, True, taps)
        ctx.save_for_backward(*saved, w)
        ctx.weight_dtype = weight.dtype
        # x is a rectifier's output and its producer skips the rectifier's backward pass: the
        # gradient of x leaves this node already zero where x is
        ctx.rectified_input = bool(rectified_input)
        return out

    @staticmethod
    def backward(ctx, gout):
        from .layers import project_back, projection_weight_grad
        *saved, w = ctx.saved_tensors
        need_x, need_w, need_h, need_b = ctx.needs_input_grad[:4]
        gx, gz, gh, gb = _node_backward(ctx, saved, gout, need_x, need_x or need_w, need_h, need_b)
        x = saved[0]
        gw = None
        if need_w:
            gw = projection_weight_grad(gz.flatten(2), x.flatten(2), ctx.weight_dtype)
        if need_x:
            gx = project_back(w, gz.flatten(2), accumulate=gx.flatten(2),
                              mask=x.flatten(2) if ctx.rectified_input else None).view_as(x)
        return gx, gw, gh, gb, None, None, None, None, None, None


def deconv_update(x: Tensor, z: Tensor, h: Tensor, bias: Optional[Tensor], *, groups: int,
                  m: int, sc: int, eps: float, relu_input: bool,
                  taps: Optional[Tensor] = None) -> Tensor:
    """One multiplicative source update.

    Args:
        x: input, ``(B, C, *S)``.
        z: projection output ``(B, groups*sc, *S)``, pre-bias and pre-ReLU on the first
            iteration (the kernels apply both on load); the rectified source afterwards.
        h: rectified filter ``(C, sc, *k)``, float32.
        bias: the projection's bias (float32) or ``None``.
        eps: stabiliser added to numerator and denominator.
        taps: optional (not in the reference): the table ``ops.prepare_taps`` made for this
            ``h``, for callers that run several updates with one filter; made here otherwise.
    """
    return DeconvUpdate.apply(x, z, h, bias, groups, m, sc, eps, relu_input, taps)


def projected_update(x: Tensor, weight: Tensor, h: Tensor, bias: Optional[Tensor], *, groups: int,
                     m: int, sc: int, eps: float, taps: Optional[Tensor] = None,
                     rectified_input: bool = False) -> Tensor:
    """``deconv_update(x, W x, h, bias, relu_input=True)`` as one autograd node (not in the
    reference, which records the projection and the update separately).

    Args:
        x: input ``(B, C, *S)``, contiguous, float32 or bfloat16 on the GPU.
        weight: the projection's weight ``(groups*sc, C)``, any floating dtype (cast to ``x``'s
            for the GEMMs; its gradient comes back in its own dtype).
        h, bias, groups, m, sc, eps, taps: as for ``deconv_update``.
        rectified_input: ``x`` is the output of a rectifier whose backward pass its producer
            skips (``Linear(..., act="relu", grad_premasked=True)``): the gradient of ``x`` is
            returned zero where ``x`` is, from the GEMM that forms it.
    """
    with torch.autocast(x.device.type, enabled=False):
        return ProjectedUpdate.apply(x, weight, h, bias, groups, m, sc, eps, taps, rectified_input)
