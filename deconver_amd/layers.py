"""Channel-first helper layers around the NDC update (``deconver/layers`` of the reference):
``Linear`` (1x1 projection, parameters held by an ``nn.Conv1d`` as there), ``MLP``,
``LayerNorm``, and the network's resampling convolutions, head and stem as subclasses of the
``torch.nn`` convolutions.  On the GPU the projections are batched channel-first GEMMs
(hipBLASLt through ``torch.bmm``) followed by one pass of the HIP library for bias, activation
and residual sum; the strided convolutions are a regrouping copy in front of the same
projection.  Parameter names and shapes match the reference, so its checkpoints load
unchanged."""

from __future__ import annotations

import math
from typing import Optional

import torch
from torch import nn
from torch.nn.modules.utils import _pair

from . import _lib, ops


def _wgrad_chunks(batch: int, n: int, min_chunk: int = 2048) -> int:
    """Number of equal chunks the voxel axis is cut into for the weight-gradient GEMM: a power
    of two that divides ``n``, leaves chunks of at least ``min_chunk`` voxels and at most 128
    GEMMs in the batch."""
    s = 1
    while s < 64 and n % (2 * s) == 0 and n // (2 * s) >= min_chunk and batch * 2 * s <= 128:
        s *= 2
    return s


def _wgrad_plan(batch: int, n: int, dtype: torch.dtype) -> int:
    """The chunk count ``projection_weight_grad`` uses, from timings on an MI355X with batch 2
    in bfloat16 (64 chunks at 128^3; 32 at 64^3, where 64 cost 0.05 ms more on the 128 x 128
    result; 16 at 32^3: 0.056 ms against 0.11-0.13 ms unchunked; none at 16^3) and batch 8 in
    float32 (none up to 256^2 voxels: there every chunked form was slower)."""
    if dtype == torch.bfloat16:
        return 1 if n < (1 << 15) else _wgrad_chunks(batch, n, 2048 if n < (1 << 17) else 8192)
    return 1 if n < (1 << 17) else _wgrad_chunks(batch, n)


def projection_weight_grad(gz: torch.Tensor, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``sum_b gz[b] x[b]^T`` for ``gz`` of shape ``(B, Cout, N)`` and ``x`` of shape
    ``(B, Cin, N)``: the weight gradient of a 1x1 projection, a ``Cout x Cin`` result summed
    over all voxels.  Short rows (the 2-D network's levels) take one batched GEMM and a sum over
    the batch; long rows are cut into equal chunks of the voxel axis that become batch entries
    (strided views, no copies).  The partial results -- float32 also for bfloat16 operands -- are
    added in float32, in one reduction."""
    B, cout, n = gz.shape
    cin = x.shape[1]
    s = _wgrad_plan(B, n, gz.dtype)
    # bfloat16 operands: the GEMMs hand out their float32 accumulators (same speed, and the
    # partial results are then not rounded to bfloat16 before they are added)
    f32 = {"out_dtype": torch.float32} if gz.is_cuda and gz.dtype == torch.bfloat16 else {}
    if s == 1:
        parts = torch.bmm(gz, x.transpose(1, 2), **f32)
    else:
        parts = gz.new_empty(B * s, cout, cin, dtype=torch.float32 if f32 else gz.dtype)
        for b in range(B):
            a = gz[b].view(cout, s, n // s).transpose(0, 1)
            c = x[b].view(cin, s, n // s).permute(1, 2, 0)
            torch.bmm(a, c, out=parts[b * s:(b + 1) * s], **f32)
    return parts.sum(0, dtype=torch.float32).to(dtype)


def project(weight: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """``W x`` per sample for contiguous ``x`` of shape ``(B, Cin, N)`` and ``weight`` of shape
    ``(Cout, Cin)`` in any floating dtype (used in ``x``'s): the library's streaming GEMM where
    it applies, else one batched hipBLASLt GEMM with the weight shared through a zero stride."""
    lib = _lib.get_library()
    if ops.pointwise_gemm_applies(lib, x, weight.shape[0]):
        with torch.cuda.device(x.device):
            return ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, weight.contiguous()), weight.shape[0])[0]
    z = x.new_empty(x.shape[0], weight.shape[0], x.shape[2])
    torch.bmm(weight.to(x.dtype).unsqueeze(0).expand(x.shape[0], -1, -1), x, out=z)
    return z


def project_back(weight: torch.Tensor, gz: torch.Tensor, accumulate: Optional[torch.Tensor] = None,
                 mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``W^T gz`` per sample (the input gradient of a 1x1 projection with ``weight`` of shape
    ``(Cout, Cin)``), plus ``accumulate`` if given (a tensor of the result's shape, which may
    be overwritten), and zero wherever ``mask <= 0`` if a mask of the result's shape is given
    (the gradient taken through the rectifier whose output the projection read).  The
    library's streaming GEMM where it applies -- the weight is packed as it lies, no transposed
    copy --, else one batched hipBLASLt GEMM."""
    B, cout, n = gz.shape
    if cout == 1:
        # one output channel (the network's head): the product is an outer product, i.e. a
        # broadcast multiplication at the memory rate (as a GEMM it ran at a fifth of it)
        gx = gz * weight.reshape(1, -1, 1).to(gz.dtype)
        gx = gx if accumulate is None else accumulate.add_(gx)
    else:
        lib = _lib.get_library()
        if gz.is_contiguous() and ops.pointwise_gemm_applies(lib, gz, weight.shape[1]):
            with torch.cuda.device(gz.device):
                wfrag = ops.pointwise_pack(lib, weight.contiguous(), transposed=True)
                return ops.pointwise_gemm(lib, gz, wfrag, weight.shape[1], residual=accumulate, mask=mask)[0]
        wt = weight.to(gz.dtype).t().unsqueeze(0).expand(B, -1, -1)
        if accumulate is not None:
            gx = accumulate.baddbmm_(wt, gz)
        else:
            gx = gz.new_empty(B, weight.shape[1], n)
            torch.bmm(wt, gz, out=gx)
    return gx if mask is None else gx.mul_(mask > 0)


class _PointwiseLinear(torch.autograd.Function):
    """``y[b] = act(W x[b] + bias) + residual[b]`` for ``x`` of shape ``(B, Cin, N)``: the 1x1
    projection as plain GEMMs on the channel-first layout (hipBLASLt through ``torch.bmm``),
    then ONE pass of the HIP library over the result for bias, activation and residual sum
    (``ndc_bias_act``).

    The same map as ``nn.Conv1d(kernel_size=1)`` (layers/linear.py:53-58) followed by the
    activation and the ``x + ...`` of the block (layers/mlp.py:40-63, deconver.py:60-64).  The
    library convolution reaches its GEMM through layout transposes of input and output and a
    separate weight-gradient kernel; here forward and input gradient are one GEMM each on
    the tensors as they lie, and the weight gradient (a ``Cout x Cin`` result summed over
    millions of voxels) is a batch of GEMMs over equal chunks of the voxel axis whose
    partial results are added in float32: 0.54 ms instead of 0.89 ms for forward + backward
    of the 128 -> 512 projection at 2 x 64^3 in bf16."""

    @staticmethod
    def forward(ctx, x, weight, bias, act, residual, grad_premasked=False):
        lib = _lib.get_library()
        # one batched GEMM on the tensors as they lie, the weight shared by the batch entries
        # through a zero stride (no copy; the same bits as one GEMM per sample, in one launch)
        # (the weight arrives in its own dtype -- float32 under autocast -- and is cast here, so
        # that its gradient leaves backward as the float32 sum it is, not rounded to bf16 first)
        B = x.shape[0]
        w = weight.detach()
        bias32 = None if bias is None else bias.detach().float().contiguous()
        # the activation's gradient needs z + bias: gelu keeps z; relu alone needs only the
        # sign of its output, which may then overwrite z
        keep_z = act == "gelu" or (act == "relu" and residual is not None)
        keep_z = keep_z and any(ctx.needs_input_grad)     # (nothing is kept for a forward-only call)
        if ops.pointwise_gemm_applies(lib, x, w.shape[0], act, keep_z):
            # the library's streaming GEMM: product, bias, activation and residual in one
            # kernel that reads x once and writes the result (and z where it is kept) once
            with torch.cuda.device(x.device):
                y, z = ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w.contiguous()),
                                          w.shape[0], bias32, residual, act, keep_z=keep_z)
            # (the packing reads the weight in its own dtype, and so does the backward's: no
            # cast copy of it is made or kept)
        else:
            w = w.to(x.dtype)
            z = x.new_empty(B, w.shape[0], x.shape[2])
            torch.bmm(w.unsqueeze(0).expand(B, -1, -1), x, out=z)
            y = z
            if bias is not None or act is not None or residual is not None:
                with torch.cuda.device(x.device):
                    y = ops.bias_act(lib, z, bias32, residual, act, inplace=not keep_z)
        kept = z if keep_z else y if act == "relu" else None
        ctx.save_for_backward(x, w, kept, bias32 if keep_z else None)
        ctx.weight_dtype = weight.dtype
        ctx.has_bias = bias is not None
        ctx.act = act
        # a ReLU whose consumer hands back a gradient that is already zero where the output is
        # (``project_back(mask=...)``): the backward then has no pass of its own for it
        ctx.premasked = bool(grad_premasked) and act == "relu" and residual is None
        return y

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy):
        x, weight, kept, bias32 = ctx.saved_tensors
        gy = gy.contiguous()
        gx = gw = gb = None
        gres = gy if ctx.needs_input_grad[4] else None
        want_gb = ctx.has_bias and ctx.needs_input_grad[2]
        gz = gy
        if ctx.premasked:
            if want_gb:
                with torch.cuda.device(gy.device):
                    gb = ops.channel_sums(_lib.get_library(), gy)
        elif ctx.act is not None:
            with torch.cuda.device(gy.device):
                gz, gb = ops.bias_act_backward(_lib.get_library(), gy, kept, bias32, ctx.act,
                                               need_bias_grad=want_gb)
        elif want_gb:
            # per-row partial sums by the library (at the copy rate), then the few per-sample
            # sums: PyTorch's one-call reduction of a (B, C, N) tensor over B and N runs at a
            # tenth of the memory bandwidth, its row sums at two thirds
            with torch.cuda.device(gy.device):
                gb = ops.channel_sums(_lib.get_library(), gy)
        if ctx.needs_input_grad[0]:
            gx = project_back(weight, gz)
        if ctx.needs_input_grad[1]:
            gw = projection_weight_grad(gz, x, ctx.weight_dtype)
        return gx, gw, gb, None, gres, None


_ACT_FUNCTIONS = {None: lambda t: t, "relu": torch.relu, "gelu": torch.nn.functional.gelu}


def pointwise_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     act: Optional[str] = None, residual: Optional[torch.Tensor] = None,
                     grad_premasked: bool = False) -> torch.Tensor:
    """``act(W x + bias) + residual``: the 1x1 projection ``(B, Cin, N) -> (B, Cout, N)`` with
    ``weight`` of shape ``(Cout, Cin)`` or ``(Cout, Cin, 1)``, optionally followed by an
    activation (``"relu"`` or ``"gelu"``, the exact one) and the sum with a tensor of the
    output's shape.  bfloat16 (stored or under autocast) and float32 tensors on the GPU run as
    batched GEMMs on the channel-first layout plus one pass of the HIP library over the result;
    everything else as the reference's ``conv1d`` followed by PyTorch's activation and sum.

    ``grad_premasked`` (GEMM route, ``act="relu"`` without residual only; ignored elsewhere): the
    caller guarantees that every gradient reaching the result is already zero where the result
    is -- its only consumer took it through the rectifier (``project_back(mask=...)``) --, so the
    backward skips the rectifier's pass."""
    w2 = weight.squeeze(-1) if weight.dim() == 3 else weight
    dtype = x.dtype
    if x.is_cuda and torch.is_autocast_enabled(x.device.type):
        dtype = torch.get_autocast_dtype(x.device.type)
    # (2-D network in float32, batch 8: 16.6 ms per step this way against 20.8 ms with the
    # GEMM left to the library's conv1d, whose weight gradient goes through layout transposes)
    if not x.is_cuda or x.dim() != 3 or dtype not in (torch.bfloat16, torch.float32):
        y = _ACT_FUNCTIONS[act](torch.nn.functional.conv1d(x, w2.unsqueeze(-1), bias))
        return y if residual is None else residual + y
    x = x.to(dtype)
    if residual is not None:
        residual = residual.to(dtype).contiguous()
    with torch.autocast(x.device.type, enabled=False):
        return _PointwiseLinear.apply(x.contiguous(), w2, bias, act, residual, grad_premasked)


def _gemm_route(x: torch.Tensor) -> bool:
    """True for the tensors whose 1x1 projection ``pointwise_linear`` runs as channel-first
    GEMMs: bfloat16 (stored or under autocast) and float32 on the GPU."""
    dtype = x.dtype
    if x.is_cuda and torch.is_autocast_enabled(x.device.type):
        dtype = torch.get_autocast_dtype(x.device.type)
    return x.is_cuda and dtype in (torch.bfloat16, torch.float32)


def _is_patch_conv(conv) -> bool:
    """A convolution whose windows tile the input: stride == kernel size, no padding, no
    dilation, one group (and no output padding on a transposed one)."""
    return (tuple(conv.stride) == tuple(conv.kernel_size) and all(p == 0 for p in conv.padding)
            and all(d == 1 for d in conv.dilation) and conv.groups == 1
            and isinstance(conv.padding, tuple)
            and all(p == 0 for p in getattr(conv, "output_padding", ())))


def patches_to_channels(x: torch.Tensor, k) -> torch.Tensor:
    """``(B, C, *S) -> (B, C * prod(k), prod(S // k))``: every ``k`` window of the grid becomes
    one column, channel-major then window offset (the order of a convolution weight's
    ``(Cin, *k)`` axes).  Rows and planes that do not fill a window are dropped, as a strided
    convolution drops them."""
    B, C = x.shape[:2]
    nd = len(k)
    if all(v == 1 for v in k):
        return x.flatten(2)
    coarse = [s // v for s, v in zip(x.shape[2:], k)]
    if any(c * v != s for c, v, s in zip(coarse, k, x.shape[2:])):
        x = x[(slice(None), slice(None), *[slice(0, c * v) for c, v in zip(coarse, k)])]
    split = [B, C]
    for c, v in zip(coarse, k):
        split += [c, v]
    x = x.reshape(split)
    order = [0, 1] + [3 + 2 * i for i in range(nd)] + [2 + 2 * i for i in range(nd)]
    return x.permute(order).reshape(B, C * math.prod(k), math.prod(coarse))


def channels_to_patches(y: torch.Tensor, k, coarse) -> torch.Tensor:
    """Inverse of ``patches_to_channels`` on an exactly tiled grid:
    ``(B, C * prod(k), prod(coarse)) -> (B, C, *(coarse * k))``."""
    B = y.shape[0]
    nd = len(k)
    C = y.shape[1] // math.prod(k)
    if all(v == 1 for v in k):
        return y.view(B, C, *coarse)
    y = y.view(B, C, *k, *coarse)
    order = [0, 1]
    for i in range(nd):
        order += [2 + nd + i, 2 + i]
    return y.permute(order).reshape(B, C, *[c * v for c, v in zip(coarse, k)])


class _Regroup2(torch.autograd.Function):
    """2 x 2 (x 2) windows of the grid <-> 2^nd channels per window on the HIP kernel
    (``ndc_regroup``); each direction's gradient is the other direction.  On the way back to
    the grid a per-channel bias can be added in the same pass."""

    @staticmethod
    def forward(ctx, x, to_channels, bias):
        lib = _lib.get_library()
        ctx.to_channels = to_channels
        ctx.has_bias = bias is not None
        with torch.cuda.device(x.device):
            if to_channels:
                return ops.windows_to_channels(lib, x)
            return ops.channels_to_windows(lib, x, None if bias is None else bias.detach().float().contiguous())

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g):
        lib = _lib.get_library()
        g = g.contiguous()
        gb = None
        with torch.cuda.device(g.device):
            if ctx.to_channels:
                return ops.channels_to_windows(lib, g), None, None
            if ctx.has_bias and ctx.needs_input_grad[2]:
                gb = ops.channel_sums(lib, g.flatten(2))
            return ops.windows_to_channels(lib, g), None, gb


def _regroup_on_hip(fine_shape, dtype, k, *tensors) -> bool:
    """2-windows in every dimension and GPU buffers the kernel takes (``tensors``: the ones
    that exist already)."""
    return (all(v == 2 for v in k) and len(k) in (2, 3) and all(t.is_cuda for t in tensors)
            and ops.regroup2_applies(tuple(fine_shape), dtype, *[t.data_ptr() for t in tensors]))


def patch_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``conv(x, weight, bias, stride=weight.shape[2:])``, no padding: a strided convolution
    whose windows tile its input is a regrouping of the grid followed by the 1x1 projection."""
    k = tuple(weight.shape[2:])
    coarse = [s // v for s, v in zip(x.shape[2:], k)]
    if x.is_cuda and torch.is_autocast_enabled(x.device.type):
        x = x.to(torch.get_autocast_dtype(x.device.type))     # before the regrouping, not after
    xc = x.contiguous()
    if _regroup_on_hip(xc.shape, xc.dtype, k, xc):
        cols = _Regroup2.apply(xc, True, None).flatten(2)
    else:
        cols = patches_to_channels(x, k)
    y = pointwise_linear(cols, weight.flatten(1), bias)
    return y.view(x.shape[0], -1, *coarse)


def patch_conv_transpose(x: torch.Tensor, weight: torch.Tensor,
                         bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``conv_transpose(x, weight, bias, stride=weight.shape[2:])``: the 1x1 projection to
    ``Cout * prod(k)`` channels, then every column spread over its window of the finer grid."""
    k = tuple(weight.shape[2:])
    # weight (Cin, Cout, *k): row (cout, offset) of the projection is weight[:, cout, offset]
    w = weight.flatten(1).t()
    fine = (x.shape[0], weight.shape[1], *[s * v for s, v in zip(x.shape[2:], k)])
    dtype = x.dtype
    if x.is_cuda and torch.is_autocast_enabled(x.device.type):
        dtype = torch.get_autocast_dtype(x.device.type)
    if x.is_cuda and _regroup_on_hip(fine, dtype, k):
        # the bias rides on the regrouping pass
        y = pointwise_linear(x.flatten(2), w, None).contiguous()
        if _regroup_on_hip(fine, y.dtype, k, y):
            return _Regroup2.apply(y.view(x.shape[0], -1, *x.shape[2:]), False, bias)
        y = channels_to_patches(y, k, x.shape[2:])
        return y if bias is None else y + bias.to(y.dtype).view(1, -1, *([1] * len(k)))
    if bias is not None:
        bias = bias.repeat_interleave(math.prod(k))
    return channels_to_patches(pointwise_linear(x.flatten(2), w, bias), k, x.shape[2:])


class _PatchConvMixin:
    """The network's 2-tap resampling convolutions (unet.py:36-60) and its 1-tap head are
    convolutions whose windows tile the input.  bfloat16 and float32 tensors on the GPU take
    the form of ``patch_conv`` here -- one regrouping copy and the projection of
    ``pointwise_linear`` instead of the library's column-matrix convolution; everything else,
    and any other stride or padding, runs the parent class's convolution.  Parameters, their
    shapes and names are the parent's."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if _is_patch_conv(self) and _gemm_route(x) and x.dim() == len(self.kernel_size) + 2:
            return patch_conv(x, self.weight, self.bias)
        return super().forward(x)


class _PatchConvTransposeMixin:
    """The transposed counterpart (unet.py:108-131), as ``patch_conv_transpose``."""

    def forward(self, x: torch.Tensor, output_size=None) -> torch.Tensor:
        if (output_size is None and _is_patch_conv(self) and _gemm_route(x)
                and x.dim() == len(self.kernel_size) + 2):
            return patch_conv_transpose(x, self.weight, self.bias)
        return super().forward(x, output_size)


def unfold_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``conv(x, weight, bias, stride=1, padding=k // 2)`` for odd kernel sizes ``k`` as a column
    matrix (every tap's shifted copy of the zero-padded input, channel-major then tap: the order
    of the weight's ``(Cin, *k)`` axes) followed by the 1x1 projection."""
    k = tuple(weight.shape[2:])
    size = x.shape[2:]
    pad = []
    for v in reversed(k):
        pad += [v // 2, v // 2]
    xp = torch.nn.functional.pad(x, pad)
    shifts = [()]
    for v in k:
        shifts = [t + (o,) for t in shifts for o in range(v)]
    cols = torch.stack([xp[(slice(None), slice(None), *[slice(o, o + n) for o, n in zip(t, size)])]
                        for t in shifts], dim=2)
    y = pointwise_linear(cols.flatten(1, 2).flatten(2), weight.flatten(1), bias)
    return y.view(x.shape[0], -1, *size)


class _UnfoldConvMixin:
    """The network's stem (unet.py:175-276: a 3-tap convolution from the few image channels to
    the first width): with few input channels the column matrix is small next to the output,
    and bfloat16 / float32 tensors on the GPU take ``unfold_conv`` -- one gather and the
    projection of ``pointwise_linear`` -- instead of the library's convolution, whose weight
    gradient alone takes longer.  Anything else (more than ``max_columns`` rows in the column matrix, other
    strides or paddings) runs the parent class's convolution."""

    max_columns = 128

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        k = tuple(self.kernel_size)
        if (_gemm_route(x) and x.dim() == len(k) + 2 and all(v % 2 == 1 for v in k)
                and isinstance(self.padding, tuple) and tuple(self.padding) == tuple(v // 2 for v in k)
                and all(v == 1 for v in self.stride) and all(v == 1 for v in self.dilation)
                and self.groups == 1 and self.padding_mode == "zeros"
                and self.in_channels * math.prod(k) <= self.max_columns):
            if torch.is_autocast_enabled(x.device.type):
                x = x.to(torch.get_autocast_dtype(x.device.type))    # before the gather, not after
            return unfold_conv(x, self.weight, self.bias)
        return super().forward(x)


class UnfoldConv1d(_UnfoldConvMixin, nn.Conv1d):
    pass


class UnfoldConv2d(_UnfoldConvMixin, nn.Conv2d):
    pass


class UnfoldConv3d(_UnfoldConvMixin, nn.Conv3d):
    pass


class PatchConv1d(_PatchConvMixin, nn.Conv1d):
    pass


class PatchConv2d(_PatchConvMixin, nn.Conv2d):
    pass


class PatchConv3d(_PatchConvMixin, nn.Conv3d):
    pass


class PatchConvTranspose1d(_PatchConvTransposeMixin, nn.ConvTranspose1d):
    pass


class PatchConvTranspose2d(_PatchConvTransposeMixin, nn.ConvTranspose2d):
    pass


class PatchConvTranspose3d(_PatchConvTransposeMixin, nn.ConvTranspose3d):
    pass


class Linear(nn.Module):
    """Pointwise linear map over channels for ``(N, C, *)`` inputs (layers/linear.py:34-58).

    The weight lives in ``self.linear`` (an ``nn.Conv1d`` with kernel size 1), hence the
    state-dict keys ``linear.weight`` ``(Cout, Cin, 1)`` and ``linear.bias``.
    """

    def __init__(self, in_channels: int, out_channels: int, bias: bool = True,
                 device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None):
        super().__init__()
        self.flatten = nn.Flatten(start_dim=2)
        self.linear = nn.Conv1d(in_channels, out_channels, kernel_size=1, bias=bias,
                                device=device, dtype=dtype)

    def forward(self, x: torch.Tensor, act: Optional[str] = None,
                residual: Optional[torch.Tensor] = None, grad_premasked: bool = False) -> torch.Tensor:
        """``act(linear(x)) + residual``; ``act`` None, ``"relu"`` or ``"gelu"``; ``residual``
        of the output's shape; ``grad_premasked`` as for ``pointwise_linear``."""
        shape = x.shape
        if residual is not None:
            residual = residual.flatten(2)
        y = pointwise_linear(self.flatten(x), self.linear.weight, self.linear.bias, act, residual,
                             grad_premasked)
        return y.view(shape[0], -1, *shape[2:])


class _FusedMLP(torch.autograd.Function):
    """``W2 gelu(W1 x + b1) + b2 + residual`` on contiguous bfloat16 ``(B, C, N)`` tensors as ONE
    autograd node on the library's streaming GEMM (layers/mlp.py:40-63 with the block's sum,
    deconver.py:60-64): two launches forward (the GELU and the kept pre-activation leave the
    first, bias and residual ride on the second), and a backward in which the input gradient
    of the second projection comes out already multiplied by the GELU's derivative, with the
    first bias's gradient summed in the same kernel -- the hidden tensor's gradient is written
    once and never read back by an activation pass."""

    @staticmethod
    def applies(lib, x: torch.Tensor, hidden: int, cout: int) -> bool:
        B, c, n = x.shape
        ok = lambda cin, co: lib.pointwise_gemm_supported(cin, co, n, _lib.NDC_BF16)   # noqa: E731
        return (x.is_cuda and x.dtype == torch.bfloat16 and ok(c, hidden) and ok(hidden, cout)
                and ok(cout, hidden) and ok(hidden, c))

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2, residual):
        lib = _lib.get_library()
        hidden, cout = w1.shape[0], w2.shape[0]
        b1f = None if b1 is None else b1.detach().float().contiguous()
        b2f = None if b2 is None else b2.detach().float().contiguous()
        with torch.cuda.device(x.device):
            a, z = ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w1.detach().contiguous()), hidden, b1f,
                                      None, "gelu", keep_z=any(ctx.needs_input_grad))
            y, _ = ops.pointwise_gemm(lib, a, ops.pointwise_pack(lib, w2.detach().contiguous()), cout, b2f,
                                      residual, None)
        ctx.save_for_backward(x, z, a, w1.detach(), w2.detach(), b1f)
        ctx.dtypes = (w1.dtype, w2.dtype)
        return y

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy):
        x, z, a, w1, w2, b1f = ctx.saved_tensors
        lib = _lib.get_library()
        gy = gy.contiguous()
        need_x, need_w1, need_b1, need_w2, need_b2, need_res = ctx.needs_input_grad
        gx = gw1 = gb1 = gw2 = gb2 = None
        with torch.cuda.device(gy.device):
            if need_b2:
                gb2 = ops.channel_sums(lib, gy)
            if need_w2:
                gw2 = projection_weight_grad(gy, a, ctx.dtypes[1])
            if need_x or need_w1 or need_b1:
                gz, gb1 = ops.pointwise_gemm_actgrad(lib, gy, ops.pointwise_pack(lib, w2.contiguous(), transposed=True),
                                                     w2.shape[1], z, b1f, "gelu", need_bias_grad=need_b1)
                if need_w1:
                    gw1 = projection_weight_grad(gz, x, ctx.dtypes[0])
                if need_x:
                    gx = project_back(w1, gz)
        return gx, gw1, gb1, gw2, gb2, (gy if need_res else None)


class MLP(nn.Module):
    """Linear - GELU - Linear on channels, with dropout after each (layers/mlp.py:40-63)."""

    def __init__(self, in_channels: int, out_channels: Optional[int] = None,
                 hidden_channels: Optional[int] = None, ratio: float = 4.0,
                 dropout: float | tuple[float, float] = 0.0, **kwargs):
        super().__init__()
        out_channels = out_channels or in_channels
        hidden_channels = hidden_channels or int(ratio * in_channels)
        p_hidden, p_out = _pair(dropout)
        self.block = nn.Sequential(
            Linear(in_channels, hidden_channels, **kwargs),
            nn.GELU(),
            nn.Dropout(p_hidden),
            Linear(hidden_channels, out_channels, **kwargs),
            nn.Dropout(p_out),
        )

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``block(x)``, plus ``residual`` if given.  With the exact GELU and no active dropout
        the activation and the sum ride on the projections (``Linear.forward``)."""
        first, act, drop1, second, drop2 = self.block
        idle = lambda d: d.p == 0 or not d.training   # noqa: E731
        if (isinstance(first, Linear) and isinstance(second, Linear) and type(act) is nn.GELU
                and act.approximate == "none" and idle(drop1) and idle(drop2)):
            fused = self._fused(first, second, x, residual)
            return second(first(x, act="gelu"), residual=residual) if fused is None else fused
        y = self.block(x)
        return y if residual is None else residual + y

    @staticmethod
    def _fused(first: "Linear", second: "Linear", x: torch.Tensor, residual: Optional[torch.Tensor]):
        """The block as one node on the streaming GEMM where all four of its products fit it
        (bfloat16, stored or under autocast; e.g. 64 -> 256 -> 64 channels), else None."""
        if not _gemm_route(x):
            return None
        dtype = torch.get_autocast_dtype(x.device.type) if torch.is_autocast_enabled(x.device.type) else x.dtype
        if dtype != torch.bfloat16:
            return None
        flat = x.flatten(2).to(dtype).contiguous()
        w1, w2 = first.linear.weight.squeeze(-1), second.linear.weight.squeeze(-1)
        if not _FusedMLP.applies(_lib.get_library(), flat, w1.shape[0], w2.shape[0]):
            return None
        res = None if residual is None else residual.flatten(2).to(dtype).contiguous()
        with torch.autocast(x.device.type, enabled=False):
            y = _FusedMLP.apply(flat, w1, first.linear.bias, w2, second.linear.bias, res)
        return y.view(x.shape[0], -1, *x.shape[2:])


class _ChannelNorm(torch.autograd.Function):
    """``nn.LayerNorm`` over the channel axis of a channel-first ``(B, C, n)`` tensor on the HIP
    kernels (``ndc_chnorm_forward`` / ``_backward``): lanes along the voxels, a loop over the
    channels, nothing transposed."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        lib = _lib.get_library()
        x = x.contiguous()
        w32 = None if weight is None else weight.detach().float().contiguous()
        b32 = None if bias is None else bias.detach().float().contiguous()
        with torch.cuda.device(x.device):
            y, stats = ops.chnorm_forward(lib, x, w32, b32, eps)
        ctx.save_for_backward(x, stats, w32)
        ctx.dtypes = (None if weight is None else weight.dtype, None if bias is None else bias.dtype)
        return y

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gy):
        x, stats, w32 = ctx.saved_tensors
        gy = gy.to(x.dtype).contiguous()
        affine = any(ctx.needs_input_grad[1:3])
        with torch.cuda.device(x.device):
            gx, gw, gb = ops.chnorm_backward(_lib.get_library(), gy, x, stats, w32, need_affine_grads=affine)
        wd, bd = ctx.dtypes
        return (gx if ctx.needs_input_grad[0] else None,
                gw.to(wd) if affine and ctx.needs_input_grad[1] and wd is not None else None,
                gb.to(bd) if affine and ctx.needs_input_grad[2] and bd is not None else None, None)


_CHNORM_MIN_VOXELS = 32768


class LayerNorm(nn.Module):
    """``nn.LayerNorm`` over the channel axis of a ``(B, C, *S)`` tensor (layers/norm.py:25-34).

    The reference moves the channel axis last, normalises and moves it back, which costs two
    generic strided copies (the norm's own and the next projection's ``contiguous()``).  On the
    GPU (float32 / bfloat16 tensors) the HIP kernels normalise over the channel axis where it
    is; parameters and state dict are ``nn.LayerNorm``'s, and under autocast the arithmetic and
    the result are float32, as PyTorch's autocast rules make them for the reference."""

    def __init__(self, dim: int, **kwargs):
        super().__init__()
        self.norm = nn.LayerNorm(dim, **kwargs)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # (small grids stay with the reference form: below 32 768 voxels in all the kernels'
        # one-thread-per-voxel launch does not fill the chip, and PyTorch's takes 0.06 ms)
        if (x.is_cuda and x.dim() >= 3 and len(self.norm.normalized_shape) == 1
                and x.shape[1] == self.norm.normalized_shape[0]
                and x.shape[0] * x[0, 0].numel() >= _CHNORM_MIN_VOXELS):
            t = x.float() if torch.is_autocast_enabled(x.device.type) else x
            if t.dtype in (torch.float32, torch.bfloat16):
                with torch.autocast(x.device.type, enabled=False):
                    y = _ChannelNorm.apply(t.flatten(2), self.norm.weight, self.norm.bias, float(self.norm.eps))
                return y.view(x.shape)
        return self.norm(x.movedim(1, -1)).movedim(-1, 1)
