"""Channel-first helper layers around the NDC update (``deconver/layers`` of the reference):
``Linear`` (1x1 projection, parameters held by an ``nn.Conv1d`` as there), ``MLP``,
``LayerNorm``.  They stay on PyTorch-ROCm GEMMs / library kernels; parameter names match the
reference so that its checkpoints load unchanged."""

from __future__ import annotations

from typing import Optional

import torch
from torch import nn
from torch.nn.modules.utils import _pair


def _wgrad_chunks(batch: int, n: int) -> int:
    """Number of equal chunks the voxel axis is cut into for the weight-gradient GEMM: a power
    of two that divides ``n``, leaves chunks of at least 2048 voxels and at most 128 GEMMs in
    the batch (measured on an MI355X: 64 chunks at 64^3 and 128^3 with batch 2, 16 at 32^3)."""
    s = 1
    while s < 64 and n % (2 * s) == 0 and n // (2 * s) >= 2048 and batch * 2 * s <= 128:
        s *= 2
    return s


class _PointwiseLinear(torch.autograd.Function):
    """``y[b] = W x[b] (+ bias)`` for ``x`` of shape ``(B, Cin, N)``: the 1x1 projection as
    plain GEMMs on the channel-first layout (hipBLASLt through ``torch.matmul`` / ``bmm``).

    The same map as ``nn.Conv1d(kernel_size=1)`` (layers/linear.py:53-58).  The library
    convolution reaches its GEMM through layout transposes of input and output and a
    separate weight-gradient kernel; here forward and input gradient are one GEMM each on
    the tensors as they lie, and the weight gradient (a ``Cout x Cin`` result summed over
    millions of voxels) is a batch of GEMMs over equal chunks of the voxel axis whose
    partial results are added in float32: 0.54 ms instead of 0.89 ms for forward + backward
    of the 128 -> 512 projection at 2 x 64^3 in bf16."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        # one GEMM per sample on the tensors as they lie (torch.matmul would fold the batch into
        # the voxel axis through two transposing copies when its input requires a gradient)
        y = x.new_empty(x.shape[0], weight.shape[0], x.shape[2])
        for b in range(x.shape[0]):
            torch.mm(weight, x[b], out=y[b])
        if bias is not None:
            y += bias.to(y.dtype).view(1, -1, 1)
        return y

    @staticmethod
    def backward(ctx, gy):
        x, weight = ctx.saved_tensors
        gy = gy.contiguous()
        gx = gw = gb = None
        if ctx.needs_input_grad[0]:
            gx = torch.empty_like(x)
            wt = weight.t()
            for b in range(x.shape[0]):
                torch.mm(wt, gy[b], out=gx[b])
        if ctx.needs_input_grad[1]:
            B, cout, n = gy.shape
            cin = x.shape[1]
            s = _wgrad_chunks(B, n) if gy.dtype in (torch.bfloat16, torch.float16) else 1
            if s == 1:
                gw = torch.bmm(gy, x.transpose(1, 2)).sum(0)
            else:
                acc = torch.zeros(cout, cin, dtype=torch.float32, device=gy.device)
                for b in range(B):
                    # chunk c of the voxel axis as batch entry c: strided views, no copies
                    a = gy[b].view(cout, s, n // s).transpose(0, 1)
                    c = x[b].view(cin, s, n // s).permute(1, 2, 0)
                    acc += torch.bmm(a, c).float().sum(0)
                gw = acc.to(weight.dtype)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            # rows first (contiguous runs of the voxel axis), then the few per-sample sums: the
            # library's one-call reduction of a (B, C, N) tensor over B and N runs at a tenth of
            # the memory bandwidth (0.19 ms at 2 x 128 x 64^3 in bf16)
            gb = gy.sum(2, dtype=torch.float32).sum(0)
        return gx, gw, gb


def pointwise_linear(x: torch.Tensor, weight: torch.Tensor,
                     bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The 1x1 projection ``(B, Cin, N) -> (B, Cout, N)`` with ``weight`` of shape
    ``(Cout, Cin)`` or ``(Cout, Cin, 1)``.  16-bit tensors on the GPU (bfloat16 / float16
    storage or autocast) run as GEMMs on the channel-first layout; everything else as the
    reference's ``conv1d``."""
    w2 = weight.squeeze(-1) if weight.dim() == 3 else weight
    dtype = x.dtype
    if x.is_cuda and torch.is_autocast_enabled(x.device.type):
        dtype = torch.get_autocast_dtype(x.device.type)
    # 16-bit GPU tensors only: in float32 the library convolution is as fast (2-D network,
    # batch 8: 24.5 against 25.5 ms per step)
    if not x.is_cuda or x.dim() != 3 or dtype not in (torch.bfloat16, torch.float16):
        return torch.nn.functional.conv1d(x, w2.unsqueeze(-1), bias)
    x, w2 = x.to(dtype), w2.to(dtype)
    with torch.autocast(x.device.type, enabled=False):
        return _PointwiseLinear.apply(x.contiguous(), w2, bias)


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

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        y = pointwise_linear(self.flatten(x), self.linear.weight, self.linear.bias)
        return y.view(shape[0], -1, *shape[2:])


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

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.block(x)


class LayerNorm(nn.Module):
    """``nn.LayerNorm`` over the channel axis of a ``(B, C, *S)`` tensor (layers/norm.py:25-34)."""

    def __init__(self, dim: int, **kwargs):
        super().__init__()
        self.norm = nn.LayerNorm(dim, **kwargs)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.norm(x.movedim(1, -1)).movedim(-1, 1)
