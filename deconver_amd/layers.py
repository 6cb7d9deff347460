"""Channel-first helper layers around the NDC update (``deconver/layers`` of the reference):
``Linear`` (1x1 projection as ``nn.Conv1d`` on the flattened volume), ``MLP``, ``LayerNorm``.
They stay on PyTorch-ROCm GEMMs / library kernels; parameter names match the reference so
that its checkpoints load unchanged."""

from __future__ import annotations

from typing import Optional

import torch
from torch import nn
from torch.nn.modules.utils import _pair


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
        y = self.linear(self.flatten(x))
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
