"""Deconver: the U-shaped segmentation network whose mixing layers are NDC updates.

API- and state-dict-compatible with the reference's model (``deconver/deconver.py:9-154``
on the skeleton of ``deconver/unet.py:36-276``): same constructor arguments, same module
tree, hence the same parameter names --

    stem.weight
    encoder.blocks.{i}.downsample.{weight,bias}                       (levels with stride > 1)
    encoder.blocks.{i}.block.blocks.{j}.dcm.in_proj.linear.weight
    encoder.blocks.{i}.block.blocks.{j}.dcm.deconv.init.{h0, linear.linear.{weight,bias}}
    encoder.blocks.{i}.block.blocks.{j}.dcm.out_proj.linear.{weight,bias}
    encoder.blocks.{i}.block.blocks.{j}.mlp.block.{0,3}.linear.{weight,bias}
    encoder.blocks.{i}.block.blocks.{j}.norm{1,2}.*                  (if the norm has parameters)
    decoder.blocks.{i}.upsample.{weight,bias}
    decoder.blocks.{i}.block.adapter.linear.weight
    decoder.blocks.{i}.block.blocks.{j}. ...                          (as in the encoder)
    head.{weight,bias}   or   heads.{j}.{weight,bias}                 (deep supervision)

Only the network the reference ships as ``Deconver`` is built here (Deconver stages at
every level); the reference's generic convolutional U-Net blocks are not part of this path.
Everything except the ``Deconv`` layers runs on PyTorch-ROCm library kernels.
"""

from __future__ import annotations

import math
from typing import Any, Optional, Sequence

import torch
from torch import Tensor, nn

from . import layers
from .layers import MLP, LayerNorm, Linear
from .ndc import Deconv
from .norm import native_norm
from .spec import as_tuple, build

__all__ = ["DeconvMixer", "DeconverBlock", "DeconverStage", "Stem", "Deconver"]


class DeconvMixer(nn.Module):
    """``out_proj(Deconv(act(in_proj(x))))`` with dropout (deconver.py:9-46).

    ``in_proj`` has no bias; the activation makes the deconvolution's input nonnegative;
    ``out_proj`` maps the ``groups * source_channels`` sources back to ``out_channels``.
    """

    def __init__(self, in_channels: int, out_channels: int, act: Any = nn.ReLU,
                 dropout: float = 0.0, **deconv_kwargs):
        super().__init__()
        self.in_proj = Linear(in_channels, out_channels, bias=False)
        self.deconv = Deconv(out_channels, **deconv_kwargs)
        self.act = build(act)
        self.out_proj = Linear(self.deconv.groups * self.deconv.source_channels, out_channels)
        self.dropout = nn.Dropout(dropout)

    def forward(self, x: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        """The mixer's output, plus ``residual`` if given (the block's ``x + dcm(...)``, which
        then rides on ``out_proj`` unless dropout is active)."""
        if type(self.act) is nn.ReLU and not self.act._forward_hooks and layers._gemm_route(x):
            # the rectifier rides on the projection (one kernel, or one pass over its output);
            # a hooked activation module is still called as a module.  Its backward rides on the
            # layer's input gradient where the layer forms that in one GEMM; x stands in for
            # the projection's output when asking (same batch, grid, device and autocast state,
            # same channel count for the square in_proj of a block)
            premasked = (type(self.deconv) is Deconv and x.shape[1] == self.in_proj.linear.out_channels
                         and not self.deconv._forward_hooks and not self.deconv._forward_pre_hooks
                         and self.deconv.takes_rectified_input(x))
            h = self.in_proj(x, act="relu", grad_premasked=premasked)
            sources = self.deconv(h, rectified_input=True) if premasked else self.deconv(h)
        else:
            sources = self.deconv(self.act(self.in_proj(x)))
        if self.dropout.p == 0 or not self.training:
            return self.out_proj(sources, residual=residual)
        y = self.dropout(self.out_proj(sources))
        return y if residual is None else residual + y


class DeconverBlock(nn.Module):
    """Pre-norm residual pair: deconvolution mixer, then channel MLP (deconver.py:49-65)."""

    def __init__(self, channels: int, norm: Any = LayerNorm, dropout: float = 0.0,
                 mlp_ratio: float = 4, **mixer_kwargs):
        super().__init__()
        norm = native_norm(norm)   # torch's InstanceNorm classes -> their HIP-backed subclasses
        self.norm1 = build(norm, channels)
        self.dcm = DeconvMixer(channels, channels, **mixer_kwargs)
        self.norm2 = build(norm, channels)
        self.mlp = MLP(channels, ratio=mlp_ratio, dropout=dropout)

    def forward(self, x: Tensor) -> Tensor:
        # (norm(x), x): on the HIP norm the residual's gradient is summed in the norm's backward
        y, x = self.norm1.with_skip(x) if hasattr(self.norm1, "with_skip") else (self.norm1(x), x)
        x = self.dcm(y, residual=x)
        y, x = self.norm2.with_skip(x) if hasattr(self.norm2, "with_skip") else (self.norm2(x), x)
        return self.mlp(y, residual=x)


class DeconverStage(nn.Module):
    """``depth`` blocks at one resolution, behind a bias-free channel adapter when the width
    changes (deconver.py:68-103).  ``spatial_size`` is accepted and unused, as there."""

    def __init__(self, in_channels: int, out_channels: int, spatial_size: Any = None,
                 depth: int = 1, adapter: Any = (Linear, {"bias": False}), **block_kwargs):
        super().__init__()
        if in_channels != out_channels:
            self.adapter = build(adapter, in_channels, out_channels)
        self.blocks = nn.ModuleList(DeconverBlock(out_channels, **block_kwargs)
                                    for _ in range(depth))

    def forward(self, x: Tensor) -> Tensor:
        if hasattr(self, "adapter"):
            x = self.adapter(x)
        for blk in self.blocks:
            x = blk(x)
        return x


class Stem(nn.Sequential):
    """Patchifying stem: strided convolution + norm (deconver.py:106-114)."""

    def __init__(self, in_channels: int, out_channels: int, patch_size: Sequence[int] = (4, 4),
                 norm: Any = LayerNorm):
        # (a convolution whose windows tile the input: same module and parameters, regrouping +
        # GEMMs on the GPU)
        conv = getattr(layers, f"PatchConv{len(patch_size)}d")
        super().__init__(conv(in_channels, out_channels, patch_size, stride=patch_size),
                         build(native_norm(norm), out_channels))


class _Down(nn.Module):
    """One encoder level: resample, then a stage (unet.py:36-60).  Parameter names
    ``downsample.*`` and ``block.*``."""

    def __init__(self, in_channels, out_channels, depth, stride, downsample, **stage_kwargs):
        super().__init__()
        if math.prod(as_tuple(stride)) == 1:
            self.downsample = nn.Identity()
        else:
            # the reference resamples by 2 at every strided level whatever `strides` says
            self.downsample = build(downsample, in_channels, out_channels, stride=2)
        self.block = DeconverStage(out_channels, out_channels, depth=depth, **stage_kwargs)

    def forward(self, x: Tensor) -> Tensor:
        return self.block(self.downsample(x))


class _Up(nn.Module):
    """One decoder level: upsample the coarse map, concatenate the skip in front of it, run
    a stage that first adapts ``2 * out_channels`` back to ``out_channels``
    (unet.py:108-131).  Parameter names ``upsample.*`` and ``block.*``."""

    def __init__(self, in_channels, out_channels, depth, stride, upsample, **stage_kwargs):
        super().__init__()
        self.upsample = build(upsample, in_channels, out_channels, stride=stride)
        self.block = DeconverStage(2 * out_channels, out_channels, depth=depth, **stage_kwargs)

    def forward(self, coarse: Tensor, skip: Tensor) -> Tensor:
        return self.block(torch.cat([skip, self.upsample(coarse)], dim=1))


class _Levels(nn.Module):
    """Holder that gives the levels the parameter prefix ``blocks.{i}``."""

    def __init__(self, levels):
        super().__init__()
        self.blocks = nn.ModuleList(levels)


def _scaled(spatial_size, factor, up):
    if not isinstance(spatial_size, Sequence):
        return spatial_size
    return tuple(d * factor if up else d // factor for d in spatial_size)


class Deconver(nn.Module):
    """Deconver segmentation network (deconver.py:117-154, unet.py:175-276).

    Args:
        in_channels, out_channels: image channels and output (logit) channels.
        spatial_dims: 2 or 3.
        spatial_size: optional input extent, handed down (rescaled) to the stages.
        encoder_depth, encoder_width, strides: blocks, channels and stride per encoder level.
        decoder_depth: blocks per decoder level (one level fewer than the encoder).
        stem: ``None`` for the default bias-free 3-tap convolution; ``nn.Identity`` for none;
            or a class / ``(class, {kwargs})`` spec called as ``stem(in_channels, width0)``.
        downsample, upsample, head: class or ``(class, {kwargs})`` specs; defaults are a
            2-tap strided convolution, a 2-tap transposed convolution and a 1-tap convolution.
        num_deep_supr: ``False`` for one head on the finest map, else the number of finest
            decoder maps that get a head (``True`` means 3); ``forward`` then returns a list.
        **kwargs: go to every ``DeconverStage`` and through it to ``DeconverBlock``,
            ``DeconvMixer`` and ``Deconv`` (``norm``, ``kernel_size``, ``groups``, ``ratio``,
            ``num_iters``, ``mlp_ratio``, ``dropout``, ...).
    """

    def __init__(self, in_channels: int, out_channels: int, spatial_dims: int = 3,
                 spatial_size: Any = None, encoder_depth: Sequence[int] = (1, 1, 1, 1, 1),
                 encoder_width: Sequence[int] = (32, 64, 128, 256, 512),
                 strides: Sequence[Any] = (1, 2, 2, 2, 2),
                 decoder_depth: Sequence[int] = (1, 1, 1, 1), stem: Any = None,
                 downsample: Any = None, upsample: Any = None, head: Any = None,
                 num_deep_supr: Any = False, **kwargs):
        super().__init__()
        self.spatial_dims = spatial_dims
        self.spatial_size = spatial_size
        conv = getattr(nn, f"Conv{spatial_dims}d")
        # same modules and parameters; their 16-bit GPU forward is a regrouping + GEMMs
        pconv = getattr(layers, f"PatchConv{spatial_dims}d")
        ptconv = getattr(layers, f"PatchConvTranspose{spatial_dims}d")
        if stem is None:
            stem = (getattr(layers, f"UnfoldConv{spatial_dims}d"), {"kernel_size": 3, "padding": 1, "bias": False})
        downsample = downsample or (pconv, {"kernel_size": 2})
        upsample = upsample or (ptconv, {"kernel_size": 2})
        head = head or (pconv, {"kernel_size": 1})

        if stem is nn.Identity:
            self.stem, width0 = nn.Identity(), in_channels
        else:
            width0 = encoder_width[0]
            self.stem = build(stem, in_channels, width0)

        size = spatial_size
        widths = [width0, *encoder_width]
        downs = []
        for i, depth in enumerate(encoder_depth):
            size = _scaled(size, strides[i], up=False)
            downs.append(_Down(widths[i], widths[i + 1], depth, strides[i], downsample,
                               spatial_size=size, **kwargs))
        self.encoder = _Levels(downs)

        rev_w = list(encoder_width)[::-1]
        rev_s = list(strides)[::-1]
        ups = []
        for i, depth in enumerate(decoder_depth):
            size = _scaled(size, rev_s[i], up=True)
            ups.append(_Up(rev_w[i], rev_w[i + 1], depth, rev_s[i], upsample,
                           spatial_size=size, **kwargs))
        self.decoder = _Levels(ups)

        if num_deep_supr in (False, None):
            self.num_deep_supr = False
            self.head = build(head, encoder_width[0], out_channels)
        else:
            self.num_deep_supr = 3 if num_deep_supr is True else int(num_deep_supr)
            self.heads = nn.ModuleList(build(head, encoder_width[j], out_channels)
                                       for j in range(self.num_deep_supr))

    def forward_features(self, x: Tensor) -> list[Tensor]:
        """Feature pyramid, finest first: decoder outputs where the decoder reaches, encoder
        outputs below."""
        feats = []
        cur = self.stem(x)
        for level in self.encoder.blocks:
            cur = level(cur)
            feats.append(cur)
        for i, level in enumerate(self.decoder.blocks):
            feats[-2 - i] = level(feats[-1 - i], feats[-2 - i])
        return feats

    def forward(self, x: Tensor):
        feats = self.forward_features(x)
        if self.num_deep_supr:
            return [h(feats[j]) for j, h in enumerate(self.heads)]
        return self.head(feats[0])
