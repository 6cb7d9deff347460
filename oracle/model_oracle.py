"""CPU oracle for the Deconver network: its forward pass as ONE function over a state dict.

TEST INFRASTRUCTURE ONLY (see ``oracle/ndc_oracle.py``): used by ``tests/`` to check the
module-based model of the package, never imported by it.

``deconver_forward(state, x, cfg)`` restates, with ``torch.nn.functional`` calls only and no
``nn.Module`` of the package, what the reference's model computes
(``deconver/deconver.py:9-154`` on ``deconver/unet.py:36-276``):

* stem: bias-free 3-tap convolution, padding 1 (``deconver.py:136-140``);
* encoder level i: 2-tap stride-2 convolution when ``strides[i] != 1`` (``unet.py:50-58``,
  always a factor 2), then ``encoder_depth[i]`` blocks;
* decoder level i: 2-tap transposed convolution with ``stride = strides[::-1][i]``,
  ``cat([skip, up], 1)``, bias-free 1x1 adapter ``2w -> w``, then blocks
  (``unet.py:108-131``, ``deconver.py:84-103``);
* block: ``x + dcm(norm1(x))`` then ``x + mlp(norm2(x))`` (``deconver.py:62-65``); the norm is
  instance norm without affine parameters (the reference's published configurations) or the
  channel layer norm of ``layers/norm.py:28-34`` when the state dict holds its weights;
* dcm: 1x1 ``in_proj`` (no bias), ReLU, the NDC layer (``OracleNDC.forward``, the literal
  form of ``deconver/deconvolution/reference.py``), 1x1 ``out_proj`` (``deconver.py:29-46``);
* mlp: 1x1, exact GELU, 1x1 (``layers/mlp.py:55-63``);
* head: 1x1 convolution on the finest decoder map (``unet.py:250-251,266-276``).

It consumes parameters by the reference's state-dict names, so a missing or misnamed key
fails loudly.  Pinned by: the published parameter counts of the reference's README
(ISLES'22 configuration 10.5 M, BraTS'23 configuration 10.6 M), and library routines for
every piece except the NDC layer, which ``tests/test_oracle_pins.py`` pins.
"""

from __future__ import annotations

from typing import Dict, Sequence

import torch
import torch.nn.functional as F

from .ndc_oracle import OracleNDC

_CONV = {2: F.conv2d, 3: F.conv3d}
_TCONV = {2: F.conv_transpose2d, 3: F.conv_transpose3d}


def _pointwise(x, w, b=None):
    """1x1 projection over channels of a ``(B, C, *S)`` tensor (weight ``(Cout, Cin, 1)``)."""
    y = F.conv1d(x.flatten(2), w, b)
    return y.view(x.shape[0], -1, *x.shape[2:])


def _norm(state: Dict[str, torch.Tensor], prefix: str, x):
    if prefix + ".norm.weight" in state:  # channel layer norm
        y = F.layer_norm(x.movedim(1, -1), (x.shape[1],), state[prefix + ".norm.weight"],
                         state[prefix + ".norm.bias"])
        return y.movedim(-1, 1)
    return F.instance_norm(x)


def _block(state, prefix, x, cfg):
    c = x.shape[1]
    ndc = OracleNDC(c, cfg["kernel_size"], ratio=cfg.get("ratio", 4), groups=cfg.get("groups", -1),
                    num_iters=cfg.get("num_iters", 1))
    u = _norm(state, prefix + ".norm1", x)
    u = cfg.get("act_fn", torch.relu)(_pointwise(u, state[prefix + ".dcm.in_proj.linear.weight"]))
    u = ndc.forward(u, state[prefix + ".dcm.deconv.init.linear.linear.weight"].squeeze(-1),
                    state[prefix + ".dcm.deconv.init.linear.linear.bias"],
                    state[prefix + ".dcm.deconv.init.h0"])
    u = _pointwise(u, state[prefix + ".dcm.out_proj.linear.weight"],
                   state[prefix + ".dcm.out_proj.linear.bias"])
    x = x + u
    v = _norm(state, prefix + ".norm2", x)
    v = _pointwise(v, state[prefix + ".mlp.block.0.linear.weight"],
                   state[prefix + ".mlp.block.0.linear.bias"])
    v = F.gelu(v)
    v = _pointwise(v, state[prefix + ".mlp.block.3.linear.weight"],
                   state[prefix + ".mlp.block.3.linear.bias"])
    return x + v


def deconver_forward(state: Dict[str, torch.Tensor], x: torch.Tensor, cfg: dict):
    """Logits of the network with parameters ``state`` for input ``x``.

    ``cfg``: ``spatial_dims``, ``encoder_depth``, ``strides``, ``decoder_depth``,
    ``kernel_size`` and optionally ``ratio``, ``groups``, ``num_iters``, ``act_fn`` (the
    mixer's activation as a function, default ``torch.relu``).
    """
    nd = cfg["spatial_dims"]
    enc_depth: Sequence[int] = cfg["encoder_depth"]
    dec_depth: Sequence[int] = cfg["decoder_depth"]
    strides = list(cfg["strides"])
    feats = []
    cur = _CONV[nd](x, state["stem.weight"], None, padding=1)
    for i, depth in enumerate(enc_depth):
        p = f"encoder.blocks.{i}"
        if strides[i] != 1:
            cur = _CONV[nd](cur, state[p + ".downsample.weight"], state[p + ".downsample.bias"],
                            stride=2)
        for j in range(depth):
            cur = _block(state, f"{p}.block.blocks.{j}", cur, cfg)
        feats.append(cur)
    rev = strides[::-1]
    for i, depth in enumerate(dec_depth):
        p = f"decoder.blocks.{i}"
        up = _TCONV[nd](feats[-1 - i], state[p + ".upsample.weight"], state[p + ".upsample.bias"],
                        stride=rev[i])
        cur = torch.cat([feats[-2 - i], up], dim=1)
        cur = _pointwise(cur, state[p + ".block.adapter.linear.weight"])
        for j in range(depth):
            cur = _block(state, f"{p}.block.blocks.{j}", cur, cfg)
        feats[-2 - i] = cur
    return _CONV[nd](feats[0], state["head.weight"], state["head.bias"])
