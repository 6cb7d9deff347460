"""CPU oracle for the NDC (nonnegative deconvolution) source update.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file: it is
used by ``tests/``, by ``__graft_entry__.smoke()`` as the checker, and by the
``cpu_baseline`` leg of ``bench.py``.

It restates, in plain PyTorch (CPU, any float dtype incl. float64), the algorithm of
the reference layer:

* ``conv_batched``        follows ``deconver/deconvolution/reference.py:33-52``
                          (per-sample conv by folding the batch into groups),
* ``swap_io`` / ``flip_taps``  follow ``reference.py:64-69`` (``t`` and ``flip``),
* ``OracleNDC.init_source_filter`` follows ``reference.py:113-118`` and
                          ``deconver/layers/linear.py:53-58`` (1x1 projection on the
                          flattened volume, then ReLU; ReLU of the batch-expanded filter),
* ``OracleNDC.update_s``  follows ``reference.py:169-173``,
* ``OracleNDC.iterate``   follows ``reference.py:181-207`` (``update``/``context``/
                          ``iterative_update`` incl. the truncated back-propagation),
* ``OracleNDC.forward``   follows ``reference.py:254-273`` (init, channel split
                          ``b (g c) ... -> (b g) c ...``, iterate, merge),
* ``op_K`` / ``op_A`` / ``update_grouped`` / ``update_backward`` restate the grouped
  form and its analytic gradients documented at
  ``deconver/deconvolution/functional.py:1-21,97-182`` and ``kernels.py:32-39``,
* ``rel_err``             follows ``tests/test_deconv_equivalence.py:51-59``.

Parity pinning (see tests/test_oracle_pins.py): the reference's own tests hold no
stored vectors for this path, so every function here is pinned by what the mathematics
fixes: brute-force loops in C (oracle/ndc_bruteforce.c) on small shapes incl. borders
and groups not in {1, C}; the adjoint identity <K u, v> = <u, A v>; delta-kernel,
fixed-point, scaling-law and constant-field closed forms of the update; float64
``gradcheck`` and literal-form autograd for the analytic gradients; the
truncated-backprop contract for ``num_grad_iters``.
"""

from __future__ import annotations

import math
from contextlib import nullcontext
from typing import Optional, Sequence

import torch
import torch.nn.functional as F

_CONVND = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}


# --------------------------------------------------------------------------- literal form


def conv_batched(inp: torch.Tensor, weight: torch.Tensor, padding, groups: int = 1):
    """Per-sample convolution: sample ``n`` of ``inp`` is correlated with ``weight[n]``.

    ``inp`` is ``(N, Cin, *S)``, ``weight`` is ``(N, Cout, Cin/groups, *k)``.  The batch
    is folded into the group axis so that one grouped cross-correlation does the work.
    """
    n = inp.shape[0]
    nd = inp.dim() - 2
    folded_in = inp.reshape(1, n * inp.shape[1], *inp.shape[2:])
    folded_w = weight.reshape(n * weight.shape[1], weight.shape[2], *weight.shape[3:])
    out = _CONVND[nd](folded_in, folded_w, groups=groups * n, padding=padding)
    return out.reshape(n, -1, *out.shape[2:])


def swap_io(h: torch.Tensor) -> torch.Tensor:
    """Swap the out/in channel axes of a batched filter ``(N, out, in, *k)``."""
    return h.transpose(1, 2)


def flip_taps(h: torch.Tensor) -> torch.Tensor:
    """Reverse every spatial axis of a batched filter ``(N, out, in, *k)``."""
    return torch.flip(h, dims=tuple(range(3 - h.dim(), 0)))


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """``max|a-b| / max|b|`` in float64 (tensor-scale normalised)."""
    diff = (a.double() - b.double()).abs().max()
    scale = b.double().abs().max().clamp_min(1e-30)
    return (diff / scale).item()


class OracleNDC:
    """Functional restatement of the original layer (no nn.Module machinery).

    Parameters are passed in explicitly so that the HIP module and the oracle can share
    one set of weights: ``weight`` is the projection ``(G*sc, C)``, ``bias`` ``(G*sc,)``,
    ``h0`` ``(C, sc, *k)``.
    """

    def __init__(self, channels: int, kernel_size: Sequence[int], source_channels=None,
                 ratio: float = 1, groups: int = -1, eps: float = 1e-16,
                 num_iters: int = 1, num_grad_iters: Optional[int] = None):
        self.channels = channels
        self.groups = channels if groups == -1 else groups
        assert channels % self.groups == 0
        self.source_channels = round(
            channels * ratio / self.groups if source_channels is None else source_channels
        )
        self.kernel_size = tuple(kernel_size)
        self.padding = tuple(k // 2 for k in self.kernel_size)
        self.eps = eps
        self.num_iters = num_iters
        self.num_grad_iters = num_iters if num_grad_iters is None else num_grad_iters

    # -- pieces ---------------------------------------------------------------------
    def init_source_filter(self, x, weight, bias, h0, gate=None):
        b = x.shape[0]
        z = F.conv1d(x.flatten(2), weight.reshape(weight.shape[0], -1, 1), bias)
        z = z.view(b, -1, *x.shape[2:])
        h = h0.expand(b, *h0.shape)
        # `gate` (no counterpart in the reference): an on/off pattern for the source's rectifier
        # given from outside instead of taken from the sign of z.  A low-precision route may
        # switch a unit whose pre-activation is within its rounding of zero; parity tests that
        # want the arithmetic, not those switches, evaluate the oracle on the route's pattern.
        s0 = F.relu(z) if gate is None else z * gate.to(z.dtype)
        return s0, F.relu(h)

    def split(self, t):  # "b (g c) ... -> (b g) c ..."
        b = t.shape[0]
        g = self.groups
        return t.reshape(b * g, t.shape[1] // g, *t.shape[2:])

    def merge(self, t):  # "(b g) c ... -> b (g c) ..."
        g = self.groups
        return t.reshape(t.shape[0] // g, g * t.shape[1], *t.shape[2:])

    def update_s(self, x, s, h):
        ht = swap_io(flip_taps(h))
        num = conv_batched(x, ht, self.padding) + self.eps
        den = conv_batched(conv_batched(s, h, self.padding), ht, self.padding) + self.eps
        return s * num / den

    def iterate(self, x, s, h):
        for it in range(1, self.num_iters + 1):
            cut = it < self.num_iters - self.num_grad_iters + 1
            with (torch.no_grad() if cut else nullcontext()):
                s = self.update_s(x, s, h)
        return s

    # -- whole layer ------------------------------------------------------------------
    def forward(self, x, weight, bias, h0, gate=None):
        s, h = self.init_source_filter(x, weight, bias, h0, gate)
        if self.groups != 1:
            x, s, h = self.split(x), self.split(s), self.split(h)
        s = self.iterate(x, s, h)
        if self.groups != 1:
            s = self.merge(s)
        return s


# --------------------------------------------------------------------------- grouped form


def _hview(h, groups, m, sc):
    ks = tuple(h.shape[2:])
    return h.reshape(groups, m, sc, *ks), ks


def op_K(u, h, groups, m, sc):
    """``K(u)[o,p] = sum_{i,tau} u[i, p+tau-pad] h[o,i,tau]`` per group: (B,G*sc,*S)->(B,G*m,*S)."""
    hv, ks = _hview(h, groups, m, sc)
    w = hv.reshape(groups * m, sc, *ks)
    return _CONVND[len(ks)](u, w, groups=groups, padding=tuple(k // 2 for k in ks))


def op_A(v, h, groups, m, sc):
    """``A(v)[i,p] = sum_{o,tau} v[o, p+pad-tau] h[o,i,tau]`` per group: (B,G*m,*S)->(B,G*sc,*S)."""
    hv, ks = _hview(h, groups, m, sc)
    nd = len(ks)
    w = hv.flip(dims=tuple(range(-nd, 0))).transpose(1, 2).reshape(groups * sc, m, *ks)
    return _CONVND[nd](v, w, groups=groups, padding=tuple(k // 2 for k in ks))


def rectified_source(z, bias, relu_input):
    s = z if bias is None else z + bias.view(1, -1, *([1] * (z.dim() - 2)))
    return torch.relu(s) if relu_input else s


def update_grouped(x, z, h, bias, groups, m, sc, eps, relu_input):
    """One update in grouped form; returns ``(out, t1)``."""
    s = rectified_source(z, bias, relu_input)
    t1 = op_K(s, h, groups, m, sc)
    out = s * (op_A(x, h, groups, m, sc) + eps) / (op_A(t1, h, groups, m, sc) + eps)
    return out, t1


def _shifted_products(a, bt, ks, groups, ca, cb):
    """``out[g,ca,cb,tau] = sum_{b,p} a[b,g,ca,p] * bt[b,g,cb,p+pad-tau]`` by explicit shifts."""
    nd = len(ks)
    bsz = a.shape[0]
    sp = a.shape[2:]
    av = a.reshape(bsz, groups, ca, *sp)
    pads = []
    for k in reversed(ks):
        pads += [k // 2, k // 2]
    btp = F.pad(bt, pads).reshape(bsz, groups, cb, *[s + 2 * (k // 2) for s, k in zip(sp, ks)])
    out = a.new_zeros(groups, ca, cb, *ks)
    red = [0] + list(range(4, 4 + nd))
    for tau in _ndrange(ks):
        # position p reads bt at p + pad - tau  ->  index p + 2*pad - tau of the padded tensor
        sl = tuple(slice(2 * (k // 2) - t_, 2 * (k // 2) - t_ + n)
                   for t_, k, n in zip(tau, ks, sp))
        shifted = btp[(slice(None), slice(None), slice(None)) + sl]
        val = (av.unsqueeze(3) * shifted.unsqueeze(2)).sum(dim=red)
        out[(slice(None), slice(None), slice(None)) + tau] = val
    return out


def _ndrange(ks):
    if len(ks) == 0:
        yield ()
        return
    for i in range(ks[0]):
        for rest in _ndrange(ks[1:]):
            yield (i,) + rest


def update_backward(x, z, h, bias, gout, groups, m, sc, eps, relu_input):
    """Analytic gradients of ``update_grouped`` w.r.t. ``(x, z, h, bias)``.

    With ``n = A(x)+eps``, ``d = A(t1)+eps``, ``s = relu(z+b)``:
    ``gn = g*s/d``; ``gd = -gn*n/d``; ``gt1 = K(gd)``; ``gx = K(gn)``;
    ``gz = [z+b>0] * (g*n/d + A(gt1))``; ``gb = sum_{b,p} gz``;
    ``gh[o,i,tau] = sum_{b,p} gt1[o,p] s[i,p+tau-pad] + gn[i,p] x[o,p+pad-tau]
    + gd[i,p] t1[o,p+pad-tau]``.
    """
    ks = tuple(h.shape[2:])
    s = rectified_source(z, bias, relu_input)
    t1 = op_K(s, h, groups, m, sc)
    n = op_A(x, h, groups, m, sc) + eps
    d = op_A(t1, h, groups, m, sc) + eps
    gn = gout * s / d
    gd = -gn * n / d
    gt1 = op_K(gd, h, groups, m, sc)
    gx = op_K(gn, h, groups, m, sc)
    gz = gout * n / d + op_A(gt1, h, groups, m, sc)
    if relu_input:
        pre = z if bias is None else z + bias.view(1, -1, *([1] * (z.dim() - 2)))
        # as autograd of torch.relu: zero where the pre-activation is <= 0, so a NaN passes
        gz = torch.where(pre <= 0, torch.zeros_like(gz), gz)
    gb = gz.sum(dim=[0] + list(range(2, gz.dim())))
    # filter gradient: (G, sc, m, *k) products, then swap to (G, m, sc, *k)
    gh_a = _shifted_products(gn, x, ks, groups, sc, m) + _shifted_products(gd, t1, ks, groups, sc, m)
    # first term: sum_p gt1[o,p] s[i,p+tau-pad] = sum_q s[i,q] gt1[o,q+pad-tau]
    gh_f = _shifted_products(s, gt1, ks, groups, sc, m)
    gh = (gh_a + gh_f).transpose(1, 2).reshape_as(h)
    return gx, gz, gh, gb


def layer_forward_grouped(x, weight, bias, h0, groups, sc, eps=1e-16, num_iters=1,
                          num_grad_iters=None):
    """Whole layer in grouped form (batch-invariant filter); differentiable by autograd."""
    num_grad_iters = num_iters if num_grad_iters is None else num_grad_iters
    c = x.shape[1]
    m = c // groups
    h = F.relu(h0)
    z = F.conv1d(x.flatten(2), weight.reshape(weight.shape[0], -1, 1), None)
    z = z.view(x.shape[0], -1, *x.shape[2:])
    s, b, relu = z, bias, True
    for it in range(1, num_iters + 1):
        cut = it < num_iters - num_grad_iters + 1
        with (torch.no_grad() if cut else nullcontext()):
            s, _ = update_grouped(x, s, h, b, groups, m, sc, eps, relu)
        b, relu = None, False
    return s


# --------------------------------------------------------------------------- init helpers


def default_parameters(channels, kernel_size, source_channels, groups, generator=None,
                       dtype=torch.float32):
    """Parameters with the same distributions as the reference initialiser
    (``reference.py:105-111``): kaiming-uniform(a=sqrt(5)) filter, Conv1d-default projection."""
    h0 = torch.empty(channels, source_channels, *kernel_size, dtype=dtype)
    torch.nn.init.kaiming_uniform_(h0, a=math.sqrt(5), generator=generator)
    out_ch = groups * source_channels
    w = torch.empty(out_ch, channels, 1, dtype=dtype)
    torch.nn.init.kaiming_uniform_(w, a=math.sqrt(5), generator=generator)
    bound = 1.0 / math.sqrt(channels)
    b = torch.empty(out_ch, dtype=dtype).uniform_(-bound, bound, generator=generator)
    return w, b, h0
