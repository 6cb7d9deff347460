"""On/off patterns of a Deconver network's rectifiers, for gradient comparisons between two
evaluations of one network (float32 on the HIP route against float64, say).

The network has two kinds of kinked nonlinearity: the mixer's activation (``nn.ReLU`` on
``in_proj(x)``, deconver.py:29-46 of the reference) and the rectifier of the NDC source
initialisation (``relu(W x + b)``, deconv.py:40-45).  A unit whose pre-activation lies within
rounding of zero may be on in one evaluation and off in the other, and one such unit moves a
weight gradient by a finite amount.  The functions here

* record the pattern an evaluation computed (``record_patterns``),
* compare it with another evaluation's pre-activations (``switched_units``),
* and evaluate a network with a recorded pattern imposed (``imposed_patterns``), so that a
  gradient difference can be attributed to the switched units -- or not.
"""

from __future__ import annotations

import contextlib
from typing import Callable, Dict

import torch
import torch.nn.functional as F
from torch import nn

import deconver_amd as dc
from deconver_amd import ndc as ndc_module


def _kinked(model: nn.Module):
    """(name, kind, module) of every rectifier: mixer activations that are ReLUs, NDC layers."""
    for name, mod in model.named_modules():
        if isinstance(mod, dc.DeconvMixer) and isinstance(mod.act, nn.ReLU):
            yield name + ".act", "act", mod
        if isinstance(mod, dc.Deconv):
            yield name + ".source", "source", mod


def record_patterns(model: nn.Module, run: Callable[[], None], keep_pre: bool = False):
    """Runs ``run()`` (a forward of ``model``) and returns ``{name: mask}``: which units of each
    rectifier were on, as the route that ran computed them -- on the HIP route the kernels'
    ``z + b > 0`` from the very ``z`` handed to them.  ``keep_pre``: also the pre-activations."""
    masks: Dict[str, torch.Tensor] = {}
    pres: Dict[str, torch.Tensor] = {}
    handles = []
    current = {}

    def note(name, pre):
        masks[name] = (pre > 0).detach()
        if keep_pre:
            pres[name] = pre.detach().clone()

    for name, kind, mod in _kinked(model):
        if kind == "act":
            handles.append(mod.act.register_forward_hook(
                lambda m, inp, out, name=name: note(name, inp[0])))
        else:
            handles.append(mod.register_forward_pre_hook(
                lambda m, inp, name=name: current.__setitem__("name", name)))
            # general route: the projection's output is the pre-activation
            handles.append(mod.init.linear.register_forward_hook(
                lambda m, inp, out, name=name: note(name, out)))

    original = ndc_module.deconv_update

    def recording_update(x, z, h, bias, **kw):
        if kw.get("relu_input"):   # HIP route, first iteration: the kernels rectify z + b
            b = 0 if bias is None else bias.view(1, -1, *([1] * (z.dim() - 2)))
            note(current["name"], z.float() + b)
        return original(x, z, h, bias, **kw)

    original_projected = ndc_module.projected_update

    def recording_projected(x, weight, h, bias, **kw):
        # HIP route, first iteration: projection and update are one node; its z is this GEMM
        # (the same call on the same operands gives the same bits)
        w = weight.detach().to(x.dtype)
        z = torch.bmm(w.unsqueeze(0).expand(x.shape[0], -1, -1), x.flatten(2))
        z = z.view(x.shape[0], -1, *x.shape[2:])
        b = 0 if bias is None else bias.view(1, -1, *([1] * (z.dim() - 2)))
        note(current["name"], z.float() + b)
        return original_projected(x, weight, h, bias, **kw)

    ndc_module.deconv_update = recording_update
    ndc_module.projected_update = recording_projected
    try:
        run()
    finally:
        ndc_module.deconv_update = original
        ndc_module.projected_update = original_projected
        for hd in handles:
            hd.remove()
    return (masks, pres) if keep_pre else masks


def switched_units(masks: Dict[str, torch.Tensor], pres: Dict[str, torch.Tensor]):
    """Per rectifier: (number of units whose recorded on/off state differs from the sign of
    ``pres``, the largest ``|pre|`` among them relative to the layer's largest ``|pre|``)."""
    out = {}
    for name, mask in masks.items():
        pre = pres[name]
        sw = mask.to(pre.device) != (pre > 0)
        n = int(sw.sum())
        rel = float(pre[sw].abs().max() / pre.abs().max()) if n else 0.0
        out[name] = (n, rel)
    return out


class _Gate(nn.Module):
    def __init__(self, mask):
        super().__init__()
        self.mask = mask

    def forward(self, x):
        return x * self.mask.to(device=x.device, dtype=x.dtype)


@contextlib.contextmanager
def imposed_patterns(model: nn.Module, masks: Dict[str, torch.Tensor]):
    """Inside the block every rectifier of ``model`` lets through exactly the units that are on
    in ``masks`` (``x * mask`` instead of ``relu(x)``).  For networks on the general route."""
    undo = []
    for name, kind, mod in _kinked(model):
        mask = masks[name]
        if kind == "act":
            undo.append((mod, "act", mod.act))
            mod.act = _Gate(mask)
        else:
            init = mod.init

            def gated(x, init=init, mask=mask):
                pre = init.linear(x)
                h = init.h0.expand(x.shape[0], *init.h0.shape)
                return pre * mask.to(device=pre.device, dtype=pre.dtype), F.relu(h)

            undo.append((init, "forward", None))
            init.forward = gated
    try:
        yield
    finally:
        for obj, attr, old in undo:
            if old is None:
                del obj.forward        # back to the class's method
            else:
                setattr(obj, attr, old)


def grad_errors(grads, ref_grads):
    """{name: (max|d| / max|ref|, cosine)}"""
    out = {}
    for name, g in grads.items():
        a, b = g.double().flatten(), ref_grads[name].double().flatten().to(g.device)
        err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-300))
        cos = float(torch.dot(a, b) / (a.norm() * b.norm()).clamp_min(1e-300))
        out[name] = (err, cos)
    return out


def audit_gradients(grads, masks, exact: nn.Module, run_exact: Callable[[], Dict[str, torch.Tensor]],
                    tol: float = 2e-2, cos_min: float = 0.9999, gated_tol: float = None,
                    max_switched: int = 16, max_switched_frac: float = 1e-6,
                    borderline: float = 1e-5):
    """Holds ``grads`` (of the network whose rectifier patterns are ``masks``) to the gradients
    of ``exact`` (same network, higher precision; ``run_exact()`` runs its forward + backward
    and returns its parameter gradients): every tensor within ``tol`` of its largest entry and
    at a cosine above ``cos_min``.

    A tensor outside that is accepted only with its cause shown: some rectifier units differ
    between the two evaluations, at most ``max_switched`` per rectifier (or the fraction
    ``max_switched_frac`` of its units, whichever is more), each with an exact pre-activation
    within ``borderline`` of the layer's largest (i.e. within the other evaluation's rounding
    of zero) -- and with the first evaluation's patterns imposed on ``exact``, EVERY tensor is
    within ``gated_tol`` (default: ``tol``) and ``cos_min``.  With ``gated_tol`` given, that
    second comparison is made whether or not the first one found an outlier: on one and the
    same on/off pattern the two evaluations differ by rounding only, so it can be much
    tighter than ``tol``.  Returns a report; raises AssertionError otherwise."""
    holder = {}

    def run_and_keep():
        holder["g"] = run_exact()

    _, pres = record_patterns(exact, run_and_keep, keep_pre=True)
    errs = grad_errors(grads, holder["g"])
    bad = {k: v for k, v in errs.items() if not (v[0] < tol and v[1] > cos_min)}
    sw = switched_units(masks, pres)
    report = {"errors": errs, "outliers": bad, "switched": {k: v for k, v in sw.items() if v[0]},
              "gated_errors": None}
    if bad:
        assert report["switched"], f"gradients differ with identical rectifier patterns: {bad}"
    for name, (n, rel) in report["switched"].items():
        assert n <= max(max_switched, max_switched_frac * masks[name].numel()), \
            f"{name}: {n} rectifier units differ, not a borderline case ({bad})"
        assert rel <= borderline, f"{name}: a switched unit lies {rel:.1e} of the layer's scale from zero ({bad})"
    if not bad and gated_tol is None:
        return report
    exact.zero_grad(set_to_none=True)
    with imposed_patterns(exact, masks):
        gated = run_exact()
    gerrs = grad_errors(grads, gated)
    report["gated_errors"] = gerrs
    gtol = tol if gated_tol is None else gated_tol
    still = {k: v for k, v in gerrs.items() if not (v[0] < gtol and v[1] > cos_min)}
    assert not still, f"not explained by the switched units {report['switched']}: {still}"
    return report
