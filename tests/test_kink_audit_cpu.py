"""The machinery behind the full-width network test's gradient criterion (tests/kink_audit.py),
exercised on the CPU in float64: a gradient outlier is accepted only when switched borderline
rectifier units explain it, and a planted error is not explained."""

import copy

import pytest
import torch
from torch import nn

import deconver_amd as dc
from tests import kink_audit as KA

NET = dict(in_channels=3, out_channels=1, spatial_dims=2, encoder_depth=(1, 1),
           encoder_width=(8, 16), strides=(1, 2), decoder_depth=(1,), kernel_size=(5, 5),
           groups=-1, ratio=4, norm=nn.InstanceNorm2d)


def _setup():
    torch.manual_seed(0)
    model = dc.Deconver(**NET).double()
    x = torch.rand(2, 3, 16, 16, dtype=torch.float64)
    g = torch.randn(2, 1, 16, 16, dtype=torch.float64)

    def run(m):
        m.zero_grad(set_to_none=True)
        m(x).backward(g)
        return {n: p.grad.detach().clone() for n, p in m.named_parameters()}
    return model, run


def _borderline_case():
    """`model` and a copy whose one borderline source unit is switched: the copy's first NDC
    layer gets its bias moved so that the pre-activation closest to zero sits at +1e-12, and
    the 'other evaluation' has that unit off."""
    model, run = _setup()
    masks, pres = KA.record_patterns(model, lambda: run(model), keep_pre=True)
    name = next(k for k in masks if k.endswith(".source"))
    pre = pres[name]
    idx = pre.abs().argmin()
    ch = int(torch.unravel_index(idx, pre.shape)[1])
    layer = dict(model.named_modules())[name[: -len(".source")]]
    with torch.no_grad():
        layer.init.linear.linear.bias[ch] -= pre.flatten()[idx] - 1e-12
    masks, pres = KA.record_patterns(model, lambda: run(model), keep_pre=True)
    assert 0 < float(pres[name].flatten()[idx]) < 1e-9
    other = {k: v.clone() for k, v in masks.items()}
    other[name].view(-1)[idx] = False     # the evaluation that rounded the other way
    with KA.imposed_patterns(model, other):
        grads_other = run(model)
    return model, run, other, grads_other


def test_patterns_recorded_on_the_general_route_and_imposed():
    model, run = _setup()
    grads = run(model)
    masks = KA.record_patterns(model, lambda: run(model))
    assert any(k.endswith(".act") for k in masks) and any(k.endswith(".source") for k in masks)
    with KA.imposed_patterns(model, masks):   # its own pattern: same function, same gradients
        again = run(model)
    for k in grads:
        assert torch.allclose(grads[k], again[k], rtol=1e-12, atol=1e-14)
    assert type(model.encoder.blocks[0].block.blocks[0].dcm.act) is nn.ReLU   # put back
    for k, g2 in run(model).items():
        assert torch.equal(g2, grads[k])


def test_switched_borderline_unit_is_found_and_explains_the_outlier():
    model, run, other, grads_other = _borderline_case()
    plain = KA.grad_errors(grads_other, run(model))
    assert max(e for e, _ in plain.values()) > 1e-6   # the switched unit moves some gradient
    report = KA.audit_gradients(grads_other, other, model, lambda: run(model), tol=1e-9, cos_min=0.0,
                                borderline=1e-9)
    assert report["outliers"], "the case must need the explanation"
    assert sum(n for n, _ in report["switched"].values()) == 1
    assert max(e for e, _ in report["gated_errors"].values()) < 1e-9


def test_planted_error_is_not_explained():
    model, run, other, grads_other = _borderline_case()
    name = next(k for k in grads_other if k.endswith("deconv.init.h0"))
    planted = {k: v.clone() for k, v in grads_other.items()}
    planted[name].view(-1)[3] += 3e-2 * planted[name].abs().max()
    with pytest.raises(AssertionError, match="not explained"):
        KA.audit_gradients(planted, other, model, lambda: run(model), tol=2e-2)
    with pytest.raises(AssertionError, match="not explained"):   # ... nor a 2e-3 one, on equal patterns
        small = {k: v.clone() for k, v in grads_other.items()}
        small[name].view(-1)[3] += 2e-3 * small[name].abs().max()
        KA.audit_gradients(small, other, model, lambda: run(model), tol=2e-2, gated_tol=1e-3)
    # and with identical patterns there is nothing to blame at all
    masks = KA.record_patterns(model, lambda: run(model))
    mine = run(model)
    mine[name].view(-1)[3] += 3e-2 * mine[name].abs().max()
    with pytest.raises(AssertionError, match="identical rectifier patterns"):
        KA.audit_gradients(mine, masks, model, lambda: run(model), tol=2e-2)
