"""Where the bfloat16 layer's input gradient loses accuracy, shown on the CPU.

The HIP route's arithmetic is reproduced with the host build of the kernels (same kernel
sources, bf16 storage, dot2 products) around a bf16-rounded projection, and compared with a
float64 evaluation of the unrounded layer.  The finding this pins: the update's kernels are
not what puts dx 3e-2 from float64 on this case -- a handful of source units whose exact
pre-activation z + b lies within bf16 rounding of zero come out switched, and each switched
unit moves dx by a finite amount.  On the on/off pattern the route computed, every output
is well inside the 2e-2 bf16 bound.
"""

import torch

import deconver_amd as dc
from deconver_amd import ops
from oracle import ndc_oracle as O
from tests.helpers import hostcheck_library

C, SC = 16, 4


def _route_on_host(x0, g0, W, b, h0):
    """(out, dx, gh0, gb, gW, gate) of the layer computed the way the HIP route does under
    bf16 autocast: bf16 x and W, bias-free bf16 projection, bias + ReLU on load in the update,
    bf16 gx / gz, bf16 sum of the two input-gradient terms."""
    lib = hostcheck_library()
    h = torch.relu(h0).float().contiguous()
    xb, Wb = x0.bfloat16().contiguous(), W.bfloat16()
    z = torch.einsum("oc,bcdhw->bodhw", Wb.float(), xb.float()).bfloat16().contiguous()
    kw = dict(groups=C, m=1, sc=SC, eps=1e-16, relu_input=True)
    out, t1, saved = ops.update_forward(lib, xb, z, h, b, save_ratio=True, **kw)
    gx, gz, gh, gb = ops.update_backward(lib, xb, z, t1, h, b, g0.bfloat16().contiguous(),
                                         saved=saved, **kw)
    back = torch.einsum("oc,bodhw->bcdhw", Wb.float(), gz.float()).bfloat16().float()
    dx = (gx.float() + back).bfloat16().float()
    gW = torch.einsum("bodhw,bcdhw->oc", gz.float(), xb.float())
    gate = (z.float() + b.view(1, -1, 1, 1, 1)) > 0
    return out.float(), dx, gh * (h0 > 0), gb, gW, gate


def _float64(x0, g0, W, b, h0, gate=None):
    oracle = O.OracleNDC(C, (3, 3, 3), ratio=4)
    leaves = [t.double().requires_grad_(True) for t in (x0, W, b, h0)]
    y = oracle.forward(*leaves, gate=gate)
    y.backward(g0.double())
    return y.detach(), leaves[0].grad, leaves[3].grad, leaves[2].grad, leaves[1].grad


def test_bf16_layer_dx_error_is_switched_rectifier_units():
    torch.manual_seed(1)
    x0 = torch.rand(2, C, 9, 8, 10)
    g0 = torch.randn(2, C * SC, 9, 8, 10)
    torch.manual_seed(0)
    layer = dc.Deconv(channels=C, kernel_size=(3, 3, 3), ratio=4, groups=-1)
    W = layer.init.linear.linear.weight.detach().squeeze(-1).contiguous()
    b = (layer.init.linear.linear.bias.detach() + 1.0).contiguous()
    h0 = layer.init.h0.detach()

    got = _route_on_host(x0, g0, W, b, h0)
    gate = got[5]
    exact = _float64(x0, g0, W, b, h0)
    same_pattern = _float64(x0, g0, W, b, h0, gate=gate)

    z_exact = torch.einsum("oc,bcdhw->bodhw", W.double(), x0.double()) + b.double().view(1, -1, 1, 1, 1)
    switched = gate != (z_exact > 0)
    assert 0 < switched.sum().item() <= 8                  # a handful of 92 160 units ...
    assert z_exact[switched].abs().max().item() < 5e-3     # ... all within bf16 rounding of zero
    names = ("out", "dx", "gh0", "gb", "gW")
    on_pattern = {n: O.rel_err(a, r) for n, a, r in zip(names, got, same_pattern)}
    vs_exact = {n: O.rel_err(a, r) for n, a, r in zip(names, got, exact)}
    assert all(v < 2e-2 for v in on_pattern.values()), on_pattern
    # the switched units alone account for what is above the bound against the exact layer
    assert vs_exact["dx"] > 2e-2 > 2 * on_pattern["dx"], (vs_exact, on_pattern)
