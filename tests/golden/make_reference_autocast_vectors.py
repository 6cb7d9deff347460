#!/usr/bin/env python3
"""Writes ``reference_autocast_vectors.json``: the reference's ORIGINAL layer
(``ReferenceDeconv``) and a small network built on it under **bfloat16 autocast** on the CPU
(``torch.autocast("cpu", dtype=torch.bfloat16)``) -- the precision regime in which the
reference's own fused route steps aside (``deconver/deconvolution/deconv.py:139-147``) and its
general path runs with whatever intermediate roundings autocast gives it.

Cases: three stage geometries of ``tests/test_deconv_equivalence.py:29-35`` (32, 64, 128
channels, 3x3x3, ratio 4) with the seeding protocol of ``make_reference_vectors.py``, and the
small network of ``:311-379``.  A source unit whose pre-activation lies within bfloat16
rounding of zero is on or off by rounding luck in ANY bfloat16 implementation, so every layer
case is screened in float64: the projection bias is raised by a stored amount until the
smallest pre-activation ``W x + b`` is ``MARGIN``; the test applies the same stored shift.

Stored per tensor: shape, sum of squares, largest magnitude and ``NPROBE`` strided entries
(``describe`` of ``make_reference_vectors.py``), for the autocast run AND for the float64 run
of the same case, so that the test can state how far bfloat16 autocast itself sits from
float64.  Only data travels.

    python tests/golden/make_reference_autocast_vectors.py      # needs /root/reference, CPU only
"""

import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from make_reference_vectors import NETWORK, REFERENCE, describe  # noqa: E402

MARGIN = 0.05
STAGES = {"stage_c32": (32, (12, 14, 13)), "stage_c64": (64, (10, 9, 11)), "stage_c128": (128, (8, 8, 8))}


def _run(module, x0, g0, autocast):
    module.zero_grad(set_to_none=True)
    x = x0.clone().requires_grad_(True)
    if autocast:
        with torch.autocast("cpu", dtype=torch.bfloat16):
            y = module(x)
        y.backward(g0.to(y.dtype))
    else:
        y = module(x)
        y.backward(g0)
    out = {"y": describe(y), "y_dtype": str(y.dtype), "grad_x": describe(x.grad)}
    for name, p in module.named_parameters():
        out["grad_" + name] = describe(p.grad)
    return out


def layer_case(ReferenceDeconv, channels, spatial, seed=0):
    kwargs = dict(channels=channels, ratio=4, groups=-1, kernel_size=(3, 3, 3), num_iters=1)
    torch.manual_seed(seed)
    ref = ReferenceDeconv(**kwargs)
    torch.manual_seed(seed + 1)
    x0 = torch.rand(2, channels, *spatial)
    torch.manual_seed(seed + 2)
    g0 = torch.randn(2, channels * 4, *spatial)
    proj = ref.init.linear.linear
    with torch.no_grad():
        z = torch.nn.functional.conv1d(x0.double().flatten(2), proj.weight.double(), proj.bias.double())
        shift = float(MARGIN - z.min())
        proj.bias.add_(shift)
    out = {"kwargs": dict(kwargs, kernel_size=list(kwargs["kernel_size"])), "spatial": list(spatial),
           "bias_shift": shift, "x": describe(x0), "g": describe(g0)}
    out["autocast"] = _run(ref, x0, g0, True)
    ref64 = ref.double()
    out["float64"] = _run(ref64, x0.double(), g0.double(), False)
    return out


def network_case(ref_pkg, deconver_module, ReferenceDeconv):
    from torch import nn
    kwargs = dict(NETWORK, norm=getattr(nn, NETWORK["norm"]), act=getattr(nn, NETWORK["act"]))
    original = deconver_module.Deconv
    deconver_module.Deconv = ReferenceDeconv
    try:
        torch.manual_seed(0)
        net = ref_pkg.Deconver(**kwargs).eval()
    finally:
        deconver_module.Deconv = original
    torch.manual_seed(1)
    x0 = torch.rand(2, 4, 16, 16, 16)
    g0 = torch.randn(2, 3, 16, 16, 16)
    out = {"x": describe(x0), "g": describe(g0)}
    out["autocast"] = _run(net, x0, g0, True)
    out["float64"] = _run(net.double(), x0.double(), g0.double(), False)
    return out


def _rel(a, b):
    pa, pb = torch.tensor(a["probe"]), torch.tensor(b["probe"])
    return float((pa - pb).abs().max() / max(b["absmax"], 1e-30))


def main():
    sys.path.insert(0, REFERENCE)
    import deconver as ref_pkg                         # the reference package (CPU only here)
    import deconver.deconver as deconver_module
    from deconver.deconvolution.reference import ReferenceDeconv

    torch.set_num_threads(max(1, (os.cpu_count() or 2) // 2))
    out = {"torch": torch.__version__, "margin": MARGIN, "layer_cases": {}}
    for name, (c, sp) in STAGES.items():
        case = out["layer_cases"][name] = layer_case(ReferenceDeconv, c, sp)
        print(name, "shift %.4f" % case["bias_shift"], "y dtype", case["autocast"]["y_dtype"],
              {k: "%.1e" % _rel(case["autocast"][k], case["float64"][k])
               for k in case["float64"] if isinstance(case["float64"][k], dict)}, flush=True)
    out["network_spec"] = NETWORK
    net = out["network"] = network_case(ref_pkg, deconver_module, ReferenceDeconv)
    worst = max((_rel(net["autocast"][k], net["float64"][k]), k) for k in net["float64"]
                if isinstance(net["float64"][k], dict))
    print("network: y %.1e, worst gradient %.1e (%s)" % (_rel(net["autocast"]["y"], net["float64"]["y"]),
                                                         worst[0], worst[1]))
    path = os.path.join(HERE, "reference_autocast_vectors.json")
    with open(path, "w") as fh:
        json.dump(out, fh, indent=0, sort_keys=True)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
