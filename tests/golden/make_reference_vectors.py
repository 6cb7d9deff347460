#!/usr/bin/env python3
"""Writes ``reference_vectors.json``: outputs and gradients of the reference's ORIGINAL layer
(``ReferenceDeconv``, its own ground truth) and of a small network built on it, in float64
on the CPU, for the case list of the reference's equivalence tests
(``tests/test_deconv_equivalence.py:29-35,112-140,142-169,311-379``).

Protocol per layer case (the reference's, ``test_deconv_equivalence.py:38-48,65-110``):
``torch.manual_seed(seed)`` builds the module, the projection bias is shifted by ``bias``,
``torch.manual_seed(seed + 1)`` draws ``x = rand(batch, C, *spatial)``,
``torch.manual_seed(seed + 2)`` draws ``g = randn_like(y)``; module and tensors are then
moved to float64 and ``y = module(x); y.backward(g)``.  Network case (``:311-379``): seed 0
builds ``Deconver(**NETWORK)`` with the original layer swapped in, ``.eval()``; seed 1
draws ``x = rand(2, 4, 16, 16, 16)`` and ``g = randn(2, 3, 16, 16, 16)``.

Only data travels: for every tensor its shape, three global checksums (sum, sum of squares,
and the dot product with a fixed cosine probe) and ``NPROBE`` evenly strided entries.
``tests/test_golden_vectors.py`` rebuilds the same weights and inputs from the seeds (the
package's constructors consume the generator as the reference's do, which
``tests/test_golden_state.py`` checks) and compares the oracle and the HIP layer with them.

    python tests/golden/make_reference_vectors.py        # needs /root/reference, CPU only
"""

import json
import math
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = os.environ.get("DECONVER_REFERENCE", "/root/reference")
NPROBE = 96

BRATS_STAGES = [(32, (12, 14, 13)), (64, (10, 9, 11)), (128, (8, 8, 8)), (256, (6, 5, 4)),
                (512, (3, 4, 3))]

LAYER_CASES = {}
for _c, _sp in BRATS_STAGES:
    for _bias in (1.0, 0.0):
        LAYER_CASES[f"stage_c{_c}_bias{_bias:g}"] = dict(
            kwargs=dict(channels=_c, ratio=4, groups=-1, kernel_size=(3, 3, 3), num_iters=1),
            batch=2, spatial=_sp, bias=_bias)
for _name, _kw, _sp in [
    ("geom_g3_3d", dict(channels=12, ratio=2, groups=3, kernel_size=(3, 3, 3)), (7, 6, 5)),
    ("geom_g1_3d", dict(channels=8, ratio=1, groups=1, kernel_size=(3, 3, 3)), (6, 6, 6)),
    ("geom_dw_2d", dict(channels=16, ratio=4, groups=-1, kernel_size=(3, 3)), (17, 15)),
    ("geom_aniso", dict(channels=6, ratio=2, groups=2, kernel_size=(3, 5, 3)), (6, 7, 5)),
    ("geom_1d", dict(channels=8, ratio=2, groups=-1, kernel_size=(5,)), (11,)),
    ("geom_g5_2d", dict(channels=10, ratio=3, groups=5, kernel_size=(3, 3)), (9, 8)),
    ("geom_dw_2d_5x5", dict(channels=32, ratio=4, groups=-1, kernel_size=(5, 5)), (24, 40)),
]:
    LAYER_CASES[_name] = dict(kwargs=dict(num_iters=1, **_kw), batch=2, spatial=_sp, bias=1.0)
for _b in (1, 3):
    LAYER_CASES[f"batch{_b}"] = dict(
        kwargs=dict(channels=16, ratio=4, groups=-1, kernel_size=(3, 3, 3), num_iters=1),
        batch=_b, spatial=(9, 8, 7), bias=1.0)
for _it, _git in [(3, 1), (5, 1), (2, 2), (3, 3)]:
    LAYER_CASES[f"iters{_it}_grad{_git}"] = dict(
        kwargs=dict(channels=8, ratio=2, groups=-1, kernel_size=(3, 3, 3), num_iters=_it,
                    num_grad_iters=_git),
        batch=2, spatial=(6, 6, 6), bias=1.0)

NETWORK = dict(in_channels=4, out_channels=3, spatial_dims=3, encoder_depth=(1, 1, 1),
               encoder_width=(8, 16, 32), strides=(1, 2, 2), decoder_depth=(1, 1),
               norm="InstanceNorm3d", act="ReLU", groups=-1, ratio=4, kernel_size=(3, 3, 3),
               num_iters=1, mlp_ratio=4)


def probe_indices(n):
    k = min(n, NPROBE)
    return [(i * (n - 1)) // max(k - 1, 1) for i in range(k)]


def describe(t):
    """Shape, checksums and strided entries of a tensor (float64)."""
    if t is None:
        return None
    v = t.detach().double().reshape(-1)
    n = v.numel()
    w = torch.cos(torch.arange(n, dtype=torch.float64) * 0.7390851332151607 + 0.25)
    idx = probe_indices(n)
    return {"shape": list(t.shape), "sum": float(v.sum()), "sumsq": float((v * v).sum()),
            "cosdot": float((v * w).sum()), "absmax": float(v.abs().max()),
            "probe": [float(v[i]) for i in idx]}


def layer_case(ReferenceDeconv, spec, seed=0):
    kwargs = {k: (tuple(v) if isinstance(v, (list, tuple)) else v) for k, v in spec["kwargs"].items()}
    torch.manual_seed(seed)
    ref = ReferenceDeconv(**kwargs)
    if spec["bias"]:
        with torch.no_grad():
            ref.init.linear.linear.bias.add_(spec["bias"])
    torch.manual_seed(seed + 1)
    x0 = torch.rand(spec["batch"], kwargs["channels"], *spec["spatial"])
    sc_total = ref.init.linear.linear.weight.shape[0]
    torch.manual_seed(seed + 2)
    g0 = torch.randn(spec["batch"], sc_total, *spec["spatial"])
    ref = ref.double()
    x = x0.double().requires_grad_(True)
    y = ref(x)
    assert y.shape == g0.shape
    if y.requires_grad:
        y.backward(g0.double())
    out = {"y": describe(y), "x": describe(x0), "g": describe(g0), "grad_x": describe(x.grad)}
    for name, p in ref.named_parameters():
        out["grad_" + name] = describe(p.grad)
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
    net = net.double()
    x = x0.double().requires_grad_(True)
    y = net(x)
    y.backward(g0.double())
    out = {"y": describe(y), "x": describe(x0), "g": describe(g0), "grad_x": describe(x.grad),
           "params": {}}
    for name, p in net.named_parameters():
        out["params"][name] = {"value": describe(p), "grad": describe(p.grad)}
    return out


def main():
    sys.path.insert(0, REFERENCE)
    import deconver as ref_pkg                         # the reference package (CPU only here)
    import deconver.deconver as deconver_module
    from deconver.deconvolution.reference import ReferenceDeconv

    torch.set_num_threads(max(1, (os.cpu_count() or 2) // 2))
    out = {"torch": torch.__version__, "nprobe": NPROBE, "layer_cases": {}, "specs": {}}
    for name, spec in LAYER_CASES.items():
        out["specs"][name] = dict(spec, kwargs={k: (list(v) if isinstance(v, tuple) else v)
                                                for k, v in spec["kwargs"].items()},
                                  spatial=list(spec["spatial"]))
        out["layer_cases"][name] = layer_case(ReferenceDeconv, spec)
        print("layer", name, "y sum %.6g" % out["layer_cases"][name]["y"]["sum"], flush=True)
    out["network_spec"] = NETWORK
    out["network"] = network_case(ref_pkg, deconver_module, ReferenceDeconv)
    print("network: %d parameters" % len(out["network"]["params"]))
    path = os.path.join(HERE, "reference_vectors.json")
    with open(path, "w") as fh:
        json.dump(out, fh, indent=0, sort_keys=True)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
