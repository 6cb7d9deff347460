#!/usr/bin/env python3
"""Writes ``reference_state.json``: parameter names, shapes and seeded-initialisation
statistics of the reference's own modules.

These are the facts about the reference that no mathematical check can pin (what its
state-dict keys are called, and in which order its constructors consume the random
generator), so they are taken from the reference itself: this script imports the package
at ``/root/reference`` on the CPU, builds a layer, a mixer and three networks under
``torch.manual_seed(0)``, and records for every parameter its shape, sum and sum of squares
(float64).  Only this data travels; ``tests/test_golden_state.py`` compares the package's
modules with it.

    python tests/golden/make_reference_state.py        # needs /root/reference
"""

import json
import os
import sys

import torch
from torch import nn

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = os.environ.get("DECONVER_REFERENCE", "/root/reference")

CASES = {
    "layer_3d": ("Deconv", dict(channels=6, kernel_size=(3, 3, 3), ratio=2, groups=-1)),
    "layer_grouped_2d": ("Deconv", dict(channels=12, kernel_size=(5, 5), ratio=2, groups=3)),
    "mixer_3d": ("DeconvMixer", dict(in_channels=5, out_channels=8, kernel_size=(3, 3, 3),
                                     ratio=4, groups=-1)),
    "tiny_2d": ("Deconver", dict(in_channels=3, out_channels=2, spatial_dims=2,
                                 encoder_depth=(1, 2, 1), encoder_width=(8, 16, 24),
                                 strides=(1, 2, 2), decoder_depth=(1, 1), norm="InstanceNorm2d",
                                 kernel_size=(5, 5), groups=-1, ratio=4)),
    "tiny_3d_layernorm": ("Deconver", dict(in_channels=2, out_channels=1, spatial_dims=3,
                                           encoder_depth=(1, 1), encoder_width=(8, 16),
                                           strides=(1, 2), decoder_depth=(2,),
                                           kernel_size=(3, 3, 3), groups=-1, ratio=2)),
    "tiny_3d_deep_supervision": ("Deconver", dict(in_channels=1, out_channels=2, spatial_dims=3,
                                                  encoder_depth=(1, 1, 1), encoder_width=(4, 8, 12),
                                                  strides=(1, 2, 2), decoder_depth=(1, 1),
                                                  norm="InstanceNorm3d", kernel_size=(3, 3, 3),
                                                  groups=-1, ratio=4, num_deep_supr=2)),
}


def resolve(kwargs):
    """Module classes are named by string in CASES so that the table is plain data."""
    out = dict(kwargs)
    if isinstance(out.get("norm"), str):
        out["norm"] = getattr(nn, out["norm"])
    return out


def describe(module):
    rows = {}
    for name, value in module.state_dict().items():
        v = value.detach().double()
        rows[name] = {"shape": list(value.shape), "sum": float(v.sum()),
                      "sumsq": float((v * v).sum())}
    return rows


def main():
    sys.path.insert(0, REFERENCE)
    import deconver as ref   # the reference package (CPU only here)
    from deconver.deconver import DeconvMixer as RefMixer

    classes = {"Deconv": ref.Deconv, "DeconvMixer": RefMixer, "Deconver": ref.Deconver}
    out = {"torch": torch.__version__, "seed": 0, "cases": {}}
    for case, (cls, kwargs) in CASES.items():
        torch.manual_seed(0)
        module = classes[cls](**resolve(kwargs))
        out["cases"][case] = {"class": cls, "kwargs": kwargs, "state": describe(module)}
    with open(os.path.join(HERE, "reference_state.json"), "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
    print("wrote", os.path.join(HERE, "reference_state.json"),
          {k: len(v["state"]) for k, v in out["cases"].items()})


if __name__ == "__main__":
    main()
