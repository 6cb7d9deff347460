"""bfloat16 autocast pinned to the reference: ``tests/golden/reference_autocast_vectors.json``
holds outputs and every gradient of the reference's ``ReferenceDeconv`` (three stage
geometries) and of the small network built on it, run under ``torch.autocast("cpu",
dtype=torch.bfloat16)`` by ``tests/golden/make_reference_autocast_vectors.py``, next to the
float64 run of the same case.  The layer cases carry a stored bias shift that keeps every
source pre-activation 0.05 clear of zero in float64 (a unit within bfloat16 rounding of zero
is on or off by rounding luck in any implementation).

* the package's general route under CPU autocast follows the reference's intermediate
  roundings: its numbers are held to the stored autocast numbers (no GPU needed);
* on a GPU, the HIP route under bfloat16 autocast is held to north_star's 2e-2 of the stored
  autocast numbers, un-gated, in the output and in every gradient;
* the small network is held to 2e-2 of the stored autocast OUTPUT.  Its gradients cannot be
  held to the stored autocast gradients: under bfloat16 the reference's own network is in a
  chaotic regime there (InstanceNorm over 64 voxels at the deepest level, rectifiers switched
  by rounding): its autocast gradients sit 0.1 (median over the parameter tensors: 0.07) and
  up to 0.26 from its float64 gradients at the stored entries.  They are held to the
  reference's own criterion for low precision instead (test_deconv_equivalence.py:332-379):
  no further from the float64 numbers than the reference's autocast run is -- in the median
  over all tensors (x1.5) and per tensor (x3, floor 2e-2; measured: worst ratio 1.9, median
  of the HIP network 0.069 against 0.072).
"""

import json
import os

import pytest
import torch
from torch import nn

import deconver_amd as dc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_autocast_vectors.json")) as fh:
    GOLDEN = json.load(fh)
NPROBE = 96
LAYER_CASES = sorted(GOLDEN["layer_cases"])


def _probe_idx(n):
    k = min(n, NPROBE)
    return [(i * (n - 1)) // max(k - 1, 1) for i in range(k)]


def _exact_match(t, ref):
    """For tensors rebuilt from seeds (inputs): stored entries and sum of squares reproduce."""
    v = t.detach().double().cpu().reshape(-1)
    return (list(t.shape) == ref["shape"]
            and (v[_probe_idx(v.numel())] - torch.tensor(ref["probe"], dtype=torch.float64)).abs().max() < 1e-12
            and abs(float((v * v).sum()) - ref["sumsq"]) <= 1e-9 * max(ref["sumsq"], 1e-300))


def _dev(t, ref, scale_ref=None):
    """Largest deviation of `t` from the stored tensor over its stored entries and its energy,
    relative to the largest magnitude of `scale_ref` (default: the stored tensor)."""
    assert list(t.shape) == ref["shape"]
    v = t.detach().double().cpu().reshape(-1)
    scale = max((scale_ref or ref)["absmax"], 1e-30)
    probes = (v[_probe_idx(v.numel())] - torch.tensor(ref["probe"], dtype=torch.float64)).abs().max().item()
    # root of the energy: a bias or a scale error on all entries shows here
    rms = abs(float((v * v).sum()) ** 0.5 - ref["sumsq"] ** 0.5) / max(v.numel(), 1) ** 0.5
    return max(probes, rms) / scale


def _stored_dev(a, b):
    """The same measure between two stored tensors (autocast run vs float64 run)."""
    pa, pb = torch.tensor(a["probe"], dtype=torch.float64), torch.tensor(b["probe"], dtype=torch.float64)
    return float((pa - pb).abs().max()) / max(b["absmax"], 1e-30)


def _layer(name, seed=0):
    case = GOLDEN["layer_cases"][name]
    kwargs = dict(case["kwargs"], kernel_size=tuple(case["kwargs"]["kernel_size"]))
    torch.manual_seed(seed)
    layer = dc.Deconv(**kwargs)
    with torch.no_grad():
        layer.init.linear.linear.bias.add_(case["bias_shift"])
    torch.manual_seed(seed + 1)
    x0 = torch.rand(2, kwargs["channels"], *case["spatial"])
    torch.manual_seed(seed + 2)
    g0 = torch.randn(2, kwargs["channels"] * 4, *case["spatial"])
    assert _exact_match(x0, case["x"]) and _exact_match(g0, case["g"])
    return case, layer, x0, g0


def _network():
    spec = dict(GOLDEN["network_spec"])
    cfg = {k: (tuple(v) if isinstance(v, list) else v) for k, v in spec.items()}
    kwargs = dict(cfg, norm=getattr(nn, cfg["norm"]), act=getattr(nn, cfg["act"]))
    torch.manual_seed(0)
    net = dc.Deconver(**kwargs).eval()
    torch.manual_seed(1)
    x0 = torch.rand(2, 4, 16, 16, 16)
    g0 = torch.randn(2, 3, 16, 16, 16)
    assert _exact_match(x0, GOLDEN["network"]["x"]) and _exact_match(g0, GOLDEN["network"]["g"])
    return net, x0, g0


def _run(module, x0, g0, device):
    module = module.to(device)
    x = x0.to(device).requires_grad_(True)
    with torch.autocast(device, dtype=torch.bfloat16):
        y = module(x)
    y.backward(g0.to(device).to(y.dtype))
    got = {"y": y, "grad_x": x.grad}
    for n, p in module.named_parameters():
        got["grad_" + n] = p.grad
    return got


@pytest.mark.parametrize("name", LAYER_CASES)
def test_reference_autocast_itself_is_within_the_bf16_bound_of_float64(name):
    """What the fixture says about the reference: on these screened cases its autocast run is
    within 1e-2 of its float64 run in every tensor (so 2e-2 around it is a meaningful band)."""
    case = GOLDEN["layer_cases"][name]
    for key, ref in case["float64"].items():
        if isinstance(ref, dict):
            assert _stored_dev(case["autocast"][key], ref) < 1e-2, key


@pytest.mark.parametrize("name", LAYER_CASES)
def test_general_route_under_cpu_autocast_follows_the_reference(name):
    """The package's general route runs the reference's sequence of operations, so under the
    same CPU autocast it takes the same intermediate roundings: stored autocast numbers
    reproduced to 2e-3 (a tenth of the bf16 bound; summation order inside the library
    convolutions is the only freedom left)."""
    case, layer, x0, g0 = _layer(name)
    got = _run(layer, x0, g0, "cpu")
    assert str(got["y"].dtype) == case["autocast"]["y_dtype"]
    for key, ref in case["autocast"].items():
        if isinstance(ref, dict):
            assert _dev(got[key], ref) < 2e-3, (key, _dev(got[key], ref))


@pytest.mark.gpu
@pytest.mark.parametrize("name", LAYER_CASES)
def test_hip_route_under_autocast_is_within_2e_2_of_the_reference_under_autocast(name):
    case, layer, x0, g0 = _layer(name)
    layer = layer.cuda()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert layer.fast_path_applicable(x0.cuda()), "expected the HIP route"
    got = _run(layer, x0, g0, "cuda")
    assert got["y"].dtype == torch.bfloat16
    devs = {key: _dev(got[key], ref) for key, ref in case["autocast"].items() if isinstance(ref, dict)}
    bad = {k: v for k, v in devs.items() if not v < 2e-2}
    assert not bad, (bad, devs)


@pytest.mark.gpu
def test_hip_network_under_autocast_against_the_reference_network_under_autocast():
    net, x0, g0 = _network()
    stored = GOLDEN["network"]
    got = _run(net, x0, g0, "cuda")
    assert _dev(got["y"], stored["autocast"]["y"]) < 2e-2
    worse, e_hips, e_refs = {}, [], []
    for key, ref64 in stored["float64"].items():
        if not isinstance(ref64, dict) or key == "y":
            continue
        e_ref = _stored_dev(stored["autocast"][key], ref64)
        e_hip = _dev(got[key], ref64)
        e_hips.append(e_hip)
        e_refs.append(e_ref)
        if not e_hip <= max(3.0 * e_ref, 2e-2):
            worse[key] = (e_hip, e_ref)
    assert not worse, worse
    med = lambda v: sorted(v)[len(v) // 2]
    assert med(e_hips) <= 1.5 * med(e_refs), (med(e_hips), med(e_refs))
