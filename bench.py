#!/usr/bin/env python3
"""Benchmark of the NDC update hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--no-cpu]
    python bench.py --workload sweep                                      (config 5, forward only)
    python bench.py --workload accuracy                                   (float32 error table)
    python bench.py --workload grid                                       (ratio x groups x kernel grid)
    python bench.py --workload valu                                       (instruction-issue ceiling probe)
    python bench.py --workload train3d|model2d [--ndc hip|pytorch|both]   (model level, below)
    python bench.py --workload block      (norm and projection-tail kernels of a Deconver block)
    python bench.py --workload mixer [--dtype bf16|fp32]                  (one DeconvMixer, fwd+bwd)
    python bench.py --workload layout                                     (channels-last copies around the update)
    python bench.py --workload graphed    (small batches: the training step eager and replayed from a HIP graph)

One step = one forward + one backward (input-, source-, filter- and bias-gradient) of the
update node on config 3 of the baseline: batch 2, 128 depthwise channels, 64^3 voxels,
3x3x3 filter, ratio 4, bfloat16 storage with float32 accumulation; inputs resident in HBM.
Prints ONE JSON line: whole-step throughput in Gvoxel/s, a ``vector_ceiling`` object (bf16:
time the kernels' v_dot2c_f32_bf16 alone would take at the measured issue rate, over the
measured time), a ``matrix_instruction_variant`` object (the same step with the library's other
kernel family switched on, `ndc_matrix_kernels(1)`: outside the specified path, not `value`),
plus a ``roofline`` object for the
slowest kernel (device time from events on the launch stream, algorithmic bytes as stated
below) and a ``cpu_baseline`` object (the oracle timed on the host cores on a bounded
sample of the same workload).

Algorithmic bytes (each compulsory tensor once, re-reads and temporaries zero), with
U = B*C*D*H*W channel-voxels and e bytes per element:
    forward      9 U e   (read x, z; write out)
    backward    14 U e   (read gout, re-read x, z; write gx, gz), attributed to its two
                          passes as pass 1 = 10 U e (x, z, gout in; gx out) and
                          pass 2 = 4 U e (gz out; its inputs are re-reads)
    whole step  23 U e

Model-level workloads (not roofline-graded; same one-JSON-line output, `roofline` and
`cpu_baseline` null):
    train3d   config 4: Deconver 3-D (widths 64-512, 3x3x3, ratio 4, InstanceNorm3d), batch 2
              of 128^3 two-channel ellipsoid phantoms, bf16 autocast, Dice+BCE, AdamW; one
              step = forward + backward + optimiser update; metric = train steps/s
    model2d   config 2: Deconver 2-D (widths 32-512, 5x5, ratio 4, InstanceNorm2d), batch 8 of
              256^2 RGB-like images, float32, Dice+BCE; one step = forward + backward
`--ndc hip` runs the NDC layers on the HIP kernels, `pytorch` on the layer's general PyTorch
route (same GPU, same weights), `both` reports the two and their ratio.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOAD = dict(batch=2, channels=128, spatial=(64, 64, 64), kernel=(3, 3, 3), ratio=4)


def make_inputs(torch, dtype, device, batch, channels, spatial, kernel, ratio, seed=0):
    """Config-3 style tensors: h = softplus(0.1 N(0,1)) > 0, x = |N(0,1)|, z = W x with the
    projection's default initialisation (bias withheld: the kernels add it), g = N(0,1)."""
    import deconver_amd as dc

    torch.manual_seed(seed)
    layer = dc.Deconv(channels=channels, kernel_size=kernel, ratio=ratio, groups=-1)
    sc = layer.source_channels
    h = torch.nn.functional.softplus(0.1 * torch.randn(channels, sc, *kernel))
    x = torch.randn(batch, channels, *spatial).abs()
    proj = layer.init.linear.linear
    x = x.to(device=device, dtype=dtype)
    w = proj.weight.detach().to(device=device, dtype=dtype)
    # (a GEMM per sample: conv1d would send MIOpen searching through its convolution algorithms,
    # seconds of set-up for tensors this size)
    z = torch.stack([w.squeeze(-1) @ xb for xb in x.flatten(2)]).view(batch, channels * sc, *spatial)
    torch.manual_seed(seed + 2)
    g = torch.randn(batch, channels * sc, *spatial).to(device=device, dtype=dtype)
    bias = proj.bias.detach().float().to(device)
    return x.contiguous(), z.contiguous(), h.float().to(device).contiguous(), bias, g.contiguous(), sc


def cpu_baseline(torch):
    """The oracle (literal restatement of the reference's update, autograd backward) on the
    host cores, float32, on the whole config-3 workload (batch 2, 128 channels, 64^3): one
    untimed and three timed steps, about 20 s of CPU work on 16 threads."""
    from oracle import ndc_oracle as O

    w = WORKLOAD
    b, c, sp, ks = w["batch"], w["channels"], w["spatial"], w["kernel"]
    sc = w["ratio"]
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(b, c, *sp, generator=gen).abs()
    s = torch.randn(b, c * sc, *sp, generator=gen).abs()
    h = torch.nn.functional.softplus(0.1 * torch.randn(c, sc, *ks, generator=gen))
    g = torch.randn(b, c * sc, *sp, generator=gen)
    layer = O.OracleNDC(c, ks, ratio=sc)

    def step():
        xs = layer.split(x.clone().requires_grad_(True))
        ss = layer.split(s.clone().requires_grad_(True))
        hs = layer.split(h.clone().requires_grad_(True).expand(b, *h.shape))
        out = layer.merge(layer.update_s(xs, ss, hs))
        out.backward(g)

    step()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    vox = b * sp[0] * sp[1] * sp[2]
    return {
        "value": vox / t / 1e9,
        "unit": "Gvoxel/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle update fwd+bwd (autograd), float32, the whole workload (B={b}, {c} "
                  f"depthwise channels, {sp[0]}^3), median of 3 steps ({t:.2f} s each) after one "
                  f"untimed step",
        "channel_voxels_per_s": vox * c / t,
    }


SWEEP_SHAPES = [   # config 5: (channels, extent, batch), bottleneck to full resolution
    (512, 16, 4), (256, 32, 2), (64, 128, 1), (32, 192, 1),
]


def sweep_rows(torch, lib, ops, dev, warmup, steps):
    """Config 5: forward-only (inference: no t1, nothing kept for backward) NDC update,
    3x3x3, ratio 4, bf16, half-normal inputs; per shape the time of one call, Gvoxel/s and the
    HBM-roofline fraction on the 9 U e algorithmic bytes."""
    rows = []
    for C, n, B in SWEEP_SHAPES:
        x, z, h, bias, _, sc = make_inputs(torch, torch.bfloat16, dev, B, C, (n, n, n), (3, 3, 3), 4)
        kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, need_t1=False)
        for _ in range(warmup):
            ops.update_forward(lib, x, z, h, bias, **kw)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            ops.update_forward(lib, x, z, h, bias, **kw)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        vox, U = B * n ** 3, B * C * n ** 3
        rows.append({"channels": C, "extent": n, "batch": B, "ms": ms,
                     "Gvoxel_per_s": vox / (ms * 1e-3) / 1e9,
                     "channel_voxels_per_s": U / (ms * 1e-3),
                     "algorithmic_bytes": 9 * U * 2,
                     "hbm_frac": 9 * U * 2 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
        del x, z
    return rows


LAYERS_2D = [   # the 2-D 5x5 form: (name, channels, extent, batch)
    ("config 1: B 1, 32 ch, 64^2", 32, 64, 1),
    ("config 2 stage 0: B 8, 32 ch, 256^2", 32, 256, 8),
]


def layers_2d_rows(torch, lib, ops, dev, warmup, steps):
    """The 2-D 5x5 form of the update node (depthwise, ratio 4, float32 storage: the reference's
    own precision): forward + backward with the forward's ratios kept, per shape the time of
    one step, of its kernels, Gvoxel/s and the HBM-roofline fraction on 23 U e (forward alone
    on 9 U e)."""
    rows = []
    for name, C, n, B in LAYERS_2D:
        x, z, h, bias, g, sc = make_inputs(torch, torch.float32, dev, B, C, (n, n), (5, 5), 4)
        kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)
        keep = lib.backward_uses_saved(ops.make_geom_for(x, h, C, 1, sc, 1e-16, True))

        def step(pt=None):
            res = ops.update_forward(lib, x, z, h, bias, save_ratio=keep, **kw)
            return ops.update_backward(lib, x, z, res[1], h, bias, g, pass_times=pt,
                                       saved=res[2] if keep else None, **kw)

        for _ in range(warmup):
            step()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        f0.record()
        for _ in range(steps):
            ops.update_forward(lib, x, z, h, bias, save_ratio=keep, **kw)
        f1.record()
        torch.cuda.synchronize()
        fwd_ms = f0.elapsed_time(f1) / steps
        pt = []
        step(pt)
        vox, U = B * n * n, B * C * n * n
        rows.append({"layer": name, "channels": C, "extent": n, "batch": B, "dtype": "f32",
                     "ms": ms, "forward_ms": fwd_ms,
                     "backward_kernel_ms": {"pass1": pt[0], "pass2": pt[1], "reduce": pt[2]},
                     "Gvoxel_per_s": vox / (ms * 1e-3) / 1e9,
                     "channel_voxels_per_s": U / (ms * 1e-3),
                     "algorithmic_bytes": 23 * U * 4,
                     "hbm_frac": 23 * U * 4 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "forward_hbm_frac": 9 * U * 4 / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
        del x, z, g
    return rows


def sweep_workload(args) -> int:
    """Config 5 alone (see sweep_rows); `value` is the geometric mean over the shapes."""
    import torch

    from deconver_amd import _lib, ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _lib.get_library()
    dev = torch.device("cuda:0")
    rows = sweep_rows(torch, lib, ops, dev, args.warmup, args.steps)
    gmean = math.exp(sum(math.log(r["Gvoxel_per_s"]) for r in rows) / len(rows))
    print(json.dumps({
        "metric": "NDC mixer forward-only Gvoxel/s (geometric mean over the sweep)",
        "value": gmean, "unit": "Gvoxel/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sum(r["ms"] for r in rows),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "config 5: forward-only NDC update shape sweep, 3x3x3, ratio 4, "
                               "bf16 storage / float32 accumulation, inference form"},
        "shapes": rows, "layers_2d": layers_2d_rows(torch, lib, ops, dev, args.warmup, args.steps),
        "roofline": None, "cpu_baseline": None}))
    return 0


ACCURACY_CASES = [   # the layer geometries of the reference's accuracy report (benchmarks/accuracy_report.py:36-50)
    ("brats23 stage C=32", dict(channels=32, ratio=4, groups=-1, kernel_size=(3, 3, 3))),
    ("brats23 stage C=64", dict(channels=64, ratio=4, groups=-1, kernel_size=(3, 3, 3))),
    ("brats23 stage C=128", dict(channels=128, ratio=4, groups=-1, kernel_size=(3, 3, 3))),
    ("brats23 stage C=256", dict(channels=256, ratio=4, groups=-1, kernel_size=(3, 3, 3))),
    ("brats23 stage C=512", dict(channels=512, ratio=4, groups=-1, kernel_size=(3, 3, 3))),
    ("fives/glas 2-D k=5", dict(channels=32, ratio=4, groups=-1, kernel_size=(5, 5))),
    ("grouped C/G=4", dict(channels=12, ratio=2, groups=3, kernel_size=(3, 3, 3))),
    ("dense groups=1", dict(channels=8, ratio=1, groups=1, kernel_size=(3, 3, 3))),
    ("grouped C/G=4, small filter", dict(channels=8, ratio=1, groups=2, kernel_size=(3, 3, 3))),
]


def _rel_err(a, ref) -> float:
    """max|a - ref| / max|ref| in float64."""
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    return float((a - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def _layer_outputs(layer, x, g):
    """Forward + backward of a Deconv layer: [y, dx, dW, db, dh0]."""
    y = layer(x)
    y.backward(g)
    p = layer.init
    return [y.detach(), x.grad, p.linear.linear.weight.grad, p.linear.linear.bias.grad, p.h0.grad]


def accuracy_workload(args) -> int:
    """Float32 accuracy of the whole layer (projection + update, all gradients) on the HIP
    route and on the layer's PyTorch route, both against the layer's PyTorch route evaluated
    in float64 on the CPU from the same parameters; `max|d| / max|ref|` per case, worst tensor."""
    import torch

    import deconver_amd as dc

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    rows = []
    for name, kw in ACCURACY_CASES:
        nd = len(kw["kernel_size"])
        spatial = (12,) * nd if nd == 3 else (48,) * nd
        torch.manual_seed(0)
        base = dc.Deconv(**kw)
        with torch.no_grad():
            base.init.linear.linear.bias.add_(1.0)
        state = base.state_dict()
        x0 = torch.rand(2, kw["channels"], *spatial)
        g0 = torch.randn(2, base.groups * base.source_channels, *spatial)
        truth = dc.Deconv(**kw, dilation=1)   # a convolution keyword selects the PyTorch route
        truth.load_state_dict(state)
        ref = _layer_outputs(truth.double(), x0.double().requires_grad_(True), g0.double())
        errs = {}
        for route, extra in (("hip", {}), ("pytorch", {"dilation": 1})):
            layer = dc.Deconv(**kw, **extra)
            layer.load_state_dict(state)
            layer = layer.to(dev)
            x = x0.to(dev).requires_grad_(True)
            on_hip = layer.fast_path_applicable(x)
            assert on_hip == (route == "hip")
            e = [_rel_err(a, r) for a, r in zip(_layer_outputs(layer, x, g0.to(dev)), ref)]
            errs[route] = {"forward": e[0], "worst_gradient": max(e[1:])}
        rows.append({"case": name, "spatial": list(spatial), **errs})
    worst = max(r["hip"]["worst_gradient"] for r in rows)
    print(json.dumps({
        "metric": "float32 layer accuracy vs float64 (worst gradient, max|d|/max|ref|)",
        "value": worst, "unit": "relative error", "n_gpus": 1, "steps": 1, "warmup": 0,
        "ms_per_step": None, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "accuracy report over the reference's layer geometries, batch 2"},
        "cases": rows, "roofline": None, "cpu_baseline": None}))
    return 0


GRID_RATIOS = (1, 2, 4)
GRID_GROUPS = (1, 2, 4, 8, -1)
GRID_KERNELS = ((3, 3, 3), (5, 5, 5))


def grid_workload(args) -> int:
    """Correctness and efficiency of the layer over ratio x groups x kernel size, float32,
    the grid of the reference's configuration sweep (benchmarks/sweep_configs.py:36-38,
    16 channels, 24^3, batch 2): per configuration the route taken, the error of the HIP
    route against the layer's PyTorch route on the same GPU, and PyTorch-route / HIP-route
    ratios of forward, backward and forward+backward time and of peak memory.  `value` is
    the geometric mean of the forward+backward speed-ups; `slower` lists configurations
    where the default route loses more than 3 % in time or memory."""
    import statistics

    import torch

    import deconver_amd as dc

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    C, n, B = 16, 24, 2

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        samples = []
        for _ in range(args.steps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) * 1e3)
        return statistics.median(samples)

    def measure(layer, x, g):
        def reset():
            layer.zero_grad(set_to_none=True)
            x.grad = None

        def fwd():
            with torch.no_grad():
                layer(x)

        def fwd_bwd():
            reset()
            layer(x).backward(g)

        t_f = timed(fwd)
        t_fb = timed(fwd_bwd)
        reset()
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        fwd_bwd()
        torch.cuda.synchronize()
        mem = torch.cuda.max_memory_allocated() / 2 ** 20
        reset()
        return {"fwd_ms": t_f, "bwd_ms": max(t_fb - t_f, 0.0), "fwd_bwd_ms": t_fb, "peak_MiB": mem}

    rows = []
    for ratio in GRID_RATIOS:
        for groups in GRID_GROUPS:
            for kernel in GRID_KERNELS:
                kw = dict(channels=C, ratio=ratio, groups=groups, kernel_size=kernel, num_iters=1)
                torch.manual_seed(0)
                general = dc.Deconv(**kw, dilation=1).to(dev)
                with torch.no_grad():   # keeps the source away from zero (1/eps ratios)
                    general.init.linear.linear.bias.add_(1.0)
                default = dc.Deconv(**kw).to(dev)
                default.load_state_dict(general.state_dict())
                torch.manual_seed(1)
                x0 = torch.rand(B, C, n, n, n, device=dev)
                route = "hip" if default.fast_path_applicable(x0) else "general"
                torch.manual_seed(2)
                g = torch.randn(B, default.groups * default.source_channels, n, n, n, device=dev)
                ref = _layer_outputs(general, x0.clone().requires_grad_(True), g)
                got = _layer_outputs(default, x0.clone().requires_grad_(True), g)
                e = [_rel_err(a, r) for a, r in zip(got, ref)]
                x = x0.clone().requires_grad_(True)
                pg, pd = measure(general, x, g), measure(default, x, g)
                rows.append({"ratio": ratio, "groups": groups, "kernel": list(kernel),
                             "m": default.filter_channels, "sc": default.source_channels,
                             "route": route, "fwd_err": e[0], "grad_err": max(e[1:]),
                             "pytorch_route": pg, "default_route": pd,
                             "speedup": {k: pg[k] / pd[k] if pd[k] > 0 else None
                                         for k in ("fwd_ms", "bwd_ms", "fwd_bwd_ms")},
                             "memory_ratio": pd["peak_MiB"] / pg["peak_MiB"]})
                del general, default, x, x0, g, ref, got
                torch.cuda.empty_cache()
    slower = [f"ratio={r['ratio']} groups={r['groups']} k={tuple(r['kernel'])} [{r['route']}]"
              for r in rows if r["speedup"]["fwd_bwd_ms"] < 0.97 or r["memory_ratio"] > 1.03]
    gmean = math.exp(sum(math.log(r["speedup"]["fwd_bwd_ms"]) for r in rows) / len(rows))
    print(json.dumps({
        "metric": "Deconv layer fwd+bwd speed-up over its PyTorch route (geometric mean over the grid)",
        "value": gmean, "unit": "x", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sum(r["default_route"]["fwd_bwd_ms"] for r in rows),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"configuration grid: ratio x groups x kernel, {C} channels, {n}^3, batch {B}"},
        "worst_fwd_err": max(r["fwd_err"] for r in rows),
        "worst_grad_err": max(r["grad_err"] for r in rows),
        "slower": slower, "rows": rows, "roofline": None, "cpu_baseline": None}))
    return 0


# Config 3's bf16 kernels issue v_mfma_f32_4x4x4_16b_bf16 (16 blocks of 4 lanes; one
# instruction covers 64 channel-voxel columns of a K- or A-type tap pair, or 64 positions of a
# filter-gradient tap row): instructions per 64 channel-voxels, and what the same sums took
# as v_dot2c_f32_bf16 per channel-voxel in the kernels they replace.
MFMA_PER_64_CHANNEL_VOXELS = {"forward": 27, "backward_pass1": 36, "backward_pass2": 18}
DOT2_PER_CHANNEL_VOXEL = {"forward": 181, "backward_pass1": 216, "backward_pass2": 126}
CLOCKS_PER_MFMA = 9.11    # per SIMD, two wavefronts resident (as the kernels run): measured by `--workload valu`
CLOCKS_PER_DOT2C = 4.52   # per SIMD, four wavefronts resident: measured by `--workload valu`


def build_valu_probe() -> str:
    """Compile bench_valu_probe.hip (beside this file) for gfx950 into ./bench_valu_probe; no GPU
    needed.  Same device flags as the library (deconver_amd/build.py)."""
    import subprocess

    from deconver_amd import build as ndc_build

    exe = os.path.join(ROOT, "bench_valu_probe")
    flags = [f for f in ndc_build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    subprocess.check_call([os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), *flags, "-o", exe,
                           os.path.join(ROOT, "bench_valu_probe.hip")], stderr=subprocess.DEVNULL)
    return exe


def valu_workload(args) -> int:
    """Instruction-issue probe (bench_valu_probe.hip, built by `python bench.py --workload valu
    --build-probe`): clocks per wavefront instruction per SIMD for the
    multiply-accumulate forms, and from the v_dot2c_f32_bf16 figure the least time the bf16
    kernels' multiply-accumulates alone take on config 3.  `value` is that vector ceiling in
    T multiply-accumulates per second."""
    import subprocess

    if args.build_probe:
        print(build_valu_probe())
        return 0
    exe = os.path.join(ROOT, "bench_valu_probe")
    if not os.path.exists(exe):
        print("bench.py --workload valu: ./bench_valu_probe is not built "
              "(python bench.py --workload valu --build-probe)", file=sys.stderr)
        return 2
    proc = subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=300)
    if proc.returncode != 0:
        print("valu_probe failed", file=sys.stderr)
        return 2
    probe = json.loads(proc.stdout)
    clk = {(r["op"], r["wavefronts_per_simd"]): r["clocks_per_instruction"] for r in probe["rows"]}
    dot2 = clk[("v_dot2c_f32_bf16 (scalar multiplicand)", 4)]
    lanes = probe["compute_units"] * 4 * 64
    hz = probe["clock_GHz"] * 1e9
    ceiling = lanes * 2 / dot2 * hz   # two multiply-accumulates per lane per instruction
    U = 2 * 128 * 64 ** 3
    least_ms = {k: U * n / lanes * dot2 / hz * 1e3 for k, n in DOT2_PER_CHANNEL_VOXEL.items()}
    mfma = clk.get(("v_mfma_f32_4x4x4_16b_bf16", 2))
    least_mfma = None if mfma is None else {
        k: U / 64 * n / (probe["compute_units"] * 4) * mfma / hz * 1e3
        for k, n in MFMA_PER_64_CHANNEL_VOXELS.items()}
    print(json.dumps({
        "metric": "vector multiply-accumulate ceiling (v_dot2c_f32_bf16 issue rate)",
        "value": ceiling / 1e12, "unit": "TMAC/s", "n_gpus": 1, "steps": 1, "warmup": 0,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "instruction-issue probe, 256 threads per workgroup, registers only"},
        "clocks_per_dot2c": dot2,
        "fmac_scalar_operand_TMACs": lanes / clk[("v_fmac_f32 (scalar multiplicand)", 4)] * hz / 1e12,
        "fmac_vector_operands_TMACs": lanes / clk[("v_fmac_f32 (vector operands)", 4)] * hz / 1e12,
        "config3_dot2c_per_channel_voxel": DOT2_PER_CHANNEL_VOXEL,
        "config3_least_ms_for_dot2c_alone": least_ms,
        "clocks_per_mfma_4x4x4_bf16": mfma,
        "mfma_TMACs": None if mfma is None else probe["compute_units"] * 4 * 1024 / mfma * hz / 1e12,
        "config3_mfma_per_64_channel_voxels": MFMA_PER_64_CHANNEL_VOXELS,
        "config3_least_ms_for_mfma_alone": least_mfma,
        "probe": probe, "roofline": None, "cpu_baseline": None}))
    return 0


MODEL_WORKLOADS = {
    "train3d": dict(
        net=dict(in_channels=2, out_channels=1, spatial_dims=3, encoder_depth=(1, 1, 1, 1),
                 encoder_width=(64, 128, 256, 512), strides=(1, 2, 2, 2), decoder_depth=(1, 1, 1),
                 kernel_size=(3, 3, 3), groups=-1, ratio=4),
        batch=2, size=(128, 128, 128), autocast=True, optimizer=True,
        metric="Deconver-3D train steps/s", unit="steps/s",
        text="config 4: Deconver 3-D training step, batch 2 of 128^3 two-channel ellipsoid "
             "phantoms, bf16 autocast, Dice+BCE, AdamW"),
    "model2d": dict(
        net=dict(in_channels=3, out_channels=1, spatial_dims=2, encoder_depth=(1, 1, 1, 1, 1),
                 encoder_width=(32, 64, 128, 256, 512), strides=(1, 2, 2, 2, 2),
                 decoder_depth=(1, 1, 1, 1), kernel_size=(5, 5), groups=-1, ratio=4),
        batch=8, size=(256, 256), autocast=False, optimizer=False,
        metric="Deconver-2D fwd+bwd steps/s", unit="steps/s",
        text="config 2: Deconver 2-D forward + backward, batch 8 of 256^2 RGB-like images, "
             "float32, Dice+BCE on smoothed-noise masks"),
}


def _progress(msg: str) -> None:
    """A line on stderr (stdout carries the one JSON line): long legs report as they go."""
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def run_model_routes(workload: str, routes, warmup: int, steps: int) -> dict:
    """One model-level workload (MODEL_WORKLOADS) on each of `routes` ("hip": the NDC layers on
    the HIP kernels; "pytorch": the same network with the layers on their general PyTorch
    route): ms per step, steps per second, last loss, peak memory."""
    import torch
    from torch import nn

    import deconver_amd as dc
    from deconver_amd import training as T

    w = MODEL_WORKLOADS[workload]
    dev = torch.device("cuda:0")
    nd = len(w["size"])
    norm = nn.InstanceNorm3d if nd == 3 else nn.InstanceNorm2d
    if nd == 3:
        images, targets = T.ellipsoid_phantoms(w["batch"], w["net"]["in_channels"], w["size"],
                                               seed=0, device=dev)
    else:
        images, targets = T.smoothed_noise_masks(w["batch"], w["net"]["in_channels"], w["size"],
                                                 seed=0, device=dev)

    def run(route):
        torch.manual_seed(0)
        # a convolution keyword argument sends the NDC layers down their general PyTorch route
        extra = {"dilation": 1} if route == "pytorch" else {}
        model = dc.Deconver(norm=norm, **w["net"], **extra).to(dev)
        layers = [m for m in model.modules() if isinstance(m, dc.Deconv)]
        on_hip = all(m.fast_path_applicable(torch.empty(1, m.channels, *([8] * nd), device=dev))
                     for m in layers)
        assert on_hip == (route == "hip"), f"route {route}: NDC layers on HIP kernels = {on_hip}"
        opt = T.make_optimizer(model)
        dtype = torch.bfloat16 if w["autocast"] else None

        def step():
            if w["optimizer"]:
                return T.train_step(model, opt, images, targets, autocast_dtype=dtype)
            model.zero_grad(set_to_none=True)
            loss = T.dice_bce_loss(model(images), targets)
            loss.backward()
            return loss.detach()

        for i in range(warmup):
            loss = step()
            torch.cuda.synchronize()
            _progress(f"{workload} on the {route} route: warm-up step {i + 1} of {warmup} done")
        torch.cuda.reset_peak_memory_stats()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss = step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        _progress(f"{workload} on the {route} route: {steps} timed steps, {dt * 1e3:.1f} ms each")
        out = dict(ms_per_step=dt * 1e3, steps_per_s=1.0 / dt, loss=float(loss), steps=steps,
                   warmup=warmup, peak_mem_GB=torch.cuda.max_memory_allocated() / 1e9)
        del model, opt
        torch.cuda.empty_cache()
        return out

    return {r: run(r) for r in routes}


def model_workload(args) -> int:
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    w = MODEL_WORKLOADS[args.workload]
    routes = ["hip", "pytorch"] if args.ndc == "both" else [args.ndc]
    res = run_model_routes(args.workload, routes, args.warmup, args.steps)
    main_r = res[routes[0]]
    vox = w["batch"] * math.prod(w["size"])
    result = {
        "metric": w["metric"], "value": main_r["steps_per_s"], "unit": w["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w["autocast"] else "f32", "data": "synthetic",
        "config": {"workload": w["text"], "ndc": routes[0], "batch": w["batch"],
                   "size": list(w["size"])},
        "Gvoxel_per_s": vox / (main_r["ms_per_step"] * 1e-3) / 1e9,
        "routes": res,
        "roofline": None, "cpu_baseline": None,
    }
    if len(routes) == 2:
        result["hip_over_pytorch"] = res["hip"]["steps_per_s"] / res["pytorch"]["steps_per_s"]
    print(json.dumps(result))
    return 0


def mixer_workload(args) -> int:
    """One DeconvMixer (in_proj -> ReLU -> NDC layer -> out_proj, the caller of the hot path,
    deconver/deconver.py:22-46) at config 3's shape: batch 2, 128 channels, 64^3, 3x3x3,
    ratio 4; bf16 autocast or float32; one step = forward + backward.  Exists so that a
    rocprofv3 kernel trace of it shows what the projections around the update cost next to
    the update itself (bytes of z and of the update's output written by one GEMM and read
    by the next kernel)."""
    import torch

    import deconver_amd as dc

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    w = WORKLOAD
    dev = torch.device("cuda:0")
    C = w["channels"]
    torch.manual_seed(0)
    mixer = dc.DeconvMixer(C, C, kernel_size=w["kernel"], ratio=w["ratio"], groups=-1).to(dev)
    x = torch.randn(w["batch"], C, *w["spatial"], device=dev).requires_grad_(True)
    g = torch.randn(w["batch"], C, *w["spatial"], device=dev)
    dtype = torch.bfloat16 if args.dtype == "bf16" else None

    def step():
        mixer.zero_grad(set_to_none=True)
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=dtype is not None):
            y = mixer(x)
        y.backward(g.to(y.dtype))

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    ms = timed(step)
    extra = {}
    if dtype is not None:
        # the same mixer as it sits inside the network: its input (the norm's output) and the
        # gradient of its output are bf16 already, so the casts of the autocast boundary above
        # (float32 input -> bf16, input gradient -> float32) do not occur
        xb = x.detach().bfloat16().requires_grad_(True)
        gb = g.bfloat16()

        def step_in_network():
            mixer.zero_grad(set_to_none=True)
            xb.grad = None
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y = mixer(xb)
            y.backward(gb)

        extra["in_network_ms_per_step"] = timed(step_in_network)
    vox = w["batch"] * math.prod(w["spatial"])
    print(json.dumps({
        "metric": "DeconvMixer fwd+bwd Gvoxel/s", "value": vox / (ms * 1e-3) / 1e9,
        "unit": "Gvoxel/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype if args.dtype == "bf16" else "f32", "data": "synthetic",
        "config": {"workload": "one DeconvMixer at config 3's shape (batch 2, 128 channels, "
                               "64^3, 3x3x3, ratio 4), forward + backward; float32 input and "
                               "upstream gradient under bf16 autocast"},
        **extra, "roofline": None, "cpu_baseline": None}))
    return 0


LAYOUT_SHAPES = [   # (name, batch, channels, extent): the update's x has C channels, its z 4 C
    ("config 3: B 2, 128 ch, 64^3", 2, 128, 64),
    ("config 4 stage 0: B 2, 64 ch, 128^3", 2, 64, 128),
]


def layout_workload(args) -> int:
    """What a caller that holds channels-last tensors pays before the update: the kernels read
    channel-first (B, C, D, H, W) tensors, so `torch.channels_last_3d` inputs are copied into
    that layout by the autograd node (x and z before the forward, gout before the backward,
    and gx / gz come back channel-first).  Times those copies (bf16) next to the update's own
    forward + backward on the same shapes."""
    import torch

    from deconver_amd import _lib, ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _lib.get_library()
    dev = torch.device("cuda:0")
    rows = []

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    for name, B, C, n in LAYOUT_SHAPES:
        x, z, h, bias, g, sc = make_inputs(torch, torch.bfloat16, dev, B, C, (n, n, n), (3, 3, 3), 4)
        kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)
        x_cl = x.contiguous(memory_format=torch.channels_last_3d)
        z_cl = z.contiguous(memory_format=torch.channels_last_3d)
        ms_x = timed(lambda: x_cl.contiguous())
        ms_z = timed(lambda: z_cl.contiguous())
        ms_back = timed(lambda: z.contiguous(memory_format=torch.channels_last_3d))
        # the same copies by the library's tiled transposition (ndc_relayout)
        lx = timed(lambda: ops.to_channel_first(lib, x_cl))
        lz = timed(lambda: ops.to_channel_first(lib, z_cl))
        lback = timed(lambda: ops.to_channels_last(lib, z))
        assert torch.equal(ops.to_channel_first(lib, z_cl), z) and torch.equal(ops.to_channels_last(lib, z), z_cl)

        def step():
            res = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
            ops.update_backward(lib, x, z, res[1], h, bias, g, saved=res[2], **kw)

        ms_step = timed(step)
        U = B * C * n ** 3
        # a step that is handed x, z, gout channels-last and must return gx, gz channels-last
        # (x, z, gout in; out, gz and gx out: gx takes about what x does)
        extra = ms_x + 2 * ms_z + 2 * ms_back + ms_x
        lextra = lx + 2 * lz + 2 * lback + lx
        rows.append({"shape": name, "update_fwd_bwd_ms": ms_step,
                     "torch_copy": {"x_to_channel_first_ms": ms_x, "z_to_channel_first_ms": ms_z,
                                    "z_to_channels_last_ms": ms_back,
                                    "GBs_z_to_channel_first": 2 * 4 * U * 2 / (ms_z * 1e-3) / 1e9,
                                    "per_step_ms": extra, "over_update": extra / ms_step},
                     "ndc_relayout": {"x_to_channel_first_ms": lx, "z_to_channel_first_ms": lz,
                                      "z_to_channels_last_ms": lback,
                                      "GBs_z_to_channel_first": 2 * 4 * U * 2 / (lz * 1e-3) / 1e9,
                                      "per_step_ms": lextra, "over_update": lextra / ms_step}})
        del x, z, g, x_cl, z_cl
    print(json.dumps({
        "metric": "layout copies around the NDC update, ms", "value": rows[0]["ndc_relayout"]["per_step_ms"],
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": rows[0]["ndc_relayout"]["per_step_ms"], "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "torch.channels_last_3d <-> channel-first copies of the update's "
                               "operands (x, z, gout in; gx, gz out), bf16"},
        "shapes": rows, "roofline": None, "cpu_baseline": None}))
    return 0


SETTLE_S = 0.3   # untimed load before the warm-up steps of the headline workload (clock settling)

BLOCK_SHAPES = [("config 4, level 0: B 2, 64 ch, 128^3", 2, 64, 128 ** 3),
                ("config 4, level 1 (= config 3): B 2, 128 ch, 64^3", 2, 128, 64 ** 3),
                ("config 4, level 3: B 2, 512 ch, 16^3", 2, 512, 16 ** 3)]


def block_rows(torch, steps: int, warmup: int) -> list:
    """The HBM-bound kernels between the NDC layers of a Deconver block (InstanceNorm as row
    normalisation, the bias / GELU / residual pass after a 1x1 projection, and the projections
    themselves on the streaming GEMM), bf16, forward and
    backward, next to PyTorch's own kernels for the same arithmetic: ms and achieved GB/s on
    the bytes each must move (U = B*C*N elements of 2 bytes: norm forward 3 U, backward 5 U;
    bias + GELU on the 4C hidden tensor forward 8 U, backward 12 U; bias + residual 3 U)."""
    import torch.nn.functional as F

    import deconver_amd as dc
    from deconver_amd import _lib, ops

    lib = _lib.get_library()
    dev = torch.device("cuda:0")

    def timed(fn):
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    rows = []
    for name, B, C, n in BLOCK_SHAPES:
        U = B * C * n * 2    # bytes of one (B, C, N) bf16 tensor
        x = torch.randn(B * C, n, device=dev).bfloat16()
        g = torch.randn(B * C, n, device=dev).bfloat16()
        y, stats = ops.rownorm_forward(lib, x, 1e-5)
        x3 = x.view(B, C, n).requires_grad_(True)
        y3 = F.instance_norm(x3)
        g3 = g.view(B, C, n)
        r = {"shape": name}

        def put(key, ms, nbytes):
            r[key] = {"ms": ms, "GBs": nbytes / (ms * 1e-3) / 1e9, "hbm_frac": nbytes / (ms * 1e-3) / 8e12}

        put("norm_forward", timed(lambda: ops.rownorm_forward(lib, x, 1e-5)), 3 * U)
        put("norm_backward", timed(lambda: ops.rownorm_backward(lib, g, y, stats)), 5 * U)
        put("norm_forward_pytorch", timed(lambda: F.instance_norm(x3)), 3 * U)
        put("norm_backward_pytorch", timed(lambda: torch.autograd.grad(y3, x3, g3, retain_graph=True)), 5 * U)
        del x, g, y, x3, y3, g3
        # LayerNorm over the channel axis (the blocks' default norm in the reference), HIP kernels
        # next to the reference's moved-axis form on PyTorch's kernels
        xc = torch.randn(B, C, n, device=dev).bfloat16()
        gc = torch.randn(B, C, n, device=dev).bfloat16()
        wln, bln = torch.rand(C, device=dev) + 0.5, torch.rand(C, device=dev)
        yc, sc_ = ops.chnorm_forward(lib, xc, wln, bln, 1e-5)
        put("layernorm_forward", timed(lambda: ops.chnorm_forward(lib, xc, wln, bln, 1e-5)), 3 * U)
        put("layernorm_backward", timed(lambda: ops.chnorm_backward(lib, gc, xc, sc_, wln)), 5 * U)
        xr = xc.clone().requires_grad_(True)
        w16, b16_ = wln.bfloat16(), bln.bfloat16()
        put("layernorm_forward_pytorch",
            timed(lambda: F.layer_norm(xr.movedim(1, -1), (C,), w16, b16_, 1e-5).movedim(-1, 1).contiguous()), 3 * U)
        yr = F.layer_norm(xr.movedim(1, -1), (C,), w16, b16_, 1e-5).movedim(-1, 1)
        put("layernorm_backward_pytorch", timed(lambda: torch.autograd.grad(yr, xr, gc, retain_graph=True)), 5 * U)
        del xc, gc, yc, sc_, xr, yr
        z = torch.randn(B, 4 * C, n, device=dev).bfloat16()
        gz = torch.randn(B, 4 * C, n, device=dev).bfloat16()
        bias = torch.randn(4 * C, device=dev)
        put("bias_gelu_forward", timed(lambda: ops.bias_act(lib, z, bias, None, "gelu")), 8 * U)
        put("bias_gelu_backward", timed(lambda: ops.bias_act_backward(lib, gz, z, bias, "gelu")), 12 * U)
        b16 = bias.bfloat16().view(1, -1, 1)
        put("bias_gelu_forward_pytorch", timed(lambda: F.gelu(z + b16)), 8 * U)
        zz = (z + b16).requires_grad_(True)
        yy = F.gelu(zz)
        put("bias_gelu_backward_pytorch",
            timed(lambda: (torch.autograd.grad(yy, zz, gz, retain_graph=True)[0].sum(2, dtype=torch.float32).sum(0))), 12 * U)
        del z, gz, zz, yy
        z1 = torch.randn(B, C, n, device=dev).bfloat16()
        res = torch.randn(B, C, n, device=dev).bfloat16()
        b1 = torch.randn(C, device=dev)
        put("bias_residual", timed(lambda: ops.bias_act(lib, z1, b1, res, None)), 3 * U)
        b1h = b1.bfloat16().view(1, -1, 1)
        put("bias_residual_pytorch", timed(lambda: res + (z1 + b1h)), 3 * U)
        del z1
        # the 1x1 projections themselves: the library's streaming GEMM next to hipBLASLt (one
        # batched launch with the weight shared through a zero stride), where the kernel applies
        if lib.pointwise_gemm_supported(C, 4 * C, n, _lib.NDC_BF16) and lib.pointwise_gemm_supported(4 * C, C, n, _lib.NDC_BF16):
            xs = torch.randn(B, C, n, device=dev).bfloat16()
            hs = torch.randn(B, 4 * C, n, device=dev).bfloat16()
            w_up = torch.randn(4 * C, C, device=dev) / C ** 0.5
            w_dn = torch.randn(C, 4 * C, device=dev) / (4 * C) ** 0.5
            f_up, f_dn, f_sq = (ops.pointwise_pack(lib, w) for w in (w_up, w_dn, w_dn[:, :C].contiguous()))
            f_upT = ops.pointwise_pack(lib, w_dn, transposed=True)     # (C x 4C storage) -> applies 4C x C
            out_up, out_dn = torch.empty_like(hs), torch.empty_like(xs)
            up16 = w_up.bfloat16().unsqueeze(0).expand(B, -1, -1)
            dn16 = w_dn.bfloat16().unsqueeze(0).expand(B, -1, -1)
            sq16 = w_dn[:, :C].bfloat16().unsqueeze(0).expand(B, -1, -1)
            put("project_up", timed(lambda: ops.pointwise_gemm(lib, xs, f_up, 4 * C)), 5 * U)
            put("project_up_hipblaslt", timed(lambda: torch.bmm(up16, xs, out=out_up)), 5 * U)
            put("project_down", timed(lambda: ops.pointwise_gemm(lib, hs, f_dn, C)), 5 * U)
            put("project_down_hipblaslt", timed(lambda: torch.bmm(dn16, hs, out=out_dn)), 5 * U)
            put("project_square", timed(lambda: ops.pointwise_gemm(lib, xs, f_sq, C)), 2 * U)
            put("project_square_hipblaslt", timed(lambda: torch.bmm(sq16, xs, out=out_dn)), 2 * U)
            # with their tails: up + bias + GELU keeping the product (1 + 4 + 4 U), down + bias +
            # residual (4 + 1 + 1 U), and the input gradient of `down` through the GELU with the
            # bias gradient's sums (1 + 4 + 4 U) -- against GEMM + separate pass above
            bias4 = torch.randn(4 * C, device=dev)
            put("project_up_bias_gelu", timed(lambda: ops.pointwise_gemm(lib, xs, f_up, 4 * C, bias4, None, "gelu", keep_z=True)), 9 * U)
            put("project_down_bias_residual", timed(lambda: ops.pointwise_gemm(lib, hs, f_dn, C, b1, res, None)), 6 * U)
            put("project_back_through_gelu", timed(lambda: ops.pointwise_gemm_actgrad(lib, xs, f_upT, 4 * C, hs, bias4, "gelu")), 9 * U)
            del xs, hs, out_up, out_dn
        del res
        rows.append(r)
        torch.cuda.empty_cache()
    return rows


def block_workload(args) -> int:
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    rows = block_rows(torch, args.steps, args.warmup)
    first = rows[0]
    ms = sum(first[k]["ms"] for k in ("norm_forward", "norm_backward", "bias_gelu_forward", "bias_gelu_backward",
                                      "bias_residual"))
    print(json.dumps({
        "metric": "Deconver block: norm and projection-tail kernels, ms", "value": ms, "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "row normalisation (InstanceNorm) and bias / GELU / residual passes of a "
                               "Deconver block at config 4's levels, bf16, HIP kernels next to PyTorch's"},
        "shapes": rows,
        "roofline": {"kernel": "norm_backward", "bound": "hbm", "achieved": first["norm_backward"]["GBs"],
                     "peak": 8000.0, "unit": "GB/s", "frac": first["norm_backward"]["hbm_frac"], "traffic": None},
        "cpu_baseline": None}))
    return 0


def graphed_workload(args) -> int:
    """Training steps on ONE small sample (a 3-D step on a 32^3 volume under bf16 autocast, a 2-D
    step on a 128^2 image in float32): there a step is bound by the rate at which the host
    launches its ~600 kernels, and replaying it from a HIP graph (training.GraphedTrainStep)
    removes that bound.  ms per step eager and replayed, same networks as train3d / model2d."""
    import torch
    from torch import nn

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    import deconver_amd as dc
    from deconver_amd import training

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    rows = []
    for name, key, size, autocast in (("3-D, one 32^3 volume, bf16 autocast", "train3d", (32, 32, 32), torch.bfloat16),
                                      ("2-D, one 128^2 image, float32", "model2d", (128, 128), None)):
        w = MODEL_WORKLOADS[key]
        torch.manual_seed(0)
        norm = nn.InstanceNorm3d if len(size) == 3 else nn.InstanceNorm2d
        model = dc.Deconver(norm=norm, **w["net"]).cuda()
        opt = training.make_optimizer(model, capturable=True)
        make = training.ellipsoid_phantoms if len(size) == 3 else training.smoothed_noise_masks
        images, targets = make(1, w["net"]["in_channels"], size, seed=0, device="cuda")
        eager = timed(lambda: training.train_step(model, opt, images, targets, autocast_dtype=autocast))
        step = training.GraphedTrainStep(model, opt, images, targets, autocast_dtype=autocast)
        replayed = timed(lambda: step(images, targets))
        rows.append({"case": name, "eager_ms": eager, "graph_ms": replayed, "speedup": eager / replayed})
        del model, opt, step
        torch.cuda.empty_cache()
    print(json.dumps({
        "metric": "small-batch training step replayed from a HIP graph, ms", "value": rows[0]["graph_ms"],
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": rows[0]["graph_ms"],
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Deconver training steps on one small sample, eager and replayed from a HIP graph"},
        "cases": rows, "roofline": None, "cpu_baseline": None}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: 200 timed steps after 50 for the headline workload (0.45 s in all: a 20-step region
    # of 36 ms ends before the clocks have settled and reads 2-3 % slow and noisy: 1.81-1.83 against
    # 1.772 +- 0.001 ms), 50 after 10 for the other kernel-level workloads, 20 after 5 for the
    # model-level ones
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--dtype", choices=("bf16", "fp32"), default="bf16")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--matrix", action="store_true",
                    help="run with the matrix-instruction kernel family on (ndc_matrix_kernels(1)): "
                         "not the specified path, reported for comparison")
    ap.add_argument("--no-train", action="store_true",
                    help="skip the Deconver-3D train-step leg that follows the timed region")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the config-5 forward sweep and the 2-D 5x5 layers that follow the timed region")
    ap.add_argument("--recompute", action="store_true",
                    help="backward re-gathers the denominator and ratio (as the reference does) "
                         "instead of reading the forward's copies")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--build-probe", action="store_true",
                    help="with --workload valu: compile the probe (no GPU needed) and exit")
    ap.add_argument("--workload", choices=("ndc", "sweep", "accuracy", "grid", "valu", "train3d", "model2d", "mixer", "layout", "block",
                                           "graphed"),
                    default="ndc",
                    help="ndc: the headline update node (default); the others are model level")
    ap.add_argument("--ndc", choices=("hip", "pytorch", "both"), default="hip",
                    help="model-level workloads: which route the NDC layers take")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = {"ndc": 200, "sweep": 50, "block": 50, "mixer": 50}.get(args.workload, 20)
    if args.warmup is None:
        args.warmup = {"ndc": 50, "sweep": 10, "block": 10, "mixer": 10}.get(args.workload, 5)
    if args.gpus != 1:
        print("bench.py measures the one-GPU hot path only: this build has no multi-GPU code "
              "path (every box has one GPU); run with --gpus 1", file=sys.stderr)
        return 2
    if args.matrix:
        os.environ["DECONVER_NDC_MATRIX"] = "1"   # read when the library is loaded

    if args.workload == "sweep":
        return sweep_workload(args)
    if args.workload == "accuracy":
        return accuracy_workload(args)
    if args.workload == "grid":
        return grid_workload(args)
    if args.workload == "valu":
        return valu_workload(args)
    if args.workload == "mixer":
        return mixer_workload(args)
    if args.workload == "layout":
        return layout_workload(args)
    if args.workload == "block":
        return block_workload(args)
    if args.workload == "graphed":
        return graphed_workload(args)
    if args.workload != "ndc":
        return model_workload(args)

    import torch

    from deconver_amd import _lib, ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the NDC update has no CPU path)", file=sys.stderr)
        return 2
    lib = _lib.get_library()
    lib.matrix_kernels(bool(args.matrix))
    dev = torch.device("cuda:0")
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    esz = 2 if dtype == torch.bfloat16 else 4
    w = WORKLOAD
    x, z, h, bias, g, sc = make_inputs(torch, dtype, dev, w["batch"], w["channels"], w["spatial"],
                                       w["kernel"], w["ratio"])
    C = w["channels"]
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)
    geom = ops.make_geom_for(x, h, C, 1, sc, 1e-16, True)
    assert lib.fused_supported(geom), "the headline workload must run on the fused kernels"

    keep = (not args.recompute) and lib.backward_uses_saved(geom)

    def step():
        # the launch sequence of the autograd node (deconver_amd/functional.py): the filter
        # table is packed once per update and serves its forward and its backward
        taps = ops.prepare_taps(lib, x, h, groups=C, m=1, sc=sc)
        res = ops.update_forward(lib, x, z, h, bias, save_ratio=keep, taps=taps, **kw)
        return ops.update_backward(lib, x, z, res[1], h, bias, g,
                                   saved=res[2] if keep else None, taps=taps, **kw)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # measured device-copy bandwidth (1 GiB read + 1 GiB written), for scale next to the
    # published 8 TB/s the roofline is quoted on
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(5):
        dst.copy_(src)
    c1.record()
    torch.cuda.synchronize()
    copy_gbs = 5 * 2 * src.numel() * 4 / (c0.elapsed_time(c1) * 1e-3) / 1e9
    del src, dst

    # the same step, untimed, until the device has been busy for SETTLE_S: after start-up and the
    # set-up above the clocks are still settling, and a timed region that begins within the first
    # tens of milliseconds of load reads 2-3 % slow (1.81-1.83 against 1.772 ms); then the W
    # warm-up steps and the K timed ones as asked
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < SETTLE_S:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # per-kernel device time: events on the stream the library launches on
    n_probe = max(3, min(10, args.steps))

    def kernel_times():
        fwd_ms, pass_ms = [], []
        for _ in range(n_probe):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            # an untimed call first: the previous iteration ended in a host synchronisation, and
            # the first kernel after an idle gap runs at ramping clocks
            ops.update_forward(lib, x, z, h, bias, save_ratio=keep, **kw)
            e0.record()
            res = ops.update_forward(lib, x, z, h, bias, save_ratio=keep, **kw)
            e1.record()
            pt = []
            ops.update_backward(lib, x, z, res[1], h, bias, g, pass_times=pt,
                                saved=res[2] if keep else None, **kw)
            torch.cuda.synchronize()
            fwd_ms.append(e0.elapsed_time(e1))
            pass_ms.append(pt)
        return {
            "forward": statistics.mean(fwd_ms),
            "backward_pass1": statistics.mean(p[0] for p in pass_ms),
            "backward_pass2": statistics.mean(p[1] for p in pass_ms),
            "backward_reduce": statistics.mean(p[2] for p in pass_ms),
        }

    k_ms = kernel_times()

    sp = w["spatial"]
    vox = w["batch"] * sp[0] * sp[1] * sp[2]
    U = vox * C
    alg = {"forward": 9 * U * esz, "backward_pass1": 10 * U * esz, "backward_pass2": 4 * U * esz}
    dominant = max(alg, key=lambda k: k_ms[k])
    achieved = alg[dominant] / (k_ms[dominant] * 1e-3) / 1e9
    # HBM bytes per launch from rocprofv3's FETCH_SIZE / WRITE_SIZE counters: they cannot be
    # read from inside this process, so the figure is the one recorded in profiles/traffic.json
    # by the profiling runs described there, stamped with the commit it was measured at
    traffic = traffic_at = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        try:
            rec = json.load(open(tpath))
            traffic = rec.get(args.dtype + ("_matrix" if args.matrix else ""), {}).get(dominant)
            traffic_at = rec.get("measured_at_commit")
        except (ValueError, OSError):
            traffic = None
    roofline = {
        "kernel": dominant,
        "bound": "hbm",
        "achieved": achieved,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS,
        "traffic": traffic,
        "traffic_measured_at_commit": traffic_at,
        "algorithmic_bytes": alg[dominant],
        "avg_launch_ms": k_ms[dominant],
        # the three kernels side by side (two of them are within a few percent of each other,
        # so which one is "dominant" can differ from run to run)
        "per_kernel": {k: {"algorithmic_bytes": alg[k], "avg_launch_ms": k_ms[k],
                           "achieved": alg[k] / (k_ms[k] * 1e-3) / 1e9,
                           "frac": alg[k] / (k_ms[k] * 1e-3) / 1e9 / HBM_PEAK_GBS} for k in alg},
    }
    step_bytes = 23 * U * esz
    result = {
        "metric": "NDC mixer fwd+bwd Gvoxel/s",
        "value": vox / (ms_per_step * 1e-3) / 1e9,
        "unit": "Gvoxel/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "pre_warmup_s": SETTLE_S,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {
            "workload": "config 3: one NDC source update, 3-D, batch 2, 128 depthwise channels, "
                        "64^3 voxels, 3x3x3 filter, ratio 4 (512 source channels), "
                        f"{args.dtype} storage / float32 accumulation; forward + input-, source-, "
                        "filter- and bias-gradient",
            "batch": w["batch"], "channels": C, "spatial": list(sp), "kernel": list(w["kernel"]),
            "ratio": w["ratio"], "num_iters": 1,
        },
        "channel_voxels_per_s": U / (ms_per_step * 1e-3),
        "step_algorithmic_bytes": step_bytes,
        "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "kernel_ms": k_ms,
        "measured_copy_GBs": copy_gbs,
        "backward_reads_forward_ratio": bool(keep),
        "roofline": roofline,
    }
    if dtype == torch.bfloat16 and keep and not args.matrix:
        # The same step on the OTHER kernel family (ndc_matrix_kernels(1): tap sums on the
        # 4x4x4 matrix instruction).  The path is specified without matrix instructions, so this
        # is not `value`; it is reported because it is the faster form on this GPU.
        lib.matrix_kernels(True)
        try:
            for _ in range(args.warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                step()
            torch.cuda.synchronize()
            m_ms = (time.perf_counter() - t0) / args.steps * 1e3
            mk = kernel_times()
        finally:
            lib.matrix_kernels(False)
        props = torch.cuda.get_device_properties(dev)
        simds = props.multi_processor_count * 4
        hz = getattr(props, "clock_rate", 2400000) * 1e3   # kHz; MI355X peak engine clock 2.4 GHz
        least = {k: U / 64 * n / simds * CLOCKS_PER_MFMA / hz * 1e3 for k, n in MFMA_PER_64_CHANNEL_VOXELS.items()}
        result["matrix_instruction_variant"] = {
            "ms_per_step": m_ms, "value": vox / (m_ms * 1e-3) / 1e9, "unit": "Gvoxel/s",
            "step_hbm_frac": step_bytes / (m_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "kernel_ms": mk,
            "hbm_frac": {k: alg[k] / (mk[k] * 1e-3) / 1e9 / HBM_PEAK_GBS for k in alg},
            # the least time its matrix instructions alone take at the measured issue rate
            "mfma_per_64_channel_voxels": MFMA_PER_64_CHANNEL_VOXELS, "clocks_per_mfma": CLOCKS_PER_MFMA,
            "mfma_least_ms": least,
        }
    if dtype == torch.bfloat16 and keep and not args.matrix:
        # the default kernels are bound by vector issue, not by HBM: the least time their
        # v_dot2c_f32_bf16 alone take, at the issue rate `--workload valu` measured
        props = torch.cuda.get_device_properties(dev)
        lanes = props.multi_processor_count * 4 * 64
        hz = getattr(props, "clock_rate", 2400000) * 1e3
        least = {k: U * n / lanes * CLOCKS_PER_DOT2C / hz * 1e3 for k, n in DOT2_PER_CHANNEL_VOXEL.items()}
        result["vector_ceiling"] = {
            "dot2c_per_channel_voxel": DOT2_PER_CHANNEL_VOXEL, "clocks_per_dot2c": CLOCKS_PER_DOT2C,
            "least_ms": least,
            "frac": {k: least[k] / k_ms[k] for k in least},
            "step_frac": sum(least.values()) / sum(k_ms[k] for k in least),
        }
    _progress(f"update node: {ms_per_step:.3f} ms per step")
    if not args.no_extras and not args.matrix:
        # outside the timed region, about a second: the other shapes the baseline asks to be
        # reported -- config 5's forward-only sweep (bf16) and the 2-D 5x5 form (float32)
        del x, z, g
        torch.cuda.empty_cache()
        x = z = g = None
        result["sweep"] = {"workload": "config 5: forward-only NDC update, 3x3x3, ratio 4, bf16, inference "
                                       "form; hbm_frac on 9 U e",
                           "shapes": sweep_rows(torch, lib, ops, dev, 10, 50)}
        result["layers_2d"] = {"workload": "2-D 5x5 update node, depthwise, ratio 4, float32, forward + "
                                           "backward; hbm_frac on 23 U e",
                               "layers": layers_2d_rows(torch, lib, ops, dev, 10, 50)}
        result["block_kernels"] = {"workload": "InstanceNorm and bias / GELU / residual passes of a Deconver block "
                                               "at config 4's levels, bf16, HIP kernels next to PyTorch's; GB/s on "
                                               "whole passes over the tensor",
                                   "shapes": block_rows(torch, 20, 5)}
        _progress("config-5 sweep, 2-D layers and block kernels done")
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch)
        _progress("CPU baseline done")
    if not args.no_train:
        # the second half of the metric, outside the timed region above: Deconver-3D train
        # steps per second (config 4) with the NDC layers on the HIP kernels and, for
        # reference, on the layers' PyTorch route on the same GPU
        x = z = g = None
        torch.cuda.empty_cache()
        try:
            if "layers_2d" in result:
                # config 2 (model level): the 2-D network's forward + backward on the HIP route
                m2 = run_model_routes("model2d", ["hip"], warmup=5, steps=20)["hip"]
                result["layers_2d"]["model2d_steps_per_s"] = m2["steps_per_s"]
                result["layers_2d"]["model2d_ms_per_step"] = m2["ms_per_step"]
                result["layers_2d"]["model2d_workload"] = MODEL_WORKLOADS["model2d"]["text"]
            t3 = run_model_routes("train3d", ["hip"], warmup=3, steps=10)
            t3.update(run_model_routes("train3d", ["pytorch"], warmup=1, steps=2))
            result["train3d_steps_per_s"] = t3["hip"]["steps_per_s"]
            result["train3d_steps_per_s_pytorch_route"] = t3["pytorch"]["steps_per_s"]
            result["train3d"] = {"workload": MODEL_WORKLOADS["train3d"]["text"], "routes": t3,
                                 "hip_over_pytorch": t3["hip"]["steps_per_s"] / t3["pytorch"]["steps_per_s"]}
            if "matrix_instruction_variant" in result:
                # the same train step with the other kernel family on (see above: not the metric)
                lib.matrix_kernels(True)
                try:
                    tm = run_model_routes("train3d", ["hip"], warmup=3, steps=10)["hip"]
                finally:
                    lib.matrix_kernels(False)
                result["matrix_instruction_variant"]["train3d_steps_per_s"] = tm["steps_per_s"]
        except Exception as exc:   # the headline line above is complete without this leg
            result["train3d_error"] = f"{type(exc).__name__}: {exc}"
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
