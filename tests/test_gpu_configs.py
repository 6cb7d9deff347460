"""The benchmark configurations at their full sizes on a real MI355X, through the C ABI.

Depthwise channels are independent end to end, so any channel slice of a full-size result
must equal the oracle evaluated on that slice alone -- which the CPU does in seconds.  This
covers what no small case reaches: the row-band / column-strip shapes the launch planner
picks for 128- and 192-column rows, volumes beyond 2^31 elements, the inference form of the
forward call (no t1, nothing kept) and the kept-ratio backward kernels the benchmark times.
Tolerances: ``max|d| / max|ref|`` <= 2e-2 for bfloat16 storage, <= 1e-4 for float32.
"""

import sys

import pytest
import torch

from deconver_amd import _lib, ops
from oracle import ndc_oracle as O

pytestmark = pytest.mark.gpu

SC = 4
KS = (3, 3, 3)
EPS = 1e-16


def _inputs(B, C, sp, dtype, seed=0, with_gout=True):
    """Half-normal x, signed z, softplus filter, small bias (config 3 / 5 construction),
    drawn on the GPU (the CPU generator needs tens of seconds for 2^30 normals); the oracle
    gets the channel slices it needs copied back."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen, device="cuda")
    h = torch.nn.functional.softplus(0.1 * rn(C, SC, *KS))
    x = rn(B, C, *sp).abs_().to(dtype)
    z = rn(B, C * SC, *sp).mul_(0.5).to(dtype)
    bias = 0.1 * rn(C * SC)
    gout = rn(B, C * SC, *sp).to(dtype) if with_gout else None
    return x, z, h, bias, gout


def _slice(c, x, z, h, bias, gout=None):
    cs = slice(c * SC, (c + 1) * SC)
    out = [x[:, c:c + 1].cpu().double(), z[:, cs].cpu().double(), h[c:c + 1].cpu().double(),
           bias[cs].cpu().double()]
    if gout is not None:
        out.append(gout[:, cs].cpu().double())
    return cs, out


# config 5: (channels, extent, batch), bottleneck to full resolution
SWEEP = [(512, 16, 4), (256, 32, 2), (64, 128, 1), (32, 192, 1)]


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("C,n,B", SWEEP)
def test_config5_inference_form_channel_slices(C, n, B, matrix):
    """Forward only, bfloat16, t1 = null, nothing kept: the call `bench.py --workload sweep`
    times, at each of its four shapes, on both bf16 kernel families (the 192-column shape is
    outside the matrix-instruction family's widths and runs the default kernels either way)."""
    print("case config5", C, n, B, matrix, flush=True)
    sp = (n, n, n)
    x, z, h, bias, _ = _inputs(B, C, sp, torch.bfloat16, with_gout=False)
    lib = _lib.get_library()
    dev = [x, z, h, bias]
    g = ops.make_geom_for(dev[0], dev[2], C, 1, SC, EPS, True)
    assert lib.fused_supported(g), "the fused kernels must cover every config-5 shape"
    assert lib.matrix_kernels(matrix) == matrix
    try:
        out, t1 = ops.update_forward(lib, *dev, groups=C, m=1, sc=SC, eps=EPS, relu_input=True,
                                     need_t1=False)
        torch.cuda.synchronize()
    finally:
        lib.matrix_kernels(False)
    assert t1 is None
    for c in (0, C // 3, C - 1):
        cs, d = _slice(c, x, z, h, bias)
        ro, _ = O.update_grouped(d[0], d[1], d[2], d[3], 1, 1, SC, EPS, True)
        e = O.rel_err(out[:, cs].cpu(), ro)
        assert e < 2e-2, f"out channel {c}: {e:.3e}"


@pytest.mark.parametrize("dtype,tol,matrix", [(torch.bfloat16, 2e-2, False), (torch.float32, 1e-4, False),
                                              (torch.bfloat16, 2e-2, True)])
def test_config3_kept_ratio_backward_channel_slices(dtype, tol, matrix):
    """Config 3 at full size with the forward's s/d and n/d kept: the kernels the headline
    benchmark times (forward with four outputs, both kept-ratio backward passes), including
    the two kept tensors themselves."""
    B, C, sp = 2, 128, (64, 64, 64)
    x, z, h, bias, gout = _inputs(B, C, sp, dtype)
    lib = _lib.get_library()
    dev = [x, z, h, bias, gout]
    kw = dict(groups=C, m=1, sc=SC, eps=EPS, relu_input=True)
    assert lib.matrix_kernels(matrix) == matrix
    try:
        out, t1, saved = ops.update_forward(lib, *dev[:4], save_ratio=True, **kw)
        gx, gz, gh, gb = ops.update_backward(lib, dev[0], dev[1], t1, dev[2], dev[3], dev[4],
                                             saved=saved, **kw)
        torch.cuda.synchronize()
    finally:
        lib.matrix_kernels(False)
    kept = saved
    for c in (1, 64, 126):
        cs, d = _slice(c, x, z, h, bias, gout)
        ro, rt1 = O.update_grouped(d[0], d[1], d[2], d[3], 1, 1, SC, EPS, True)
        rgx, rgz, rgh, rgb = O.update_backward(d[0], d[1], d[2], d[3], d[4], 1, 1, SC, EPS, True)
        s = O.rectified_source(d[1], d[3], True)
        den = O.op_A(rt1, d[2], 1, 1, SC) + EPS
        num = O.op_A(d[0], d[2], 1, 1, SC) + EPS
        errs = dict(out=O.rel_err(out[:, cs].cpu(), ro), t1=O.rel_err(t1[:, c:c + 1].cpu(), rt1),
                    s_over_den=O.rel_err(kept[0][:, cs].cpu(), s / den),
                    ratio=O.rel_err(kept[1][:, cs].cpu(), num / den),
                    gx=O.rel_err(gx[:, c:c + 1].cpu(), rgx), gz=O.rel_err(gz[:, cs].cpu(), rgz),
                    gh=O.rel_err(gh[c:c + 1].cpu(), rgh), gb=O.rel_err(gb[cs].cpu(), rgb))
        bad = {k: v for k, v in errs.items() if not v < tol}
        assert not bad, f"channel {c}: {bad} (all: {errs})"


@pytest.mark.parametrize("matrix", [False, True])
def test_config4_stage0_layer_channel_slices(matrix):
    """Config 4's full-resolution layer: batch 2, 64 channels, 128^3, bfloat16.  The source
    tensors hold 2^30 elements (2 GiB) each, so tensor bases need 64-bit arithmetic; rows of
    128 columns take the widest column strip.  Forward and the kept-ratio backward, on both
    bf16 kernel families (at this width the second family's forward and pass 2)."""
    B, C, sp = 2, 64, (128, 128, 128)
    dtype = torch.bfloat16
    x, z, h, bias, gout = _inputs(B, C, sp, dtype, seed=4)
    assert z.numel() == 2 ** 30
    lib = _lib.get_library()
    dev = [x, z, h, bias, gout]
    kw = dict(groups=C, m=1, sc=SC, eps=EPS, relu_input=True)
    assert lib.matrix_kernels(matrix) == matrix
    try:
        out, t1, saved = ops.update_forward(lib, *dev[:4], save_ratio=True, **kw)
        gx, gz, gh, gb = ops.update_backward(lib, dev[0], dev[1], t1, dev[2], dev[3], dev[4],
                                             saved=saved, **kw)
        torch.cuda.synchronize()
    finally:
        lib.matrix_kernels(False)
    del saved
    # the last channel of the last sample sits past the 2^31-byte and 2^31-element marks
    for c in (0, C - 1):
        cs, d = _slice(c, x, z, h, bias, gout)
        ro, _ = O.update_grouped(d[0], d[1], d[2], d[3], 1, 1, SC, EPS, True)
        rgx, rgz, rgh, rgb = O.update_backward(d[0], d[1], d[2], d[3], d[4], 1, 1, SC, EPS, True)
        errs = dict(out=O.rel_err(out[:, cs].cpu(), ro), gx=O.rel_err(gx[:, c:c + 1].cpu(), rgx),
                    gz=O.rel_err(gz[:, cs].cpu(), rgz), gh=O.rel_err(gh[c:c + 1].cpu(), rgh),
                    gb=O.rel_err(gb[cs].cpu(), rgb))
        bad = {k: v for k, v in errs.items() if not v < 2e-2}
        assert not bad, f"channel {c}: {bad} (all: {errs})"


def test_config4_full_size_train_steps_on_both_routes():
    """Config 4 at full size (Deconver 3-D, widths 64-512, batch 2 of 128^3, bf16 autocast,
    Dice+BCE, AdamW): two training steps from the same weights with the NDC layers on the HIP
    kernels and on the layers' PyTorch route; the losses of both steps agree to 3e-2 (bf16
    arithmetic on either side), and the step lowers the loss on both."""
    from torch import nn

    import deconver_amd as dc
    from deconver_amd import training as T

    net = dict(in_channels=2, out_channels=1, spatial_dims=3, encoder_depth=(1, 1, 1, 1),
               encoder_width=(64, 128, 256, 512), strides=(1, 2, 2, 2), decoder_depth=(1, 1, 1),
               kernel_size=(3, 3, 3), groups=-1, ratio=4, norm=nn.InstanceNorm3d)
    images, targets = T.ellipsoid_phantoms(2, 2, (128, 128, 128), seed=0, device="cuda")
    losses = {}
    for route, extra in (("hip", {}), ("pytorch", {"dilation": 1})):
        torch.manual_seed(0)
        model = dc.Deconver(**net, **extra).cuda()
        layers = [m for m in model.modules() if isinstance(m, dc.Deconv)]
        on_hip = all(m.fast_path_applicable(torch.empty(1, m.channels, 8, 8, 8, device="cuda"))
                     for m in layers)
        assert on_hip == (route == "hip") and len(layers) == 7
        opt = T.make_optimizer(model)
        losses[route] = []
        for step in range(2):
            losses[route].append(float(T.train_step(model, opt, images, targets,
                                                    autocast_dtype=torch.bfloat16)))
            # straight to the process's stderr (past pytest's capture): this test runs for a
            # minute or two, most of it the library's kernel selection on the PyTorch route
            sys.__stderr__.write(f"[config 4, {route} route] step {step + 1}: loss {losses[route][-1]:.4f}\n")
            sys.__stderr__.flush()
        del model, opt
        torch.cuda.empty_cache()
    for a, b in zip(losses["hip"], losses["pytorch"]):
        assert abs(a - b) < 3e-2 * abs(b), losses
    assert losses["hip"][1] < losses["hip"][0] and losses["pytorch"][1] < losses["pytorch"][0], losses
