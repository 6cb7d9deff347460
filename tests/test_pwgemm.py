"""The streaming GEMM of the 1x1 projections (``ndc_pointwise_gemm``) against ``conv1d`` in
float64 (the map of the reference's ``Linear``, layers/linear.py:53-58, with the tail its callers
apply, deconver.py:41-46, 60-64, layers/mlp.py:40-63)."""

import pytest
import torch
import torch.nn.functional as F

from deconver_amd import _lib, ops
from tests.helpers import hostcheck_library


def _case(B, cin, cout, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, cin, n, generator=g).bfloat16()
    w = torch.randn(cout, cin, generator=g) / cin ** 0.5
    bias = torch.randn(cout, generator=g)
    res = torch.randn(B, cout, n, generator=g).bfloat16()
    return x, w, bias, res


def _reference(x, w, bias, res, act):
    """float64 on the bf16-rounded operands (the kernel rounds W to bf16 when packing)."""
    z = F.conv1d(x.double(), w.bfloat16().double().unsqueeze(-1))
    u = z if bias is None else z + bias.double().view(1, -1, 1)
    y = {None: lambda t: t, "relu": torch.relu, "gelu": F.gelu}[act](u)
    return z, (y if res is None else y + res.double())


def _rel(a, ref):
    return float((a.double().cpu() - ref).abs().max() / ref.abs().max())


def test_support_predicate():
    lib = hostcheck_library()
    bf, f32 = _lib.NDC_BF16, _lib.NDC_F32
    assert lib.pointwise_gemm_supported(64, 256, 128 ** 3, bf)
    assert lib.pointwise_gemm_supported(256, 64, 64, bf) and lib.pointwise_gemm_supported(128, 512, 4096, bf)
    assert not lib.pointwise_gemm_supported(64, 256, 128 ** 3, f32)       # bfloat16 only
    assert lib.pointwise_gemm_supported(512, 128, 4096, bf)               # many input channels: up to 128 out
    assert not lib.pointwise_gemm_supported(512, 256, 4096, bf) and not lib.pointwise_gemm_supported(336, 64, 4096, bf)
    assert not lib.pointwise_gemm_supported(256, 512, 4096, bf)           # weights beyond 128 KiB
    assert not lib.pointwise_gemm_supported(64, 48, 4096, bf)             # cout not a multiple of 32
    assert not lib.pointwise_gemm_supported(64, 64, 100, bf)              # n not a multiple of 64
    assert lib.pointwise_weight_bytes(64, 256) == 64 * 256 * 2


@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pack_order_on_the_host_build(transposed, dtype):
    lib = hostcheck_library()
    cout, cin = 64, 128
    w = (torch.arange(cout * cin, dtype=torch.float32).view(cout, cin) % 251 - 125).to(dtype)
    stored = w.t().contiguous() if transposed else w
    frag = ops.pointwise_pack(lib, stored, transposed=transposed).view(cout // 32, cin // 16, 2, 32, 8)
    # fragment (c, s), lane (kb, i), element e  <->  W[32 c + i][16 s + 8 kb + e]
    want = w.bfloat16().view(cout // 32, 32, cin // 16, 2, 8).permute(0, 2, 3, 1, 4)
    assert torch.equal(frag, want)


@pytest.mark.parametrize("B,cin,cout,n", [(2, 64, 96, 128), (1, 128, 32, 64), (1, 256, 64, 64), (1, 384, 64, 64)])
@pytest.mark.parametrize("act,with_bias,with_res,keep", [(None, False, False, False), (None, True, True, False),
                                                          ("gelu", True, False, True), ("relu", False, True, True)])
def test_host_build_matches_float64(B, cin, cout, n, act, with_bias, with_res, keep):
    lib = hostcheck_library()
    if cin > 256 and (act or keep):
        x, w, _, _ = _case(B, cin, cout, n)
        assert not ops.pointwise_gemm_applies(lib, x, cout, act, keep)
        with pytest.raises(_lib.NdcError):    # plain product, bias and residual only
            ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w), cout, None, None, act, keep_z=keep)
        return
    x, w, bias, res = _case(B, cin, cout, n)
    bias, res = (bias if with_bias else None), (res if with_res else None)
    y, z = ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w), cout, bias, res, act, keep_z=keep)
    zr, yr = _reference(x, w, bias, res, act)
    assert y.dtype == torch.bfloat16 and _rel(y, yr) < 1e-2
    assert (z is not None) == keep
    if keep:
        assert _rel(z, zr) < 1e-2


def test_bad_arguments_are_refused():
    lib = hostcheck_library()
    x, w, bias, res = _case(1, 64, 32, 64)
    wf = ops.pointwise_pack(lib, w)
    with pytest.raises(ValueError):
        ops.pointwise_gemm(lib, x, wf, 64)                      # not this projection's weights
    with pytest.raises(ValueError):
        ops.pointwise_gemm(lib, x, wf, 32, bias=bias.double())
    with pytest.raises(_lib.NdcError):
        ops.pointwise_gemm(lib, x[:, :, :32].contiguous(), wf, 32)   # n = 32
    with pytest.raises(ValueError):
        ops.pointwise_pack(lib, w.t())                          # not contiguous


@pytest.mark.gpu
@pytest.mark.parametrize("B,cin,cout,n", [
    (2, 64, 256, 64 * 64 * 8), (2, 256, 64, 64 * 64 * 8), (1, 64, 64, 4096), (2, 128, 512, 32 ** 3),
    (3, 128, 128, 64 * 33), (1, 256, 256, 64 * 7), (2, 64, 32, 64),
    (2, 512, 128, 64 * 64 * 4), (1, 512, 64, 64 * 5), (1, 1024, 32, 128), (2, 320, 96, 64 * 3)])
@pytest.mark.parametrize("act,with_bias,with_res,keep", [(None, False, False, False), (None, True, True, False),
                                                          ("gelu", True, False, True), ("relu", False, False, False)])
def test_gpu_matches_float64(B, cin, cout, n, act, with_bias, with_res, keep):
    lib = _lib.get_library()
    if cin > 256 and (act or keep):
        pytest.skip("more than 256 input channels: plain product, bias and residual only")
    x, w, bias, res = _case(B, cin, cout, n, seed=1)
    bias, res = (bias if with_bias else None), (res if with_res else None)
    dev = [t.cuda() if t is not None else None for t in (x, w, bias, res)]
    assert ops.pointwise_gemm_applies(lib, dev[0], cout)
    y, z = ops.pointwise_gemm(lib, dev[0], ops.pointwise_pack(lib, dev[1]), cout, dev[2], dev[3], act, keep_z=keep)
    zr, yr = _reference(x, w, bias, res, act)
    assert _rel(y, yr) < 1e-2
    if keep:
        assert _rel(z, zr) < 1e-2
    # the same product through the transposed packing (what the input gradient uses)
    y2, _ = ops.pointwise_gemm(lib, dev[0], ops.pointwise_pack(lib, dev[1].t().contiguous(), transposed=True),
                               cout, dev[2], dev[3], act)
    assert torch.equal(y, y2)


@pytest.mark.gpu
def test_gpu_equals_the_host_build_bit_for_bit_up_to_summation_order():
    """Device (matrix instruction, float32 accumulation in its own order) against the host loops."""
    x, w, bias, res = _case(2, 64, 64, 256, seed=2)
    host, _ = ops.pointwise_gemm(hostcheck_library(), x, ops.pointwise_pack(hostcheck_library(), w), 64, bias, res)
    lib = _lib.get_library()
    dev, _ = ops.pointwise_gemm(lib, x.cuda(), ops.pointwise_pack(lib, w.cuda()), 64, bias.cuda(), res.cuda())
    assert _rel(dev, host.double()) < 8e-3


def _actgrad_reference(gy, w, z, bias, act):
    """float64: (W gy) * act'(z + bias) and its sum over batch and voxels."""
    prod = F.conv1d(gy.double(), w.bfloat16().double().unsqueeze(-1))
    u = (z.double() + bias.double().view(1, -1, 1)).requires_grad_(True)
    {"relu": torch.relu, "gelu": F.gelu}[act](u).sum().backward()
    gz = prod * u.grad
    return gz, gz.sum((0, 2))


@pytest.mark.parametrize("act", ["gelu", "relu"])
def test_activation_gradient_epilogue_on_the_host_build(act):
    lib = hostcheck_library()
    g = torch.Generator().manual_seed(4)
    B, cin, cout, n = 2, 64, 96, 128
    gy = torch.randn(B, cin, n, generator=g).bfloat16()
    w = torch.randn(cout, cin, generator=g) / 8
    z = torch.randn(B, cout, n, generator=g).bfloat16()
    bias = torch.randn(cout, generator=g)
    gz, gb = ops.pointwise_gemm_actgrad(lib, gy, ops.pointwise_pack(lib, w), cout, z, bias, act)
    rz, rb = _actgrad_reference(gy, w, z, bias, act)
    assert _rel(gz, rz) < 1e-2 and _rel(gb, rb) < 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("act", ["gelu", "relu"])
@pytest.mark.parametrize("B,cin,cout,n", [(2, 64, 256, 64 * 64 * 4), (1, 128, 128, 64 * 9), (2, 256, 64, 4096)])
def test_gpu_activation_gradient_epilogue(act, B, cin, cout, n):
    lib = _lib.get_library()
    g = torch.Generator().manual_seed(5)
    gy = torch.randn(B, cin, n, generator=g).bfloat16()
    w = torch.randn(cout, cin, generator=g) / cin ** 0.5
    z = torch.randn(B, cout, n, generator=g).bfloat16()
    bias = torch.randn(cout, generator=g)
    gz, gb = ops.pointwise_gemm_actgrad(lib, gy.cuda(), ops.pointwise_pack(lib, w.cuda()), cout, z.cuda(),
                                        bias.cuda(), act)
    rz, rb = _actgrad_reference(gy, w, z, bias, act)
    assert _rel(gz, rz) < 1e-2
    assert gb.dtype == torch.float32 and _rel(gb, rb) < 2e-3
    gz2, none = ops.pointwise_gemm_actgrad(lib, gy.cuda(), ops.pointwise_pack(lib, w.cuda()), cout, z.cuda(),
                                           bias.cuda(), act, need_bias_grad=False)
    assert none is None and torch.equal(gz, gz2)


@pytest.mark.gpu
@pytest.mark.parametrize("with_residual", [False, True])
def test_mlp_as_one_node_matches_float64(with_residual):
    """The 64 -> 256 -> 64 MLP of the network's first level under bf16 autocast: forward, input,
    residual and parameter gradients against the same module in float64 on the CPU."""
    import copy
    from deconver_amd.layers import MLP, _FusedMLP
    torch.manual_seed(6)
    mlp = MLP(64)
    ref = copy.deepcopy(mlp).double()
    mlp = mlp.cuda()
    x0, r0 = torch.randn(2, 64, 8, 8, 64), torch.randn(2, 64, 8, 8, 64)
    g0 = torch.randn(2, 64, 8, 8, 64)
    x = x0.cuda().bfloat16().requires_grad_(True)
    r = r0.cuda().bfloat16().requires_grad_(True) if with_residual else None
    assert _FusedMLP.applies(_lib.get_library(), x.flatten(2), 256, 64)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = mlp(x, residual=r)
    assert y.dtype == torch.bfloat16
    assert "_FusedMLP" in type(y.grad_fn.next_functions[0][0]).__name__   # (under the final view)
    y.backward(g0.cuda().bfloat16())
    xr = x.detach().double().cpu().requires_grad_(True)
    rr = r.detach().double().cpu().requires_grad_(True) if with_residual else None
    yr = ref(xr, residual=rr)
    yr.backward(g0.bfloat16().double())
    assert _rel(y.detach(), yr.detach()) < 1e-2
    assert _rel(x.grad, xr.grad) < 2e-2
    if with_residual:
        assert _rel(r.grad, rr.grad) < 1e-2
    for (name, p), (_, q) in zip(mlp.named_parameters(), ref.named_parameters()):
        assert p.grad.dtype == torch.float32 and _rel(p.grad, q.grad) < 2e-2, name


def _masked_reference(x, w, bias, res, mask):
    z, y = _reference(x, w, bias, res, None)
    return torch.where(mask.double() > 0, y, torch.zeros_like(y))


@pytest.mark.parametrize("cin,cout", [(64, 96), (384, 64)])
def test_masked_form_on_the_host_build(cin, cout):
    lib = hostcheck_library()
    x, w, bias, res = _case(2, cin, cout, 128, seed=7)
    mask = torch.randn(2, cout, 128, generator=torch.Generator().manual_seed(8)).bfloat16()
    mask[0, 0, :5] = 0      # zero counts as off
    y, none = ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w), cout, bias, res, mask=mask)
    assert none is None and _rel(y, _masked_reference(x, w, bias, res, mask)) < 1e-2
    assert bool((y[mask <= 0] == 0).all())
    with pytest.raises(ValueError):
        ops.pointwise_gemm(lib, x, ops.pointwise_pack(lib, w), cout, act="relu", mask=mask)


@pytest.mark.gpu
@pytest.mark.parametrize("B,cin,cout,n,with_res", [(2, 256, 64, 64 * 64 * 4, True), (2, 512, 128, 64 * 33, True),
                                                   (1, 64, 64, 4096, False), (2, 128, 512, 64 * 9, True)])
def test_gpu_masked_form(B, cin, cout, n, with_res):
    lib = _lib.get_library()
    x, w, bias, res = _case(B, cin, cout, n, seed=9)
    res = res if with_res else None
    mask = torch.relu(torch.randn(B, cout, n, generator=torch.Generator().manual_seed(10))).bfloat16()
    dev = [t.cuda() if t is not None else None for t in (x, w, res, mask)]
    y, _ = ops.pointwise_gemm(lib, dev[0], ops.pointwise_pack(lib, dev[1]), cout, None, dev[2], mask=dev[3])
    assert _rel(y, _masked_reference(x, w, None, res, mask)) < 1e-2
    assert bool((y[dev[3] <= 0] == 0).all())
    # where the mask is on, the masked form equals the plain one bit for bit
    plain, _ = ops.pointwise_gemm(lib, dev[0], ops.pointwise_pack(lib, dev[1]), cout, None, dev[2])
    assert torch.equal(y[dev[3] > 0], plain[dev[3] > 0])


@pytest.mark.gpu
@pytest.mark.parametrize("channels,size", [(64, (8, 8, 64)), (128, (4, 8, 64))])
def test_mixer_with_the_rectifier_on_its_neighbours_matches_float64(channels, size):
    """DeconvMixer under bf16 autocast: the ReLU's forward on in_proj, its backward in the layer's
    input-gradient GEMM (no pass of its own) -- output and every gradient against the same mixer
    in float64 on the CPU, on a case a float64 screen keeps clear of the rectifiers' kinks."""
    import copy
    import deconver_amd as dc
    torch.manual_seed(11)
    mixer = dc.DeconvMixer(channels, channels, kernel_size=(3, 3, 3), ratio=4, groups=-1)
    with torch.no_grad():
        mixer.deconv.init.linear.linear.bias.add_(1.0)
    ref = copy.deepcopy(mixer).double()
    mixer = mixer.cuda()
    x0 = torch.randn(2, channels, *size)
    g0 = torch.randn(2, channels, *size)
    x = x0.cuda().bfloat16().requires_grad_(True)
    assert mixer.deconv.takes_rectified_input(x)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = mixer(x)
    y.backward(g0.cuda().bfloat16())
    xr = x.detach().double().cpu().requires_grad_(True)
    yr = ref(xr)
    yr.backward(g0.bfloat16().double())
    assert _rel(y.detach(), yr.detach()) < 2e-2
    cos = torch.nn.functional.cosine_similarity(x.grad.double().cpu().flatten(), xr.grad.flatten(), dim=0)
    assert cos > 0.999, float(cos)
    for (name, p), (_, q) in zip(mixer.named_parameters(), ref.named_parameters()):
        c = torch.nn.functional.cosine_similarity(p.grad.double().cpu().flatten(), q.grad.flatten(), dim=0)
        assert c > 0.998, (name, float(c))
