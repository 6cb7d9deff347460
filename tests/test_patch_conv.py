"""The resampling convolutions as regrouping + 1x1 projection (layers.patch_conv,
layers.patch_conv_transpose) against torch's convolutions: same values, same gradients, same
parameters.  The reference uses ``nn.ConvNd(kernel_size=2, stride=2)`` and
``nn.ConvTransposeNd(kernel_size=2, stride=2)`` (unet.py:36-60, 108-131) and a 1-tap head."""

import pytest
import torch
import torch.nn.functional as F
from torch import nn

import deconver_amd as dc
from deconver_amd import _lib, layers, ops
from tests.helpers import hostcheck_library


@pytest.mark.parametrize("k,size", [((2, 2), (6, 8)), ((2, 2, 2), (4, 6, 8)), ((2, 2, 2), (5, 6, 7)),
                                     ((1, 1, 1), (3, 4, 5)), ((2, 3), (4, 9)), ((4, 4), (8, 12))])
def test_patch_conv_is_the_strided_convolution(k, size):
    torch.manual_seed(0)
    nd = len(k)
    conv = getattr(F, f"conv{nd}d")
    x = torch.randn(2, 3, *size, dtype=torch.float64, requires_grad=True)
    w = torch.randn(5, 3, *k, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, dtype=torch.float64, requires_grad=True)
    ref = conv(x, w, b, stride=k)
    got = layers.patch_conv(x, w, b)
    assert got.shape == ref.shape
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)
    g = torch.randn_like(ref)
    for a, r in zip(torch.autograd.grad(got, (x, w, b), g), torch.autograd.grad(ref, (x, w, b), g)):
        torch.testing.assert_close(a, r, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(layers.patch_conv(x, w, None), conv(x, w, None, stride=k), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("k,size", [((2, 2), (3, 4)), ((2, 2, 2), (2, 3, 4)), ((1, 1), (3, 4)), ((3, 2), (2, 5))])
def test_patch_conv_transpose_is_the_transposed_convolution(k, size):
    torch.manual_seed(1)
    nd = len(k)
    tconv = getattr(F, f"conv_transpose{nd}d")
    x = torch.randn(2, 4, *size, dtype=torch.float64, requires_grad=True)
    w = torch.randn(4, 3, *k, dtype=torch.float64, requires_grad=True)
    b = torch.randn(3, dtype=torch.float64, requires_grad=True)
    ref = tconv(x, w, b, stride=k)
    got = layers.patch_conv_transpose(x, w, b)
    assert got.shape == ref.shape
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)
    g = torch.randn_like(ref)
    for a, r in zip(torch.autograd.grad(got, (x, w, b), g), torch.autograd.grad(ref, (x, w, b), g)):
        torch.testing.assert_close(a, r, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(layers.patch_conv_transpose(x, w, None), tconv(x, w, None, stride=k),
                               rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("k,size", [((3, 3), (5, 7)), ((3, 3, 3), (4, 5, 6)), ((1, 3, 5), (3, 4, 7))])
def test_unfold_conv_is_the_same_padded_convolution(k, size):
    torch.manual_seed(6)
    nd = len(k)
    conv = getattr(F, f"conv{nd}d")
    x = torch.randn(2, 2, *size, dtype=torch.float64, requires_grad=True)
    w = torch.randn(5, 2, *k, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, dtype=torch.float64, requires_grad=True)
    ref = conv(x, w, b, padding=tuple(v // 2 for v in k))
    got = layers.unfold_conv(x, w, b)
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)
    g = torch.randn_like(ref)
    for a, r in zip(torch.autograd.grad(got, (x, w, b), g), torch.autograd.grad(ref, (x, w, b), g)):
        torch.testing.assert_close(a, r, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(layers.unfold_conv(x, w, None), conv(x, w, None, padding=tuple(v // 2 for v in k)),
                               rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape", [(2, 3, 4, 8), (1, 2, 6, 16), (2, 2, 4, 6, 8), (1, 3, 2, 2, 24)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_host_regroup_is_the_strided_regrouping(shape, dtype):
    """ndc_regroup (host build) against the view / permute form, both directions, with bias."""
    lib = hostcheck_library()
    if shape[-1] % (16 // (2 if dtype == torch.bfloat16 else 4)):
        pytest.skip("row is not a whole number of 16-byte vectors")
    nd = len(shape) - 2
    x = torch.randn(*shape).to(dtype)
    assert ops.regroup2_applies(shape, dtype, x.data_ptr())
    cols = ops.windows_to_channels(lib, x)
    ref = layers.patches_to_channels(x, (2,) * nd)
    assert cols.shape == (shape[0], shape[1] * 2 ** nd, *[v // 2 for v in shape[2:]])
    assert torch.equal(cols.flatten(2), ref)
    assert torch.equal(ops.channels_to_windows(lib, cols), x)
    bias = torch.randn(shape[1])
    want = (x.float() + bias.view(1, -1, *([1] * nd))).to(dtype)
    assert torch.equal(ops.channels_to_windows(lib, cols, bias), want)


def test_regroup_refuses_what_the_kernel_does_not_take():
    lib = hostcheck_library()
    x = torch.zeros(1, 1, 3, 8)
    assert not ops.regroup2_applies((1, 1, 3, 8), torch.float32, x.data_ptr())      # odd extent
    assert not ops.regroup2_applies((1, 1, 4, 6), torch.float32, x.data_ptr())      # 6 floats: not 16-byte rows
    assert not ops.regroup2_applies((1, 1, 4, 8), torch.float64, x.data_ptr())
    assert not ops.regroup2_applies((1, 1, 4, 8), torch.float32, x.data_ptr() + 4)  # unaligned
    out = torch.zeros(1, 4, 1, 4)
    with pytest.raises(_lib.NdcError):
        lib.regroup2(x.data_ptr(), out.data_ptr(), None, 1, 1, 1, 3, 8, False, _lib.NDC_F32, True, None)
    with pytest.raises(_lib.NdcError):   # a bias only on the way back to the grid
        lib.regroup2(x.data_ptr(), out.data_ptr(), out.data_ptr(), 1, 1, 1, 2, 8, False, _lib.NDC_F32, True, None)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 3, 4, 8), (2, 5, 64, 128), (2, 4, 8, 16, 32), (1, 3, 6, 10, 24), (2, 16, 32, 32, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hip_regroup_is_the_strided_regrouping(shape, dtype):
    lib = _lib.get_library()
    if shape[-1] % (16 // (2 if dtype == torch.bfloat16 else 4)):
        pytest.skip("row is not a whole number of 16-byte vectors")
    nd = len(shape) - 2
    x = torch.randn(*shape, device="cuda").to(dtype)
    cols = ops.windows_to_channels(lib, x)
    assert torch.equal(cols.flatten(2), layers.patches_to_channels(x, (2,) * nd))
    assert torch.equal(ops.channels_to_windows(lib, cols), x)
    bias = torch.randn(shape[1], device="cuda")
    want = (x.float() + bias.view(1, -1, *([1] * nd))).to(dtype)
    assert torch.equal(ops.channels_to_windows(lib, cols, bias), want)


def test_one_dimensional_network_builds_and_runs():
    """spatial_dims = 1: the same subclasses exist for 1-D convolutions (the regrouping is then
    the strided view; the kernel takes 2-D and 3-D grids)."""
    torch.manual_seed(4)
    net = dc.Deconver(in_channels=1, out_channels=2, spatial_dims=1, encoder_depth=(1, 1), encoder_width=(4, 8),
                      strides=(1, 2), decoder_depth=(1,), kernel_size=(3,), ratio=2)
    assert isinstance(net.stem, layers.UnfoldConv1d) and isinstance(net.head, layers.PatchConv1d)
    assert isinstance(net.encoder.blocks[1].downsample, layers.PatchConv1d)
    assert isinstance(net.decoder.blocks[0].upsample, layers.PatchConvTranspose1d)
    x = torch.rand(2, 1, 16)
    y = net(x)
    assert y.shape == (2, 2, 16)
    y.sum().backward()
    k = (2,)
    w = torch.randn(5, 3, 2, dtype=torch.float64)
    xx = torch.randn(2, 3, 10, dtype=torch.float64)
    torch.testing.assert_close(layers.patch_conv(xx, w, None), F.conv1d(xx, w, None, stride=k), rtol=1e-12, atol=1e-12)


def test_regrouping_round_trip():
    x = torch.arange(2 * 3 * 4 * 6 * 8, dtype=torch.float32).view(2, 3, 4, 6, 8)
    cols = layers.patches_to_channels(x, (2, 2, 2))
    assert cols.shape == (2, 24, 2 * 3 * 4)
    assert torch.equal(layers.channels_to_patches(cols, (2, 2, 2), (2, 3, 4)), x)


def test_modules_keep_the_parent_parameters_and_route():
    """Same parameter names and shapes as the torch modules, so reference checkpoints load;
    on the CPU (and in float32) the parent's convolution runs; other strides always do."""
    torch.manual_seed(2)
    for cls, parent, args in ((layers.PatchConv3d, nn.Conv3d, (3, 5, 2)), (layers.PatchConvTranspose2d, nn.ConvTranspose2d, (3, 5, 2))):
        mod, ref = cls(*args, stride=2), parent(*args, stride=2)
        assert isinstance(mod, parent)
        assert {k: v.shape for k, v in mod.state_dict().items()} == {k: v.shape for k, v in ref.state_dict().items()}
        ref.load_state_dict(mod.state_dict())
        x = torch.randn(2, 3, *([4] * (mod.weight.dim() - 2)))
        assert torch.equal(mod(x), ref(x))
    odd = layers.PatchConv2d(3, 5, 3, stride=1, padding=1)
    assert not layers._is_patch_conv(odd)
    assert layers._is_patch_conv(layers.PatchConv2d(3, 5, 2, stride=2))
    assert layers._is_patch_conv(layers.PatchConv3d(3, 5, 1))
    assert not layers._is_patch_conv(layers.PatchConvTranspose2d(3, 5, 2, stride=2, output_padding=1))
    assert not layers._is_patch_conv(layers.PatchConv2d(4, 4, 2, stride=2, groups=2))
    x = torch.randn(1, 3, 6, 6)
    assert odd(x).shape == (1, 5, 6, 6)


def test_network_uses_them_with_the_reference_state_dict_names():
    net = dc.Deconver(in_channels=1, out_channels=2, spatial_dims=2, encoder_depth=(1, 1), encoder_width=(4, 8),
                      strides=(1, 2), decoder_depth=(1,), kernel_size=(3, 3), ratio=2)
    assert isinstance(net.encoder.blocks[1].downsample, layers.PatchConv2d)
    assert isinstance(net.decoder.blocks[0].upsample, layers.PatchConvTranspose2d)
    assert isinstance(net.head, layers.PatchConv2d)
    assert isinstance(net.stem, layers.UnfoldConv2d) and isinstance(net.stem, nn.Conv2d)
    assert tuple(net.stem.weight.shape) == (4, 1, 3, 3) and net.stem.bias is None
    keys = set(net.state_dict())
    assert {"encoder.blocks.1.downsample.weight", "encoder.blocks.1.downsample.bias",
            "decoder.blocks.0.upsample.weight", "decoder.blocks.0.upsample.bias", "head.weight", "head.bias"} <= keys


@pytest.mark.gpu
@pytest.mark.parametrize("nd", [2, 3])
@pytest.mark.parametrize("regime", ["bf16 autocast", "float32"])
def test_regrouped_route_matches_the_library_convolution_on_the_gpu(nd, regime):
    """The resampling convolutions and the stem on the GPU, in the two regimes that take the
    regrouped form -- bf16 autocast (the 3-D training step) and float32 (the 2-D network):
    values and gradients against torch's convolution of the same operands, bf16 to 2e-2 of the
    largest entry, float32 to 1e-5 (against float64)."""
    import contextlib
    torch.manual_seed(3)
    bf16 = regime == "bf16 autocast"
    tol = 2e-2 if bf16 else 1e-5
    ctx = (lambda: torch.autocast("cuda", dtype=torch.bfloat16)) if bf16 else contextlib.nullcontext
    hi = (lambda t: t) if bf16 else (lambda t: t.double())      # the reference's precision
    size = (16, 12, 24)[:nd]
    conv, tconv = getattr(F, f"conv{nd}d"), getattr(F, f"conv_transpose{nd}d")
    down = getattr(layers, f"PatchConv{nd}d")(16, 32, 2, stride=2).cuda()
    up = getattr(layers, f"PatchConvTranspose{nd}d")(32, 16, 2, stride=2).cuda()
    stem = getattr(layers, f"UnfoldConv{nd}d")(2, 16, 3, padding=1, bias=False).cuda()
    x = torch.randn(2, 16, *size, device="cuda", requires_grad=True)
    img = torch.randn(2, 2, *size, device="cuda")
    params = (x, down.weight, down.bias, up.weight, up.bias)
    with ctx():
        y = up(down(x))
        ys = stem(img)
    ref_params = [hi(p.detach()).requires_grad_(True) for p in params]
    sw = hi(stem.weight.detach()).requires_grad_(True)
    with ctx():
        rx, dw, db, uw, ub = ref_params
        ref = tconv(conv(rx, dw, db, stride=2), uw, ub, stride=2)
        rs = conv(hi(img), sw, None, padding=1)
    assert y.dtype == (torch.bfloat16 if bf16 else torch.float32) and y.shape == ref.shape
    assert ys.dtype == y.dtype and ys.shape == rs.shape
    g, gs = torch.randn_like(y), torch.randn_like(ys)
    got = (y, ys, *torch.autograd.grad(y, params, g), *torch.autograd.grad(ys, stem.weight, gs))
    want = (ref, rs, *torch.autograd.grad(ref, ref_params, hi(g)), *torch.autograd.grad(rs, sw, hi(gs)))
    for a, r in zip(got, want):
        assert a.shape == r.shape
        err = float((a.detach().double() - r.detach().double()).abs().max() / r.detach().double().abs().max())
        assert err <= tol, err


@pytest.mark.gpu
def test_full_size_regrouping_round_trip():
    """The first resampling step of the 3-D network (B 2, 64 channels, 128^3, bf16): to channels
    and back is the identity, bit for bit, and a sampled window lands where the strided view
    puts it."""
    lib = _lib.get_library()
    torch.manual_seed(13)
    x = torch.randn(2, 64, 128, 128, 128, device="cuda").bfloat16()
    cols = ops.windows_to_channels(lib, x)
    assert cols.shape == (2, 512, 64, 64, 64)
    assert torch.equal(ops.channels_to_windows(lib, cols), x)
    for (b, c, d, h, w) in ((0, 0, 0, 0, 0), (1, 63, 63, 63, 63), (1, 17, 5, 40, 9)):
        for kd in (0, 1):
            for kh in (0, 1):
                for kw in (0, 1):
                    assert cols[b, c * 8 + (kd * 2 + kh) * 2 + kw, d, h, w] == x[b, c, 2 * d + kd, 2 * h + kh, 2 * w + kw]


def test_host_regroup_on_random_grids():
    """Random even grids (hypothesis): the host build's regrouping equals the strided view in
    both directions, 2-D and 3-D, float32 and bfloat16."""
    from hypothesis import given, settings, strategies as st

    lib = hostcheck_library()

    @settings(max_examples=40, deadline=None)
    @given(st.integers(1, 2), st.integers(1, 3), st.integers(1, 3), st.integers(1, 4), st.integers(1, 3),
           st.booleans(), st.booleans())
    def check(B, C, d2, h2, w8, three_d, bf16):
        dtype = torch.bfloat16 if bf16 else torch.float32
        W = w8 * (8 if bf16 else 4)
        shape = (B, C, 2 * d2, 2 * h2, W) if three_d else (B, C, 2 * h2, W)
        x = torch.randn(*shape).to(dtype)
        nd = len(shape) - 2
        cols = ops.windows_to_channels(lib, x)
        assert torch.equal(cols.flatten(2), layers.patches_to_channels(x, (2,) * nd))
        assert torch.equal(ops.channels_to_windows(lib, cols), x)

    check()


@pytest.mark.gpu
@pytest.mark.parametrize("regime", ["bf16 autocast", "float32"])
def test_patchifying_stem_on_the_gpu(regime):
    """``Stem`` (deconver.py:106-114: a 4 x 4 patchifying convolution + norm) on the GPU: windows
    other than 2 x 2 are regrouped by a strided view; values and weight gradient against
    torch's convolution in float64."""
    import contextlib
    torch.manual_seed(9)
    bf16 = regime == "bf16 autocast"
    stem = dc.Stem(3, 16, patch_size=(4, 4)).cuda()
    conv = stem[0]
    assert isinstance(conv, layers.PatchConv2d)
    x = torch.randn(2, 3, 32, 40, device="cuda")
    with (torch.autocast("cuda", dtype=torch.bfloat16) if bf16 else contextlib.nullcontext()):
        y = conv(x)
    w64 = conv.weight.detach().double().requires_grad_(True)
    ref = F.conv2d(x.double(), w64, conv.bias.detach().double(), stride=4)
    g = torch.randn_like(y)
    (gw,) = torch.autograd.grad(y, conv.weight, g)
    (gw_ref,) = torch.autograd.grad(ref, w64, g.double())
    tol = 2e-2 if bf16 else 1e-5
    for a, r in ((y, ref), (gw, gw_ref)):
        assert a.shape == r.shape
        assert float((a.detach().double() - r.detach()).abs().max() / r.detach().abs().max()) <= tol
    assert stem(x).shape == (2, 16, 8, 10)


@pytest.mark.gpu
def test_one_dimensional_network_on_the_gpu_matches_float64():
    """A 1-D network in float32 on the GPU (1-D resampling convolutions regrouped by the strided
    view, InstanceNorm1d and projection tails on the kernels, NDC layers on the direct kernels)
    against the same network in float64 on the CPU."""
    import copy
    torch.manual_seed(5)
    net = dc.Deconver(in_channels=2, out_channels=1, spatial_dims=1, encoder_depth=(1, 1), encoder_width=(8, 16),
                      strides=(1, 2), decoder_depth=(1,), kernel_size=(5,), ratio=4, norm=nn.InstanceNorm1d)
    x = torch.rand(2, 2, 4096)
    ref = copy.deepcopy(net).double()(x.double())
    y = net.cuda()(x.cuda())
    assert float((y.cpu().double() - ref).abs().max() / ref.abs().max()) <= 1e-4
