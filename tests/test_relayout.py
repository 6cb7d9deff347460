"""ndc_relayout, the channels-last entry: the copy between torch.channels_last(_3d) tensors and
the channel-first layout the update kernels read.  Bit-exact against torch's own copy (it is a
permutation of elements); on the CPU through the host build, on the GPU through the HIP
library, and through the autograd node (channels-last operands in, results out in the layout
of the tensor they belong to)."""

import pytest
import torch

import deconver_amd as dc
from deconver_amd import _lib, ops
from tests.helpers import hostcheck_library, make_case

SHAPES = [   # (B, C, *S): even and odd extents, one and several tiles, 2-D and 3-D
    (2, 8, 4, 6, 10), (1, 3, 5, 7), (3, 70, 9, 13), (2, 128, 4, 8, 16), (1, 5, 3, 3, 3), (2, 64, 66, 2),
]


def _cl(t):
    return t.contiguous(memory_format=torch.channels_last if t.dim() == 4 else torch.channels_last_3d)


def _roundtrip(lib, shape, dtype, device):
    gen = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=gen).to(dtype).to(device)
    x_cl = _cl(x)
    assert ops.is_channels_last(x_cl) or x_cl.is_contiguous()
    got = ops.to_channel_first(lib, x_cl)
    assert got.is_contiguous() and torch.equal(got, x)
    back = ops.to_channels_last(lib, x)
    assert back.stride() == x_cl.stride() and torch.equal(back, x)
    # the storage itself is the permuted tensor
    perm = (0, *range(2, x.dim()), 1)
    assert torch.equal(back.permute(perm).contiguous().view(-1), x.permute(perm).contiguous().view(-1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_relayout_on_the_host_build(shape, dtype):
    _roundtrip(hostcheck_library(), shape, dtype, "cpu")


def test_relayout_rejects_bad_arguments():
    lib = hostcheck_library()
    x = torch.zeros(2, 4, 3, 3)
    with pytest.raises(_lib.NdcError):
        lib.relayout(x.data_ptr(), x.data_ptr(), 2, 4, 9, _lib.NDC_F32, False, None)   # in place
    with pytest.raises(_lib.NdcError):
        lib.relayout(x.data_ptr(), None, 2, 4, 9, _lib.NDC_F32, False, None)
    y = torch.zeros_like(x)
    with pytest.raises(_lib.NdcError):
        lib.relayout(x.data_ptr(), y.data_ptr(), 2, 4, 9, 7, False, None)               # dtype tag


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES + [(2, 32, 24, 40, 64), (1, 130, 31, 33)])
def test_relayout_on_the_gpu(shape, dtype):
    _roundtrip(_lib.get_library(), shape, dtype, "cuda")


@pytest.mark.gpu
def test_relayout_unaligned_bf16_views_on_the_gpu():
    """A bf16 tensor that starts at an odd element (2-byte aligned only) takes the one-element
    path and still comes out right."""
    lib = _lib.get_library()
    base = torch.randn(2 * 6 * 8 * 10 + 1, device="cuda").bfloat16()
    x_cl_storage = base[1:]                                   # (B, S, C) data, misaligned for pairs
    x = x_cl_storage.view(2, 80, 6).permute(0, 2, 1).reshape(2, 6, 8, 10)   # channel-first values
    out = torch.empty(2, 6, 80, device="cuda", dtype=torch.bfloat16)
    lib.relayout(x_cl_storage.data_ptr(), out.data_ptr(), 2, 6, 80, _lib.NDC_BF16, False,
                 torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(out.view(2, 6, 8, 10), x)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,ks,sp", [(torch.bfloat16, (3, 3, 3), (8, 10, 16)), (torch.float32, (5, 5), (24, 40))])
def test_update_node_takes_channels_last_operands(dtype, ks, sp):
    """deconv_update on channels-last x, z and upstream gradient: same bits as on channel-first
    tensors, and out / gx / gz come back channels-last."""
    C, sc = 16, 4
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=2, dtype=dtype, bias_shift=0.3, device="cuda")
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)

    def run(cl):
        leaves = [t.clone() for t in (x, z, h, bias)]
        if cl:
            leaves[0], leaves[1] = _cl(leaves[0]), _cl(leaves[1])
        leaves = [t.requires_grad_(True) for t in leaves]
        out = dc.deconv_update(*leaves, **kw)
        out.backward(_cl(gout) if cl else gout)
        return out.detach(), [t.grad for t in leaves]

    out_cf, grads_cf = run(False)
    out_cl, grads_cl = run(True)
    assert ops.is_channels_last(out_cl) and ops.is_channels_last(grads_cl[0]) and ops.is_channels_last(grads_cl[1])
    assert out_cf.is_contiguous() and grads_cf[0].is_contiguous()
    assert torch.equal(out_cl, out_cf)
    for a, b in zip(grads_cl, grads_cf):
        assert torch.equal(a, b)
