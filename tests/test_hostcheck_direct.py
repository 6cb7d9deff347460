"""The direct kernels, executed on the host build, against the oracle (float64)."""

import pytest
import torch

from deconver_amd import _lib, ops
from oracle import ndc_oracle as O
from tests.helpers import hostcheck_library, make_case

GEOMS = [
    # (C, groups, sc, kernel, spatial)
    (6, 3, 2, (3, 3, 3), (5, 4, 3)),
    (8, 8, 4, (3, 3, 3), (6, 5, 7)),
    (4, 1, 3, (3, 3, 3), (3, 4, 3)),
    (4, 4, 4, (5, 5), (9, 8)),
    (6, 2, 2, (3, 5, 3), (4, 6, 3)),
    (8, 8, 2, (5,), (11,)),
    (10, 5, 3, (3, 3), (9, 8)),
]


def _oracle(x, z, h, bias, gout, G, m, sc, eps, relu):
    d = [t.double() if t is not None else None for t in (x, z, h, bias, gout)]
    out, t1 = O.update_grouped(d[0], d[1], d[2], d[3], G, m, sc, eps, relu)
    grads = O.update_backward(d[0], d[1], d[2], d[3], d[4], G, m, sc, eps, relu)
    return out, t1, grads


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("relu,with_bias", [(True, True), (True, False), (False, False)])
def test_direct_update_fp32(geom, relu, with_bias):
    C, G, sc, ks, sp = geom
    m = C // G
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, bias_shift=0.3, positive_z=not relu)
    if not with_bias:
        bias = None
    eps = 1e-16
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=G, m=m, sc=sc, eps=eps,
                                 relu_input=relu, path=_lib.PATH_DIRECT)
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, G, m, sc, eps, relu)
    assert O.rel_err(out, ro) < 1e-5
    assert O.rel_err(t1, rt1) < 1e-5
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=G, m=m, sc=sc,
                                         eps=eps, relu_input=relu, path=_lib.PATH_DIRECT)
    assert O.rel_err(gx, rgx) < 1e-4
    assert O.rel_err(gz, rgz) < 1e-4
    assert O.rel_err(gh, rgh) < 1e-4
    if with_bias:
        assert O.rel_err(gb, rgb) < 1e-4
    else:
        assert gb is None


def test_direct_update_bf16_storage():
    C, G, sc, ks, sp = 8, 8, 4, (3, 3, 3), (6, 5, 7)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, dtype=torch.bfloat16, bias_shift=0.3)
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=G, m=1, sc=sc, eps=1e-16,
                                 relu_input=True, path=_lib.PATH_DIRECT)
    assert out.dtype == torch.bfloat16
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, G, 1, sc, 1e-16, True)
    assert O.rel_err(out, ro) < 2e-2
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=G, m=1, sc=sc,
                                         eps=1e-16, relu_input=True, path=_lib.PATH_DIRECT)
    for got, ref in ((gx, rgx), (gz, rgz), (gh, rgh), (gb, rgb)):
        assert O.rel_err(got, ref) < 2e-2


def test_partial_outputs_and_gconv():
    C, G, sc, ks, sp = 6, 3, 2, (3, 3, 3), (5, 4, 3)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, bias_shift=0.3)
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=G, m=2, sc=sc, eps=1e-16,
                                 relu_input=True, path=_lib.PATH_DIRECT)
    full = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=G, m=2, sc=sc, eps=1e-16,
                               relu_input=True, path=_lib.PATH_DIRECT)
    for mask in ((1, 0, 0, 0), (0, 1, 0, 0), (0, 0, 1, 0), (0, 0, 0, 1), (1, 0, 1, 0)):
        part = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=G, m=2, sc=sc,
                                   eps=1e-16, relu_input=True, need_x=bool(mask[0]),
                                   need_z=bool(mask[1]), need_h=bool(mask[2]),
                                   need_b=bool(mask[3]), path=_lib.PATH_DIRECT)
        for want, a, b in zip(mask, part, full):
            if want:
                assert torch.equal(a, b)
            else:
                assert a is None
    k = ops.gconv(lib, z, h, groups=G, m=2, sc=sc, adjoint=False)
    a = ops.gconv(lib, x, h, groups=G, m=2, sc=sc, adjoint=True)
    assert O.rel_err(k, O.op_K(z.double(), h.double(), G, 2, sc)) < 1e-5
    assert O.rel_err(a, O.op_A(x.double(), h.double(), G, 2, sc)) < 1e-5


def test_c_abi_error_codes():
    lib = hostcheck_library()
    g = _lib.make_geom(1, 2, 1, 2, (4, 4), (3, 3), _lib.NDC_F32, True, 1e-16)
    assert lib.check_geometry(g) == 0
    g.kernel[2] = 4  # even kernel
    assert lib.check_geometry(g) == -2
    g.kernel[2] = 3
    g.dtype = 7
    assert lib.check_geometry(g) == -3
    g.dtype = 0
    with pytest.raises(_lib.NdcError):
        lib.forward(g, None, None, None, None, None, None, None, None, None, 0, None)
    with pytest.raises(ValueError):
        _lib.make_geom(1, 1, 1, 1, (2, 2, 2, 2), (3, 3, 3, 3), 0, True, 0.0)
