"""The fused LDS-tiled kernels, executed on the host build (bounds-, race- and
uninitialised-read-checked LDS), against the oracle in float64."""

import pytest
import torch

from deconver_amd import _lib, ops
from oracle import ndc_oracle as O
from tests.helpers import host_faults, hostcheck_library, make_case

# (C, sc, kernel, spatial, batch)
FUSED_GEOMS = [
    (3, 4, (3, 3, 3), (5, 9, 8), 2),      # several row bands, ragged last band
    (2, 4, (3, 3, 3), (4, 16, 16), 1),
    (2, 4, (3, 3, 3), (3, 7, 13), 2),     # odd extents, W not a multiple of anything
    (1, 4, (3, 3, 3), (1, 4, 5), 1),      # single plane
    (2, 4, (3, 3, 3), (6, 3, 70), 1),     # W > 64: two wavefronts per row
    (3, 4, (5, 5), (9, 12), 2),           # 2-D 5x5 (marches along H)
    (2, 4, (5, 5), (3, 70), 1),
    (2, 4, (3, 3), (7, 9), 2),            # 2-D 3x3
    (2, 4, (5, 5), (70, 12), 1),          # 2-D, long march: split into two segments
    (1, 4, (5, 5), (101, 6), 2),          # 2-D, three segments, ragged last one
    (1, 4, (3, 3, 3), (37, 4, 6), 1),     # 3-D, two segments
    (2, 4, (3, 3, 3), (3, 10, 256), 1),   # wide rows of a tall plane: the column-pair variant's
                                          # LDS does not fit, the plan falls back to one column
]


def _oracle(x, z, h, bias, gout, C, sc, eps, relu):
    d = [t.double() if t is not None else None for t in (x, z, h, bias, gout)]
    out, t1 = O.update_grouped(d[0], d[1], d[2], d[3], C, 1, sc, eps, relu)
    grads = O.update_backward(d[0], d[1], d[2], d[3], d[4], C, 1, sc, eps, relu)
    return out, t1, grads


def test_fused_coverage_predicate():
    lib = hostcheck_library()
    ok = _lib.make_geom(2, 8, 1, 4, (8, 8, 8), (3, 3, 3), _lib.NDC_F32, True, 1e-16)
    assert lib.fused_supported(ok)
    for bad in (
        _lib.make_geom(2, 4, 2, 4, (8, 8, 8), (3, 3, 3), 0, True, 1e-16),     # m = 2
        _lib.make_geom(2, 8, 1, 3, (8, 8, 8), (3, 3, 3), 0, True, 1e-16),     # sc = 3
        _lib.make_geom(2, 8, 1, 4, (8, 8, 8), (3, 5, 3), 0, True, 1e-16),     # anisotropic
        _lib.make_geom(2, 8, 1, 4, (8, 8, 600), (3, 3, 3), 0, True, 1e-16),   # row too wide
    ):
        assert not lib.fused_supported(bad)
        bad.path = _lib.PATH_FUSED
        assert lib.check_geometry(bad) == -2
        bad.path = _lib.PATH_AUTO
        assert lib.check_geometry(bad) == 0   # the direct kernels still cover it


def _saved_refs(x, z, h, bias, C, sc, eps, relu):
    """s/(A(t1)+eps) and (A(x)+eps)/(A(t1)+eps) from the oracle's operators, float64."""
    xd, zd, hd = x.double(), z.double(), h.double()
    s = O.rectified_source(zd, None if bias is None else bias.double(), relu)
    t1 = O.op_K(s, hd, C, 1, sc)
    den = O.op_A(t1, hd, C, 1, sc) + eps
    return s / den, (O.op_A(xd, hd, C, 1, sc) + eps) / den


@pytest.mark.parametrize("geom", FUSED_GEOMS)
@pytest.mark.parametrize("relu,with_bias", [(True, True), (False, False)])
def test_fused_forward_backward_fp32(geom, relu, with_bias):
    C, sc, ks, sp, B = geom
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=B, bias_shift=0.3, positive_z=not relu)
    if not with_bias:
        bias = None
    eps = 1e-16
    host_faults(lib)
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=C, m=1, sc=sc, eps=eps,
                                 relu_input=relu, path=_lib.PATH_FUSED)
    n, first = host_faults(lib)
    assert n == 0, f"forward LDS faults: {n} ({first})"
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, C, sc, eps, relu)
    assert O.rel_err(out, ro) < 1e-5
    assert O.rel_err(t1, rt1) < 1e-5
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=C, m=1, sc=sc,
                                         eps=eps, relu_input=relu, path=_lib.PATH_FUSED)
    n, first = host_faults(lib)
    assert n == 0, f"backward LDS faults: {n} ({first})"
    assert O.rel_err(gx, rgx) < 1e-4
    assert O.rel_err(gz, rgz) < 1e-4
    assert O.rel_err(gh, rgh) < 1e-4
    if with_bias:
        assert O.rel_err(gb, rgb) < 1e-4


def test_backward_uses_saved_predicate():
    lib = hostcheck_library()
    mk = lambda dt, ks, sp, m=1, g=8: _lib.make_geom(2, g, m, 4, sp, ks, dt, True, 1e-16)
    for g in (mk(_lib.NDC_BF16, (3, 3, 3), (8, 8, 8)), mk(_lib.NDC_F32, (3, 3, 3), (8, 8, 8)),
              mk(_lib.NDC_BF16, (5, 5), (8, 8)), mk(_lib.NDC_BF16, (3, 3, 3), (8, 8, 7))):
        assert lib.backward_uses_saved(g)               # every fused kernel family reads them
    assert not lib.backward_uses_saved(mk(_lib.NDC_F32, (3, 3, 3), (8, 8, 8), m=2, g=4))  # direct path


def test_fused_inference_needs_no_t1():
    C, sc, ks, sp = 2, 4, (3, 3, 3), (4, 6, 8)
    lib = hostcheck_library()
    x, z, h, bias, _ = make_case(C, C, sc, ks, sp, bias_shift=0.3)
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=C, m=1, sc=sc, eps=1e-16,
                                 relu_input=True, need_t1=False)
    assert t1 is None
    ref, _ = O.update_grouped(x.double(), z.double(), h.double(), bias.double(), C, 1, sc, 1e-16, True)
    assert O.rel_err(out, ref) < 1e-5


BF16_GEOMS = [
    FUSED_GEOMS[0],                       # dot2 kernels: odd plane count, ragged last band
    FUSED_GEOMS[5],                       # 2-D 5x5 (FMA kernels, bf16 storage)
    (2, 4, (3, 3, 3), (4, 16, 16), 1),    # dot2: even plane count
    (1, 4, (3, 3, 3), (1, 4, 6), 1),      # dot2: single plane
    (2, 4, (3, 3, 3), (6, 3, 70), 1),     # dot2: two wavefronts per row
    (2, 4, (3, 3, 3), (3, 7, 13), 2),     # odd width: unpaired FMA kernels
    (2, 4, (3, 3, 3), (3, 10, 256), 1),   # dot2: widest row (512 threads, > 64 KiB of LDS)
]


@pytest.fixture
def matrix_switch():
    """Sets the host build's kernel-family switch for one test and puts it back to off."""
    lib = hostcheck_library()
    yield lib.matrix_kernels
    lib.matrix_kernels(False)


def test_matrix_kernels_are_off_by_default():
    assert hostcheck_library().matrix_kernels() is False


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("geom", BF16_GEOMS)
def test_fused_bf16_storage(geom, matrix, matrix_switch):
    C, sc, ks, sp, B = geom
    lib = hostcheck_library()
    assert matrix_switch(matrix) == matrix
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=B, dtype=torch.bfloat16, bias_shift=0.3)
    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=C, m=1, sc=sc, eps=1e-16,
                                 relu_input=True, path=_lib.PATH_FUSED)
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, C, sc, 1e-16, True)
    assert out.dtype == torch.bfloat16 and O.rel_err(out, ro) < 2e-2
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=C, m=1, sc=sc,
                                         eps=1e-16, relu_input=True, path=_lib.PATH_FUSED)
    for got, ref in ((gx, rgx), (gz, rgz), (gh, rgh), (gb, rgb)):
        assert O.rel_err(got, ref) < 2e-2
    assert host_faults(lib)[0] == 0


# workgroups of four full wavefronts (the shape of the large 3-D configurations)
FULL_WG_GEOMS = [
    (1, 4, (3, 3, 3), (3, 16, 64), 1),    # 32 lanes per row, 8 strips
    (2, 4, (3, 3, 3), (2, 32, 32), 1),    # 16 lanes per row, 16 strips
    (1, 4, (3, 3, 3), (4, 9, 128), 2),    # 64 lanes per row, 4 strips, ragged band
    (1, 4, (3, 3, 3), (5, 40, 64), 1),    # several row bands
    (2, 4, (3, 3, 3), (4, 7, 16), 1),     # 8 lanes per row: bf16 matrix-instruction forward and pass 1, dot2 pass 2
    (1, 4, (3, 3, 3), (3, 5, 8), 2),      # 4 lanes per row: one block of the matrix instruction per row
]


@pytest.mark.parametrize("geom", FUSED_GEOMS[:3] + FUSED_GEOMS[5:6] + FUSED_GEOMS[7:9] + FUSED_GEOMS[10:11]
                         + FULL_WG_GEOMS)
@pytest.mark.parametrize("dtype,matrix", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("relu", [True, False])
def test_fused_saved_denominator_and_ratio(geom, dtype, matrix, relu, matrix_switch):
    """The forward's optional s/d and n/d outputs, and a backward that consumes them (bf16: on
    both kernel families)."""
    assert matrix_switch(matrix) == matrix
    C, sc, ks, sp, B = geom
    tol_f, tol_b = (1e-5, 1e-4) if dtype == torch.float32 else (2e-2, 2e-2)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=B, dtype=dtype, bias_shift=0.3,
                                    positive_z=not relu)
    kw = dict(groups=C, m=1, sc=sc, eps=1e-6, relu_input=relu, path=_lib.PATH_FUSED)
    host_faults(lib)
    out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    out0, t10 = ops.update_forward(lib, x, z, h, bias, **kw)
    assert torch.equal(out, out0) and torch.equal(t1, t10)
    r_inv, r_ratio = _saved_refs(x, z, h, bias, C, sc, 1e-6, relu)
    assert O.rel_err(saved[0], r_inv) < tol_f
    assert O.rel_err(saved[1], r_ratio) < tol_f
    _, _, refs = _oracle(x, z, h, bias, gout, C, sc, 1e-6, relu)
    got = ops.update_backward(lib, x, z, t1, h, bias, gout, saved=saved, **kw)
    for a, r in zip(got, refs):
        assert O.rel_err(a, r) < tol_b
    n, first = host_faults(lib)
    assert n == 0, f"LDS faults: {n} ({first})"
    with pytest.raises(_lib.NdcError):   # both or neither
        lib.backward(ops.make_geom_for(x, h, C, 1, sc, 1e-6, relu), x.data_ptr(), z.data_ptr(),
                     t1.data_ptr(), saved[0].data_ptr(), None, h.data_ptr(), None,
                     gout.data_ptr(), None, out.data_ptr(), None, None, None, 0, None)


@pytest.mark.parametrize("dtype,saved,matrix,sp", [
    (torch.float32, False, False, (4, 6, 8)),
    (torch.float32, True, False, (4, 6, 8)),
    (torch.bfloat16, False, False, (4, 6, 8)),
    (torch.bfloat16, True, False, (4, 6, 8)),
    (torch.bfloat16, True, True, (4, 7, 16)),    # matrix-instruction forward and pass 1
    (torch.bfloat16, True, True, (3, 5, 32)),    # ... and pass 2
])
def test_fused_partial_outputs(dtype, saved, matrix, sp, matrix_switch):
    """Null gx / gz / gh / gb outputs (what autograd passes for a leaf that needs no gradient):
    every subset that is asked for equals the full call's, on the FMA kernels, the bf16 dot2
    kernels and the bf16 matrix-instruction kernels, with and without the kept ratios."""
    assert matrix_switch(matrix) == matrix
    C, sc, ks = 2, 4, (3, 3, 3)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, dtype=dtype, bias_shift=0.3)
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, path=_lib.PATH_FUSED)
    host_faults(lib)
    res = ops.update_forward(lib, x, z, h, bias, save_ratio=saved, **kw)
    t1, sv = res[1], (res[2] if saved else None)
    full = ops.update_backward(lib, x, z, t1, h, bias, gout, saved=sv, **kw)
    for mask in ((1, 0, 0, 0), (0, 1, 0, 0), (0, 0, 1, 0), (0, 0, 0, 1), (0, 1, 0, 1), (1, 0, 1, 0)):
        part = ops.update_backward(lib, x, z, t1, h, bias, gout, need_x=bool(mask[0]),
                                   need_z=bool(mask[1]), need_h=bool(mask[2]),
                                   need_b=bool(mask[3]), saved=sv, **kw)
        for want, a, b in zip(mask, part, full):
            assert (a is None) == (not want)
            if want:
                assert torch.equal(a, b)
    n, first = host_faults(lib)
    assert n == 0, f"LDS faults: {n} ({first})"


def test_family_named_per_call(matrix_switch):
    """ndc_geom.path = FUSED_VECTOR / FUSED_MATRIX fixes the kernel family of a call whatever
    the process default says; AUTO and FUSED follow the default."""
    C, sc, ks, sp = 2, 4, (3, 3, 3), (4, 7, 16)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, dtype=torch.bfloat16, bias_shift=0.3)
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)

    def run(path):
        out, t1, sv = ops.update_forward(lib, x, z, h, bias, save_ratio=True, path=path, **kw)
        return (out, t1) + tuple(ops.update_backward(lib, x, z, t1, h, bias, gout, saved=sv, path=path, **kw))

    assert matrix_switch(False) is False
    vec = run(_lib.PATH_FUSED)
    assert matrix_switch(True) is True
    mat = run(_lib.PATH_FUSED)
    assert not torch.equal(vec[4], mat[4])   # gh: float32 sums in another order
    for default in (False, True):
        matrix_switch(default)
        for path, want in ((_lib.PATH_FUSED_VECTOR, vec), (_lib.PATH_FUSED_MATRIX, mat),
                           (_lib.PATH_AUTO, mat if default else vec)):
            for a, b in zip(run(path), want):
                assert torch.equal(a, b)
    g = ops.make_geom_for(x, h, C, 1, sc, 1e-16, True, 5)
    assert lib.check_geometry(g) != 0        # no such path value


# rows as wide as the large 3-D configurations use (128^3, 192^3 and the widest the 3-D
# kernels accept, 256 columns): the launch planner picks other strip counts and LDS pitches there
WIDE_GEOMS = [
    (1, 4, (3, 3, 3), (3, 10, 128), 1),
    (1, 4, (3, 3, 3), (2, 9, 192), 1),
    (1, 4, (3, 3, 3), (2, 6, 256), 2),
    (1, 4, (3, 3, 3), (2, 5, 250), 1),
]


@pytest.mark.parametrize("geom", WIDE_GEOMS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fused_wide_rows(geom, dtype):
    """Wide rows through the bounds/race checker: the inference form of the forward (no t1,
    nothing kept), the training form with the kept ratio, and both backward forms."""
    C, sc, ks, sp, B = geom
    tol_f, tol_b = (1e-5, 1e-4) if dtype == torch.float32 else (2e-2, 2e-2)
    lib = hostcheck_library()
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=B, dtype=dtype, bias_shift=0.3)
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, path=_lib.PATH_FUSED)
    host_faults(lib)
    out_inf, none = ops.update_forward(lib, x, z, h, bias, need_t1=False, **kw)
    assert none is None
    out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    assert torch.equal(out, out_inf)
    ro, rt1, refs = _oracle(x, z, h, bias, gout, C, sc, 1e-16, True)
    assert O.rel_err(out, ro) < tol_f and O.rel_err(t1, rt1) < tol_f
    for sv in (saved, None):
        got = ops.update_backward(lib, x, z, t1, h, bias, gout, saved=sv, **kw)
        for a, r in zip(got, refs):
            assert O.rel_err(a, r) < tol_b
    n, first = host_faults(lib)
    assert n == 0, f"LDS faults: {n} ({first})"


@pytest.mark.parametrize("dtype,path,relu,matrix", [
    (torch.float32, _lib.PATH_FUSED, True, False), (torch.float32, _lib.PATH_FUSED, False, False),
    (torch.bfloat16, _lib.PATH_FUSED, True, False), (torch.bfloat16, _lib.PATH_FUSED, False, False),
    (torch.bfloat16, _lib.PATH_FUSED, True, True), (torch.bfloat16, _lib.PATH_FUSED, False, True),
    (torch.float32, _lib.PATH_DIRECT, True, False), (torch.float32, _lib.PATH_DIRECT, False, False),
])
def test_nan_in_source_propagates_like_torch(dtype, path, relu, matrix, matrix_switch):
    """A NaN in z is handed on where the reference's PyTorch arithmetic hands it on
    (torch.relu and a plain load both propagate it; reference.py:113-118,169-173): the set of
    non-finite entries of out, t1 and of every gradient equals the oracle's.  The bf16 dot2
    kernels multiply the column neighbour of a stencil's edge by a zero tap (half-empty
    column pairs), so there a non-finite value may also reach the entries one column further:
    every entry the oracle marks is marked, and nothing beyond that one column.  The
    matrix-instruction forward multiplies a fourth window column by a zero tap: two columns."""
    C, sc, ks, sp = 2, 4, (3, 3, 3), (4, 16, 16)
    lib = hostcheck_library()
    assert matrix_switch(matrix) == matrix
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=1, dtype=dtype, bias_shift=0.3,
                                    positive_z=not relu)
    if not relu:
        bias = None
    z[0, 5, 2, 7, 9] = float("nan")
    z[0, 2, 0, 0, 0] = float("-inf") if relu else float("nan")
    wide = dtype == torch.bfloat16

    def same_set(got, ref):
        bad_got, bad_ref = ~torch.isfinite(got), ~torch.isfinite(ref)
        if not wide or got.dim() != 5 or got.shape[-1] != sp[-1]:
            return torch.equal(bad_got, bad_ref)
        grown = bad_ref.clone()
        for _ in range(2 if matrix else 1):
            wider = grown.clone()
            wider[..., 1:] |= grown[..., :-1]
            wider[..., :-1] |= grown[..., 1:]
            grown = wider
        return bool((bad_got >= bad_ref).all() and (bad_got <= grown).all())

    out, t1 = ops.update_forward(lib, x, z, h, bias, groups=C, m=1, sc=sc, eps=1e-16,
                                 relu_input=relu, path=path)
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, C, sc, 1e-16, relu)
    assert same_set(out, ro)
    assert torch.equal(torch.isfinite(t1), torch.isfinite(rt1))
    assert not torch.isfinite(ro).all() and torch.isfinite(ro).any()
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout, groups=C, m=1, sc=sc,
                                         eps=1e-16, relu_input=relu, path=path)
    for got, ref in ((gx, rgx), (gz, rgz), (gh, rgh)):
        assert same_set(got, ref)
    fin = torch.isfinite(ro) & torch.isfinite(out)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    assert ((out.double() - ro)[fin].abs().max() / ro[fin].abs().max()) < tol


@pytest.mark.parametrize("dtype,matrix", [(torch.bfloat16, False), (torch.bfloat16, True), (torch.float32, False)])
def test_prepared_taps_give_the_same_results(dtype, matrix, matrix_switch):
    """ndc_prepare_taps + ndc_forward_taps / ndc_backward_taps against the entry points that
    pack the table themselves: bit-equal.  float32 geometries have no table (0 bytes)."""
    C, sc, ks, sp = 3, 4, (3, 3, 3), (5, 9, 8)
    lib = hostcheck_library()
    matrix_switch(matrix)
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=2, dtype=dtype, bias_shift=0.3)
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True)
    taps = ops.prepare_taps(lib, x, h, groups=C, m=1, sc=sc)
    assert (taps is not None) == (dtype == torch.bfloat16)
    out0, t0, saved0 = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    if taps is None:
        return
    assert taps.numel() == lib.taps_bytes(ops.make_geom_for(x, h, C, 1, sc, 0.0, True)) >= C * 1272
    out1, t1, saved1 = ops.update_forward(lib, x, z, h, bias, save_ratio=True, taps=taps, **kw)
    assert torch.equal(out0, out1) and torch.equal(t0, t1)
    assert torch.equal(saved0[0], saved1[0]) and torch.equal(saved0[1], saved1[1])
    g0 = ops.update_backward(lib, x, z, t0, h, bias, gout, saved=saved0, **kw)
    g1 = ops.update_backward(lib, x, z, t0, h, bias, gout, saved=saved0, taps=taps, **kw)
    for a, b in zip(g0, g1):
        assert torch.equal(a, b)
    assert host_faults(lib)[0] == 0
