"""Parity of the HIP kernels (through the C ABI) with the oracle, on a real MI355X.

Tolerances are north_star's: ``max|d| / max|ref|`` <= 1e-4 for float32 and <= 2e-2 for
bfloat16 storage with float32 accumulation; the oracle is evaluated in float64 on the same
(bf16-valued, where applicable) inputs.
"""

import pytest
import torch

import deconver_amd as dc
from deconver_amd import _lib, ops
from oracle import ndc_oracle as O
from tests.helpers import make_case

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}

# (C, groups, sc, kernel, spatial, batch)
DIRECT_GEOMS = [
    (12, 3, 8, (3, 3, 3), (7, 6, 5), 2),
    (8, 1, 1, (3, 3, 3), (6, 6, 6), 2),
    (16, 16, 4, (3, 3), (17, 15), 2),
    (6, 2, 6, (3, 5, 3), (6, 7, 5), 2),
    (8, 8, 2, (5,), (11,), 2),
    (10, 5, 6, (3, 3), (9, 8), 2),
]
FUSED_GEOMS = [
    (32, 32, 4, (3, 3, 3), (12, 14, 13), 2),
    (64, 64, 4, (3, 3, 3), (10, 9, 11), 2),
    (128, 128, 4, (3, 3, 3), (8, 8, 8), 2),
    (256, 256, 4, (3, 3, 3), (6, 5, 4), 2),
    (512, 512, 4, (3, 3, 3), (3, 4, 3), 2),
    (16, 16, 4, (3, 3, 3), (9, 8, 7), 3),
    (4, 4, 4, (3, 3, 3), (5, 20, 70), 1),
    (8, 8, 4, (3, 3, 3), (20, 33, 64), 1),
    (32, 32, 4, (5, 5), (64, 64), 1),
    (8, 8, 4, (5, 5), (40, 100), 2),
    (16, 16, 4, (3, 3), (17, 15), 2),
    # widest row of the bf16 dot2 kernels (512 threads, > 64 KiB of LDS); in float32 the
    # column-pair kernels' LDS does not fit and the plan falls back to the one-column ones
    (4, 4, 4, (3, 3, 3), (6, 10, 256), 1),
    # widths the bf16 matrix-instruction kernels cover (multiples of 8 that divide 128): the
    # widest, one with several rows per wavefront, one below the width from which pass 2 uses them
    (4, 4, 4, (3, 3, 3), (6, 12, 128), 1),
    (8, 8, 4, (3, 3, 3), (7, 9, 32), 2),
    (8, 8, 4, (3, 3, 3), (5, 6, 16), 2),
]


def _lib_gpu():
    return _lib.get_library()


def _oracle(x, z, h, bias, gout, G, m, sc, eps, relu):
    d = [t.detach().cpu().double() if t is not None else None for t in (x, z, h, bias, gout)]
    out, t1 = O.update_grouped(d[0], d[1], d[2], d[3], G, m, sc, eps, relu)
    grads = O.update_backward(d[0], d[1], d[2], d[3], d[4], G, m, sc, eps, relu)
    return out, t1, grads


# (storage type, matrix-instruction kernels on): the bf16 3x3x3 geometries have two kernel
# families, the default one on the vector unit and the one ndc_matrix_kernels(1) selects
FAMILIES = [pytest.param(torch.float32, False, id="f32"), pytest.param(torch.bfloat16, False, id="bf16"),
            pytest.param(torch.bfloat16, True, id="bf16-matrix")]


@pytest.fixture
def matrix_switch():
    """Sets the library's kernel-family switch for one test and puts it back to off."""
    lib = _lib.get_library()
    yield lib.matrix_kernels
    lib.matrix_kernels(False)


def _run_case(geom, dtype, path, relu=True, with_bias=True, saved=False):
    C, G, sc, ks, sp, B = geom
    m = C // G
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, B=B, dtype=dtype, bias_shift=0.3,
                                    positive_z=not relu, device="cuda")
    if not with_bias:
        bias = None
    lib = _lib_gpu()
    kw = dict(groups=G, m=m, sc=sc, eps=1e-16, relu_input=relu, path=path)
    res = ops.update_forward(lib, x, z, h, bias, save_ratio=saved, **kw)
    out, t1 = res[0], res[1]
    gx, gz, gh, gb = ops.update_backward(lib, x, z, t1, h, bias, gout,
                                         saved=res[2] if saved else None, **kw)
    torch.cuda.synchronize()
    ro, rt1, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, G, m, sc, 1e-16, relu)
    tol = TOL[dtype]
    errs = dict(out=O.rel_err(out.cpu(), ro), t1=O.rel_err(t1.cpu(), rt1),
                gx=O.rel_err(gx.cpu(), rgx), gz=O.rel_err(gz.cpu(), rgz),
                gh=O.rel_err(gh.cpu(), rgh))
    if with_bias:
        errs["gb"] = O.rel_err(gb.cpu(), rgb)
    bad = {k: v for k, v in errs.items() if not v < tol}
    assert not bad, f"{geom} {dtype} path={path} saved={saved}: {bad} (all: {errs})"
    if saved:
        # the kept tensors themselves: s/(A(t1)+eps) and (A(x)+eps)/(A(t1)+eps)
        d = [t.detach().cpu().double() for t in (x, z, h)]
        s = O.rectified_source(d[1], None if bias is None else bias.cpu().double(), relu)
        den = O.op_A(O.op_K(s, d[2], G, m, sc), d[2], G, m, sc) + 1e-16
        assert O.rel_err(res[2][0].cpu(), s / den) < tol
        assert O.rel_err(res[2][1].cpu(), (O.op_A(d[0], d[2], G, m, sc) + 1e-16) / den) < tol
    return errs


@pytest.mark.parametrize("geom", DIRECT_GEOMS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_direct_kernels(geom, dtype):
    _run_case(geom, dtype, _lib.PATH_DIRECT)


@pytest.mark.parametrize("geom", FUSED_GEOMS)
@pytest.mark.parametrize("dtype,matrix", FAMILIES)
def test_fused_kernels(geom, dtype, matrix, matrix_switch):
    print("case", geom, dtype, matrix, flush=True)
    assert matrix_switch(matrix) == matrix
    _run_case(geom, dtype, _lib.PATH_FUSED)


@pytest.mark.parametrize("geom", FUSED_GEOMS)
@pytest.mark.parametrize("dtype,matrix", FAMILIES)
def test_fused_kernels_with_saved_ratio(geom, dtype, matrix, matrix_switch):
    """Backward fed with the forward's denominator and ratio instead of re-gathering them."""
    print("case saved", geom, dtype, matrix, flush=True)
    assert matrix_switch(matrix) == matrix
    _run_case(geom, dtype, _lib.PATH_FUSED, saved=True)


@pytest.mark.parametrize("geom", DIRECT_GEOMS + FUSED_GEOMS[:2] + FUSED_GEOMS[8:9])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gconv_matches_oracle(geom, dtype):
    """ndc_gconv, the counterpart of kernels.gconv (kernels.py:728-759): K and A on their own,
    plain and with the forward's on-load bias + ReLU of the input."""
    C, G, sc, ks, sp, B = geom
    m = C // G
    x, z, h, bias, _ = make_case(C, G, sc, ks, sp, B=B, dtype=dtype, bias_shift=0.1, device="cuda")
    lib = _lib_gpu()
    tol = TOL[dtype]
    hd, zd, xd = h.cpu().double(), z.cpu().double(), x.cpu().double()
    k_plain = ops.gconv(lib, z, h, groups=G, m=m, sc=sc, adjoint=False)
    k_rect = ops.gconv(lib, z, h, groups=G, m=m, sc=sc, adjoint=False, bias=bias, relu_input=True)
    a_plain = ops.gconv(lib, x, h, groups=G, m=m, sc=sc, adjoint=True)
    torch.cuda.synchronize()
    assert k_plain.dtype == dtype and k_plain.shape == x.shape and a_plain.shape == z.shape
    assert O.rel_err(k_plain.cpu(), O.op_K(zd, hd, G, m, sc)) < tol
    s = O.rectified_source(zd, bias.cpu().double(), True)
    assert O.rel_err(k_rect.cpu(), O.op_K(s, hd, G, m, sc)) < tol
    assert O.rel_err(a_plain.cpu(), O.op_A(xd, hd, G, m, sc)) < tol


def test_saved_ratio_later_iteration_form():
    _run_case(FUSED_GEOMS[0], torch.bfloat16, _lib.PATH_FUSED, relu=False, with_bias=False,
              saved=True)
    _run_case(DIRECT_GEOMS[0], torch.float32, _lib.PATH_DIRECT, saved=True)


@pytest.mark.parametrize("relu,with_bias", [(True, False), (False, False)])
def test_fused_later_iteration_form(relu, with_bias):
    _run_case(FUSED_GEOMS[0], torch.float32, _lib.PATH_FUSED, relu=relu, with_bias=with_bias)


def test_fused_matches_direct_at_size():
    """A size the CPU oracle would take minutes for: the two HIP paths check each other."""
    C, sc, ks, sp = 16, 4, (3, 3, 3), (32, 64, 64)
    x, z, h, bias, gout = make_case(C, C, sc, ks, sp, B=1, bias_shift=0.3, device="cuda")
    lib = _lib_gpu()
    res = {}
    for path in (_lib.PATH_DIRECT, _lib.PATH_FUSED):
        kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, path=path)
        out, t1 = ops.update_forward(lib, x, z, h, bias, **kw)
        res[path] = (out, t1) + tuple(ops.update_backward(lib, x, z, t1, h, bias, gout, **kw))
    torch.cuda.synchronize()
    for name, a, b in zip(("out", "t1", "gx", "gz", "gh", "gb"), res[_lib.PATH_FUSED],
                          res[_lib.PATH_DIRECT]):
        assert O.rel_err(a, b) < 1e-4, name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_full_size_scaling_laws(dtype):
    """Config 3 at full size (batch 2, 128 channels, 64^3), where no oracle run is affordable:
    what the update's algebra fixes exactly.  Doubling x doubles A(x) exactly in binary
    floating point, so out(2x) = 2 out(x) up to the eps term; halving the filter halves K and
    A, so out(h/2) = 2 out(h); the backward is linear in gout, so doubling gout doubles every
    gradient exactly (gh and gb are summed in a fixed order)."""
    C, sc, sp = 128, 4, (64, 64, 64)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(2, C, *sp, generator=gen).abs().to(dtype).cuda()
    z = (torch.randn(2, C * sc, *sp, generator=gen) * 0.5).to(dtype).cuda()
    h = torch.nn.functional.softplus(0.1 * torch.randn(C, sc, 3, 3, 3, generator=gen)).cuda()
    bias = (0.1 * torch.randn(C * sc, generator=gen)).cuda()
    gout = torch.randn(2, C * sc, *sp, generator=gen).to(dtype).cuda()
    lib = _lib_gpu()
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, path=_lib.PATH_FUSED)

    out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    out2 = ops.update_forward(lib, x * 2, z, h, bias, **kw)[0]
    assert O.rel_err(out2.float(), out.float() * 2) < 1e-6
    outh = ops.update_forward(lib, x, z, h * 0.5, bias, **kw)[0]
    assert O.rel_err(outh.float(), out.float() * 2) < 1e-6
    del out2, outh

    g1 = ops.update_backward(lib, x, z, t1, h, bias, gout, saved=saved, **kw)
    g2 = ops.update_backward(lib, x, z, t1, h, bias, gout * 2, saved=saved, **kw)
    torch.cuda.synchronize()
    for name, a, b in zip(("gx", "gz", "gh", "gb"), g1, g2):
        assert torch.equal(b.float(), a.float() * 2), name
    # and the saved-tensor backward agrees with the re-gathering one
    g3 = ops.update_backward(lib, x, z, t1, h, bias, gout, **kw)
    tol = TOL[dtype]
    for name, a, b in zip(("gx", "gz", "gh", "gb"), g1, g3):
        assert O.rel_err(a.float(), b.float()) < tol, name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_graph_capture_replays_match_eager(dtype):
    """The library neither allocates nor synchronises, so a forward + backward pair can be
    captured in a HIP graph; every replay (with eager work and synchronisations between
    them) must reproduce the eager results bit for bit."""
    C, sc, sp = 16, 4, (12, 16, 32)
    x, z, h, bias, gout = make_case(C, C, sc, (3, 3, 3), sp, B=2, dtype=dtype, bias_shift=0.3,
                                    device="cuda")
    lib = _lib_gpu()
    kw = dict(groups=C, m=1, sc=sc, eps=1e-16, relu_input=True, path=_lib.PATH_FUSED)

    def step():
        out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
        return (out,) + tuple(ops.update_backward(lib, x, z, t1, h, bias, gout, saved=saved, **kw))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()   # warm-up off the default stream, as graph capture asks
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    gens = torch.Generator().manual_seed(7)
    for replay in range(3):
        x.copy_(torch.rand(x.shape, generator=gens).to(dtype))
        gout.copy_(torch.randn(gout.shape, generator=gens).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "gx", "gz", "gh", "gb"), got, want):
            assert torch.equal(a, b), f"replay {replay}: {name}"


@pytest.mark.parametrize("matrix", [False, True])
@pytest.mark.parametrize("geom", [FUSED_GEOMS[2], FUSED_GEOMS[7], (24, 24, 4, (3, 3, 3), (9, 16, 192), 1)])
def test_prepared_taps_bit_equal_on_gpu(geom, matrix, matrix_switch):
    """ndc_prepare_taps once, then ndc_forward_taps / ndc_backward_taps: the same bits as the
    entry points that pack the filter table on every call (bf16 3x3x3 kernels; the last case
    is a 192-column row, i.e. six wavefronts per workgroup in the forward)."""
    C, G, sc, ks, sp, B = geom
    lib = _lib_gpu()
    matrix_switch(matrix)
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, B=B, dtype=torch.bfloat16, bias_shift=0.3,
                                    device="cuda")
    kw = dict(groups=G, m=1, sc=sc, eps=1e-16, relu_input=True)
    taps = ops.prepare_taps(lib, x, h, groups=G, m=1, sc=sc)
    assert taps is not None and taps.data_ptr() % 256 == 0
    out0, t0, saved0 = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    out1, t1, saved1 = ops.update_forward(lib, x, z, h, bias, save_ratio=True, taps=taps, **kw)
    assert torch.equal(out0, out1) and torch.equal(t0, t1)
    assert torch.equal(saved0[0], saved1[0]) and torch.equal(saved0[1], saved1[1])
    g0 = ops.update_backward(lib, x, z, t0, h, bias, gout, saved=saved0, **kw)
    g1 = ops.update_backward(lib, x, z, t0, h, bias, gout, saved=saved0, taps=taps, **kw)
    for a, b in zip(g0, g1):
        assert torch.equal(a, b)
    ro, _, (rgx, rgz, rgh, rgb) = _oracle(x, z, h, bias, gout, G, 1, sc, 1e-16, True)
    assert O.rel_err(out1.float().cpu(), ro) < 2e-2
    for got, ref in zip(g1, (rgx, rgz, rgh, rgb)):
        assert O.rel_err(got.float().cpu(), ref) < 2e-2


def test_matrix_kernel_switch_defaults_to_off_and_changes_the_kernels(matrix_switch):
    """ndc_matrix_kernels: off in a fresh library; turned on, the bf16 3x3x3 update runs other
    kernels (the filter gradient's float32 sums come out in another order) that agree with the
    default ones to the bf16 tolerance."""
    lib = _lib_gpu()
    assert lib.matrix_kernels() is False
    C, G, sc, ks, sp, B = FUSED_GEOMS[7]
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, B=B, dtype=torch.bfloat16, bias_shift=0.3, device="cuda")
    kw = dict(groups=G, m=1, sc=sc, eps=1e-16, relu_input=True)

    def run():
        out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
        return (out, t1) + tuple(ops.update_backward(lib, x, z, t1, h, bias, gout, saved=saved, **kw))
    base = run()
    assert matrix_switch(True) is True
    other = run()
    assert matrix_switch(False) is False
    again = run()
    for a, b in zip(base, again):
        assert torch.equal(a, b)
    assert not torch.equal(base[4], other[4])          # gh: float32, other summation order
    for a, b in zip(base, other):
        assert O.rel_err(a.float().cpu(), b.float().cpu().double()) < 2e-2


def test_family_named_per_call_from_two_threads(matrix_switch):
    """ndc_geom.path = FUSED_VECTOR / FUSED_MATRIX names the kernel family of one call: two
    threads run the two families at the same time, each on its own stream, while the main thread
    keeps flipping the process default; every call returns the bits of the family it named
    (forward on one thread and backward on another cannot disagree)."""
    import threading

    lib = _lib_gpu()
    C, G, sc, ks, sp, B = FUSED_GEOMS[7]
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, B=B, dtype=torch.bfloat16, bias_shift=0.3, device="cuda")
    kw = dict(groups=G, m=1, sc=sc, eps=1e-16, relu_input=True)

    def run(path):
        out, t1, saved = ops.update_forward(lib, x, z, h, bias, save_ratio=True, path=path, **kw)
        return (out, t1) + tuple(ops.update_backward(lib, x, z, t1, h, bias, gout, saved=saved, path=path, **kw))

    # what each family returns, from the process-wide switch with the default path
    assert matrix_switch(False) is False
    want = {_lib.PATH_FUSED_VECTOR: run(_lib.PATH_AUTO)}
    assert matrix_switch(True) is True
    want[_lib.PATH_FUSED_MATRIX] = run(_lib.PATH_AUTO)
    matrix_switch(False)
    torch.cuda.synchronize()
    assert not torch.equal(want[_lib.PATH_FUSED_VECTOR][4], want[_lib.PATH_FUSED_MATRIX][4])

    failures, stop = [], threading.Event()

    def worker(path):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(6):
                    got = run(path)
                    stream.synchronize()
                    for a, b in zip(got, want[path]):
                        if not torch.equal(a, b):
                            failures.append(path)
        except Exception as e:   # noqa: BLE001 - reported below
            failures.append(repr(e))

    threads = [threading.Thread(target=worker, args=(p,)) for p in (_lib.PATH_FUSED_VECTOR, _lib.PATH_FUSED_MATRIX)]
    for t in threads:
        t.start()
    flips = 0
    while any(t.is_alive() for t in threads):
        matrix_switch(bool(flips & 1))
        flips += 1
        stop.wait(0.001)
    for t in threads:
        t.join()
    assert not failures, failures
    assert flips > 0


def test_autograd_node_names_its_family_once(matrix_switch):
    """The update node reads the family in its forward and names it in both calls: flipping
    the process default between forward and backward does not change the backward."""
    C, G, sc, ks, sp, B = FUSED_GEOMS[7]
    x, z, h, bias, gout = make_case(C, G, sc, ks, sp, B=B, dtype=torch.bfloat16, bias_shift=0.3, device="cuda")

    def run(flip):
        leaves = [t.clone().requires_grad_(True) for t in (x, z, h, bias)]
        matrix_switch(True)
        out = dc.deconv_update(*leaves, groups=G, m=1, sc=sc, eps=1e-16, relu_input=True)
        if flip:
            matrix_switch(False)
        out.backward(gout)
        matrix_switch(False)
        return [t.grad.clone() for t in leaves]

    for a, b in zip(run(False), run(True)):
        assert torch.equal(a, b)
