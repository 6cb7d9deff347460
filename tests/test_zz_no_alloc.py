"""ndc_forward_noalloc: the forward entry point that takes no workspace and allocates nothing
(its scratch is a device array inside the library), against ndc_forward on the same inputs.

Both run the same kernels, so the results must be bit-equal (well inside the 2e-2 / 1e-4
parity bars).  Two calls in a row, the second on a smaller input, show that nothing left in
the shared array by one call leaks into the next."""

import pytest
import torch

from deconver_amd import _lib, ops
from tests.helpers import make_case

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 1 << 20


def _both(lib, C, sp, B, dtype, keep):
    x, z, h, bias, _ = make_case(C, C, 4, (3, 3, 3), sp, B=B, dtype=dtype, bias_shift=0.3,
                                 seed=C, device="cuda")
    kw = dict(groups=C, m=1, sc=4, eps=1e-16, relu_input=True)
    ref = ops.update_forward(lib, x, z, h, bias, save_ratio=keep, **kw)
    ref = [ref[0], ref[1]] + (list(ref[2]) if keep else [])
    g = ops.make_geom_for(x, h, C, 1, 4, 1e-16, True)
    got = [torch.empty_like(z), torch.empty_like(x)] + ([torch.empty_like(z), torch.empty_like(z)] if keep else [])
    for t in got:
        t.fill_(float("nan"))
    ptrs = [t.data_ptr() for t in got] + [None] * (4 - len(got))
    lib.forward_noalloc(g, x.data_ptr(), z.data_ptr(), h.data_ptr(), bias.data_ptr(), *ptrs,
                        torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return g, ref, got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_noalloc_forward_matches_forward_twice_in_a_row(dtype):
    lib = _lib.get_library()
    # first a larger problem, then a smaller one that leaves most of the array's earlier
    # contents in place
    for C, sp, B, keep in ((48, (10, 12, 16), 2, True), (6, (5, 6, 8), 1, False)):
        g, ref, got = _both(lib, C, sp, B, dtype, keep)
        if dtype == torch.bfloat16:
            assert lib.forward_workspace_bytes(g) > 0, "this geometry must use the scratch array"
        for name, a, b in zip(("out", "t1", "s_over_den", "ratio"), got, ref):
            assert torch.equal(a, b), f"{name} differs (C={C})"


def test_noalloc_forward_refuses_what_does_not_fit():
    lib = _lib.get_library()
    C = 2304   # 2304 channels x 1272 bytes of packed taps > 1 MiB
    g = _lib.make_geom(1, C, 1, 4, (2, 2, 2), (3, 3, 3), _lib.NDC_BF16, True, 1e-16)
    assert lib.forward_workspace_bytes(g) > SCRATCH_BYTES
    x = torch.zeros(1, C, 2, 2, 2, dtype=torch.bfloat16, device="cuda")
    z = torch.zeros(1, 4 * C, 2, 2, 2, dtype=torch.bfloat16, device="cuda")
    h = torch.ones(C, 4, 3, 3, 3, device="cuda")
    out = torch.full_like(z, 7.0)
    with pytest.raises(_lib.NdcError, match="scratch"):
        lib.forward_noalloc(g, x.data_ptr(), z.data_ptr(), h.data_ptr(), None, out.data_ptr(),
                            None, None, None, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all()), "a refused call must not launch anything"


def test_noalloc_forward_allocates_nothing_and_replays_in_a_graph():
    """After ndc_noalloc_init the entry point only launches kernels: device memory in use
    (the driver's count and torch's) is the same before and after a call, and a call captured
    in a HIP graph replays to the eager result, several times, with eager work and
    synchronisations between the replays."""
    lib = _lib.get_library()
    lib.noalloc_init()
    C, sp, B = 24, (8, 10, 16), 2
    x, z, h, bias, _ = make_case(C, C, 4, (3, 3, 3), sp, B=B, dtype=torch.bfloat16, bias_shift=0.3,
                                 seed=3, device="cuda")
    kw = dict(groups=C, m=1, sc=4, eps=1e-16, relu_input=True)
    ref = ops.update_forward(lib, x, z, h, bias, save_ratio=True, **kw)
    ref = [ref[0], ref[1], *ref[2]]
    g = ops.make_geom_for(x, h, C, 1, 4, 1e-16, True)
    assert lib.forward_workspace_bytes(g) > 0
    got = [torch.empty_like(z), torch.empty_like(x), torch.empty_like(z), torch.empty_like(z)]
    args = (g, x.data_ptr(), z.data_ptr(), h.data_ptr(), bias.data_ptr(), *[t.data_ptr() for t in got])

    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    used0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    lib.forward_noalloc(*args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (used0, reserved0)
    assert free1 == free0, "the call changed the device memory in use"
    for a, b in zip(got, ref):
        assert torch.equal(a, b)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):   # (captures on a side stream, which is then the current one)
        lib.forward_noalloc(*args, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        for t in got:
            t.fill_(float("nan"))            # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "t1", "s_over_den", "ratio"), got, ref):
            assert torch.equal(a, b), f"{name} differs on replay {rep}"
