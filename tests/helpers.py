"""Shared helpers of the test-suite."""

import os

import torch

from deconver_amd import _lib, build as ndc_build

_HOST = None


def hostcheck_library() -> _lib.NdcLibrary:
    """The sequential host build of the kernels (CPU tests only), rebuilt when stale."""
    global _HOST
    if _HOST is None:
        so = os.path.join(os.path.dirname(_lib.LIB_PATH), "libndc_hostcheck.so")
        csrc = ndc_build.CSRC
        newest = max(os.path.getmtime(os.path.join(csrc, f)) for f in os.listdir(csrc))
        if not os.path.exists(so) or os.path.getmtime(so) < newest:
            ndc_build.build_hostcheck(sanitize=False)
        _HOST = _lib.NdcLibrary(so)
    return _HOST


def make_case(C, G, sc, ks, sp, B=2, seed=0, dtype=torch.float32, bias_shift=0.0,
              positive_z=False, device="cpu"):
    """Seeded inputs of one update: x >= 0, z, rectified filter h, bias, upstream gradient."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.rand(B, C, *sp, generator=gen)
    z = torch.rand(B, G * sc, *sp, generator=gen) - (0.0 if positive_z else 0.4)
    h = torch.relu(torch.rand(C, sc, *ks, generator=gen) - 0.15)
    bias = torch.rand(G * sc, generator=gen) - 0.5 + bias_shift
    gout = torch.randn(B, G * sc, *sp, generator=gen)
    x, z, gout = (t.to(dtype) for t in (x, z, gout))
    return [t.to(device) for t in (x, z, h, bias, gout)]


def host_faults(lib) -> tuple:
    """(count, first message) of LDS races / out-of-bounds / uninitialised reads the host
    execution has seen since the last query."""
    import ctypes

    buf = ctypes.create_string_buffer(256)
    fn = lib._dll.ndc_host_faults
    fn.restype = ctypes.c_longlong
    n = fn(buf, 256)
    return n, buf.value.decode()
