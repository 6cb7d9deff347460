"""The HIP library loads and exports every entry point the public header declares; the
host-only entry points (no kernel launch) behave.  No GPU needed."""

import ctypes
import os
import re

import pytest

from deconver_amd import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include",
                      "deconver_ndc.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ndc_[a-z_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(_lib.EXPORTS)


@pytest.mark.skipif(not _lib.library_available(), reason="libdeconver_ndc.so has not been built")
def test_hip_library_exports_every_declared_symbol():
    dll = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(dll, name), name


@pytest.mark.skipif(not _lib.library_available(), reason="libdeconver_ndc.so has not been built")
def test_host_only_entry_points():
    lib = _lib.get_library()
    assert lib.version() >= 100
    g = _lib.make_geom(2, 128, 1, 4, (64, 64, 64), (3, 3, 3), _lib.NDC_BF16, True, 1e-16)
    assert lib.check_geometry(g) == 0 and lib.fused_supported(g)
    assert lib.backward_workspace_bytes(g, 1, 1, 1, 1) > 2 * 128 * 64 ** 3 * 2
    g2 = _lib.make_geom(2, 4, 3, 5, (7, 6, 5), (3, 5, 3), _lib.NDC_F32, True, 1e-16)
    assert lib.check_geometry(g2) == 0 and not lib.fused_supported(g2)
    assert lib._dll.ndc_status_string(-4).decode().startswith("workspace")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_library", None)
    with pytest.raises(_lib.NdcError, match="no CPU or PyTorch fallback"):
        _lib.get_library()


def test_header_is_plain_c():
    """The boundary is a C ABI: the header must compile as C99 and as C++ on its own."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no C compiler here")
    for args in (["gcc", "-std=c99", "-x", "c"], ["g++", "-std=c++11", "-x", "c++"]):
        if not shutil.which(args[0]):
            continue
        proc = subprocess.run(args + ["-fsyntax-only", "-Wall", "-Werror", HEADER], capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr
