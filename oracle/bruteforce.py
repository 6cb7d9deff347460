"""ctypes access to the brute-force float64 C restatement (oracle/ndc_bruteforce.c).

TEST INFRASTRUCTURE ONLY.  ``build()`` compiles it with gcc into ``oracle/_build``.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libndc_bruteforce.so")
_lib = None


class _Geom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("B", "G", "m", "sc", "D", "H", "W", "kD", "kH", "kW")]


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "ndc_bruteforce.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _geom(x_shape, sc, groups, ks):
    b, c = x_shape[:2]
    sp = [1] * (3 - len(ks)) + list(x_shape[2:])
    k3 = [1] * (3 - len(ks)) + list(ks)
    return _Geom(b, groups, c // groups, sc, *sp, *k3)


def _p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double)) if a is not None else None


def _c(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float64)


def K(u, h, groups, m, sc):
    u, h = _c(u), _c(h)
    ks = h.shape[2:]
    xs = (u.shape[0], groups * m) + u.shape[2:]
    g = _geom(xs, sc, groups, ks)
    out = np.empty(xs, dtype=np.float64)
    _load().ndc_bf_K(ctypes.byref(g), _p(u), _p(h), _p(out))
    return out


def A(v, h, groups, m, sc):
    v, h = _c(v), _c(h)
    ks = h.shape[2:]
    g = _geom(v.shape, sc, groups, ks)
    out = np.empty((v.shape[0], groups * sc) + v.shape[2:], dtype=np.float64)
    _load().ndc_bf_A(ctypes.byref(g), _p(v), _p(h), _p(out))
    return out


def update(x, z, h, bias, groups, m, sc, eps, relu_input):
    x, z, h, bias = _c(x), _c(z), _c(h), _c(bias)
    g = _geom(x.shape, sc, groups, h.shape[2:])
    out = np.empty_like(z)
    t1 = np.empty_like(x)
    _load().ndc_bf_update(ctypes.byref(g), _p(x), _p(z), _p(h), _p(bias),
                          ctypes.c_double(eps), int(relu_input), _p(out), _p(t1))
    return out, t1


def backward(x, z, h, bias, gout, groups, m, sc, eps, relu_input):
    x, z, h, bias, gout = _c(x), _c(z), _c(h), _c(bias), _c(gout)
    g = _geom(x.shape, sc, groups, h.shape[2:])
    gx, gz, gh = np.empty_like(x), np.empty_like(z), np.empty_like(h)
    gb = np.empty(groups * sc, dtype=np.float64)
    _load().ndc_bf_backward(ctypes.byref(g), _p(x), _p(z), _p(h), _p(bias), _p(gout),
                            ctypes.c_double(eps), int(relu_input), _p(gx), _p(gz), _p(gh), _p(gb))
    return gx, gz, gh, gb
