"""ctypes binding of the C ABI declared in ``include/deconver_ndc.h``.

The product library is ``libdeconver_ndc.so`` (hipcc, gfx950), built in-tree by
``deconver_amd.build``.  There is no CPU fallback: if the library is missing,
``get_library()`` raises.
"""

from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional, Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdeconver_ndc.so")

NDC_F32, NDC_BF16 = 0, 1
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
PATH_AUTO, PATH_DIRECT, PATH_FUSED, PATH_FUSED_MATRIX, PATH_FUSED_VECTOR = 0, 1, 2, 3, 4

EXPORTS = (
    "ndc_version",
    "ndc_status_string",
    "ndc_fused_supported",
    "ndc_check_geometry",
    "ndc_backward_uses_saved",
    "ndc_matrix_kernels",
    "ndc_forward",
    "ndc_forward_workspace_bytes",
    "ndc_forward_noalloc",
    "ndc_noalloc_init",
    "ndc_taps_bytes",
    "ndc_prepare_taps",
    "ndc_forward_taps",
    "ndc_backward_taps",
    "ndc_backward_workspace_bytes",
    "ndc_backward",
    "ndc_backward_profiled",
    "ndc_gconv",
    "ndc_relayout",
    "ndc_rownorm_workspace_bytes",
    "ndc_rownorm_forward",
    "ndc_rownorm_backward",
    "ndc_bias_act_parts",
    "ndc_bias_act",
    "ndc_bias_act_backward",
    "ndc_regroup",
    "ndc_row_sums",
    "ndc_chnorm_parts",
    "ndc_chnorm_forward",
    "ndc_chnorm_backward",
    "ndc_pointwise_gemm_supported",
    "ndc_pointwise_weight_bytes",
    "ndc_pointwise_pack",
    "ndc_pointwise_gemm",
    "ndc_pointwise_gemm_parts",
    "ndc_pointwise_gemm_actgrad",
    "ndc_pointwise_gemm_masked",
)


class Geom(ctypes.Structure):
    """Mirror of ``struct ndc_geom``."""

    _fields_ = [
        ("batch", ctypes.c_int32),
        ("groups", ctypes.c_int32),
        ("m", ctypes.c_int32),
        ("sc", ctypes.c_int32),
        ("size", ctypes.c_int32 * 3),
        ("kernel", ctypes.c_int32 * 3),
        ("dtype", ctypes.c_int32),
        ("relu_input", ctypes.c_int32),
        ("path", ctypes.c_int32),
        ("eps", ctypes.c_float),
    ]


def make_geom(batch: int, groups: int, m: int, sc: int, spatial: Sequence[int],
              kernel: Sequence[int], dtype: int, relu_input: bool, eps: float,
              path: int = PATH_AUTO) -> Geom:
    rank = len(spatial)
    if not 1 <= rank <= 3 or len(kernel) != rank:
        # same error class the reference raises for an unsupported rank
        # (deconver/deconvolution/kernels.py:715-716)
        raise ValueError(f"unsupported spatial rank {rank} / kernel rank {len(kernel)}")
    size = (ctypes.c_int32 * 3)(*([1] * (3 - rank) + [int(v) for v in spatial]))
    kern = (ctypes.c_int32 * 3)(*([1] * (3 - rank) + [int(v) for v in kernel]))
    return Geom(int(batch), int(groups), int(m), int(sc), size, kern, int(dtype),
                1 if relu_input else 0, int(path), float(eps))


class NdcError(RuntimeError):
    pass


class NdcLibrary:
    """A loaded build of the C ABI (the HIP product, or the host checker in CPU tests)."""

    def __init__(self, path: str):
        self.path = path
        self._dll = ctypes.CDLL(path)
        d = self._dll
        vp, fp = ctypes.c_void_p, ctypes.c_void_p
        gp = ctypes.POINTER(Geom)
        d.ndc_version.restype = ctypes.c_int
        d.ndc_status_string.restype = ctypes.c_char_p
        d.ndc_status_string.argtypes = [ctypes.c_int]
        d.ndc_fused_supported.argtypes = [gp]
        d.ndc_check_geometry.argtypes = [gp]
        d.ndc_backward_uses_saved.argtypes = [gp]
        d.ndc_matrix_kernels.argtypes = [ctypes.c_int]
        d.ndc_forward.argtypes = [gp, vp, vp, fp, fp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp]
        if hasattr(d, "ndc_forward_noalloc"):   # HIP build only
            d.ndc_forward_noalloc.argtypes = [gp, vp, vp, fp, fp, vp, vp, vp, vp, vp]
        d.ndc_forward_workspace_bytes.restype = ctypes.c_size_t
        d.ndc_forward_workspace_bytes.argtypes = [gp]
        d.ndc_backward_workspace_bytes.restype = ctypes.c_size_t
        d.ndc_backward_workspace_bytes.argtypes = [gp] + [ctypes.c_int] * 4
        d.ndc_backward.argtypes = [gp, vp, vp, vp, vp, vp, fp, fp, vp, vp, vp, fp, fp, vp,
                                   ctypes.c_size_t, vp]
        d.ndc_backward_profiled.argtypes = d.ndc_backward.argtypes + [ctypes.POINTER(ctypes.c_float)]
        d.ndc_gconv.argtypes = [gp, vp, fp, fp, ctypes.c_int, vp, vp]
        d.ndc_relayout.argtypes = [vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_int, ctypes.c_int, vp]
        d.ndc_rownorm_workspace_bytes.restype = ctypes.c_size_t
        d.ndc_rownorm_workspace_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64]
        d.ndc_rownorm_forward.argtypes = [vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                          ctypes.c_float, vp, ctypes.c_size_t, vp]
        d.ndc_rownorm_backward.argtypes = [vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                           vp, ctypes.c_size_t, vp]
        d.ndc_bias_act_parts.restype = ctypes.c_int64
        d.ndc_bias_act_parts.argtypes = [ctypes.c_int64, ctypes.c_int64]
        d.ndc_bias_act.argtypes = [vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_int, ctypes.c_int, vp]
        d.ndc_bias_act_backward.argtypes = [vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                            ctypes.c_int, ctypes.c_int, vp]
        d.ndc_chnorm_parts.restype = ctypes.c_int64
        d.ndc_chnorm_parts.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        d.ndc_chnorm_forward.argtypes = [vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_int, ctypes.c_float, vp]
        d.ndc_chnorm_backward.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                          ctypes.c_int, vp]
        d.ndc_row_sums.argtypes = [vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, vp]
        d.ndc_pointwise_gemm_supported.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        d.ndc_pointwise_weight_bytes.restype = ctypes.c_size_t
        d.ndc_pointwise_weight_bytes.argtypes = [ctypes.c_int64, ctypes.c_int64]
        d.ndc_pointwise_pack.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, ctypes.c_int64, ctypes.c_int64, vp]
        d.ndc_pointwise_gemm.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_int64, ctypes.c_int, ctypes.c_int, vp]
        d.ndc_pointwise_gemm_masked.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                                ctypes.c_int64, ctypes.c_int, vp]
        d.ndc_pointwise_gemm_parts.restype = ctypes.c_int64
        d.ndc_pointwise_gemm_parts.argtypes = []
        d.ndc_pointwise_gemm_actgrad.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.c_int64, ctypes.c_int64,
                                                 ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, vp]
        d.ndc_regroup.argtypes = [vp, vp, vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp]
        d.ndc_taps_bytes.restype = ctypes.c_size_t
        d.ndc_taps_bytes.argtypes = [gp]
        d.ndc_prepare_taps.argtypes = [gp, fp, vp, ctypes.c_size_t, vp]
        d.ndc_forward_taps.argtypes = [gp, vp, vp, fp, vp, fp, vp, vp, vp, vp, vp]
        d.ndc_backward_taps.argtypes = [gp, vp, vp, vp, vp, vp, fp, vp, fp, vp, vp, vp, fp, fp, vp,
                                        ctypes.c_size_t, vp]
        # answers of the geometry queries, per geometry: they depend on nothing else, and a
        # layer asks the same few questions on every call
        self._answers = {}

    @staticmethod
    def _key(g: Geom) -> tuple:
        return (g.batch, g.groups, g.m, g.sc, tuple(g.size), tuple(g.kernel), g.dtype,
                g.relu_input, g.path)

    def _cached(self, what: str, g: Geom, extra, ask):
        key = (what, self._key(g), extra)
        try:
            return self._answers[key]
        except KeyError:
            if len(self._answers) > 4096:
                self._answers.clear()
            val = self._answers[key] = ask()
            return val

    def _check(self, status: int, what: str) -> None:
        if status != 0:
            msg = self._dll.ndc_status_string(status).decode()
            raise NdcError(f"{what} failed: {msg} (status {status})")

    def version(self) -> int:
        return self._dll.ndc_version()

    def fused_supported(self, g: Geom) -> bool:
        return self._cached("fused", g, None,
                            lambda: bool(self._dll.ndc_fused_supported(ctypes.byref(g))))

    def check_geometry(self, g: Geom) -> int:
        return self._cached("check", g, None, lambda: self._dll.ndc_check_geometry(ctypes.byref(g)))

    def matrix_kernels(self, enabled: Optional[bool] = None) -> bool:
        """Get or set whether the bf16 3x3x3 kernels built on the 4x4x4 matrix instruction may
        be chosen (off by default)."""
        return bool(self._dll.ndc_matrix_kernels(-1 if enabled is None else int(bool(enabled))))

    def backward_uses_saved(self, g: Geom) -> bool:
        return self._cached("saved", g, None,
                            lambda: bool(self._dll.ndc_backward_uses_saved(ctypes.byref(g))))

    def forward_workspace_bytes(self, g: Geom) -> int:
        return self._cached("fws", g, None,
                            lambda: self._dll.ndc_forward_workspace_bytes(ctypes.byref(g)))

    def taps_bytes(self, g: Geom) -> int:
        """Bytes of a prepared filter table for ``g`` (0: its kernels read the filter itself)."""
        return self._cached("taps", g, None, lambda: self._dll.ndc_taps_bytes(ctypes.byref(g)))

    def prepare_taps(self, g: Geom, h: int, taps: int, taps_bytes: int, stream) -> None:
        self._check(self._dll.ndc_prepare_taps(ctypes.byref(g), h, taps, taps_bytes, stream),
                    "ndc_prepare_taps")

    def forward_taps(self, g: Geom, x, z, h, taps, bias, out, t1, s_over_den, ratio, stream) -> None:
        """``forward`` with a filter table prepared by ``prepare_taps``: no workspace."""
        self._check(self._dll.ndc_forward_taps(ctypes.byref(g), x, z, h, taps, bias, out, t1,
                                               s_over_den, ratio, stream), "ndc_forward_taps")

    def backward_taps(self, g: Geom, x, z, t1, s_over_den, ratio, h, taps, bias, gout, gx, gz, gh,
                      gb, ws, ws_bytes, stream) -> None:
        self._check(
            self._dll.ndc_backward_taps(ctypes.byref(g), x, z, t1, s_over_den, ratio, h, taps, bias,
                                        gout, gx, gz, gh, gb, ws, ws_bytes, stream),
            "ndc_backward_taps")

    def forward(self, g: Geom, x: int, z: int, h: int, bias: Optional[int], out: int,
                t1: Optional[int], s_over_den: Optional[int], ratio: Optional[int],
                ws: Optional[int], ws_bytes: int, stream: Optional[int]) -> None:
        self._check(self._dll.ndc_forward(ctypes.byref(g), x, z, h, bias, out, t1, s_over_den, ratio,
                                          ws, ws_bytes, stream), "ndc_forward")

    def forward_noalloc(self, g: Geom, x: int, z: int, h: int, bias: Optional[int], out: int,
                        t1: Optional[int], s_over_den: Optional[int], ratio: Optional[int],
                        stream: Optional[int]) -> None:
        """``forward`` with the scratch in the library's own device array (no workspace)."""
        self._check(self._dll.ndc_forward_noalloc(ctypes.byref(g), x, z, h, bias, out, t1,
                                                  s_over_den, ratio, stream), "ndc_forward_noalloc")

    def noalloc_init(self) -> None:
        """Set-up of ``forward_noalloc`` on the current device (needed before a stream capture)."""
        self._check(self._dll.ndc_noalloc_init(), "ndc_noalloc_init")

    def backward_workspace_bytes(self, g: Geom, need_gx, need_gz, need_gh, need_gb) -> int:
        flags = (int(need_gx), int(need_gz), int(need_gh), int(need_gb))
        return self._cached("bws", g, flags, lambda: self._dll.ndc_backward_workspace_bytes(
            ctypes.byref(g), *flags))

    def backward(self, g: Geom, x, z, t1, s_over_den, ratio, h, bias, gout, gx, gz, gh, gb, ws,
                 ws_bytes, stream) -> None:
        self._check(
            self._dll.ndc_backward(ctypes.byref(g), x, z, t1, s_over_den, ratio, h, bias, gout, gx,
                                   gz, gh, gb, ws, ws_bytes, stream),
            "ndc_backward")

    def backward_profiled(self, g: Geom, x, z, t1, s_over_den, ratio, h, bias, gout, gx, gz, gh, gb,
                          ws, ws_bytes, stream):
        """``backward`` plus the device time (ms) of pass 1, pass 2 and the reduction."""
        ms = (ctypes.c_float * 3)()
        self._check(
            self._dll.ndc_backward_profiled(ctypes.byref(g), x, z, t1, s_over_den, ratio, h, bias,
                                            gout, gx, gz, gh, gb, ws, ws_bytes, stream, ms),
            "ndc_backward_profiled")
        return tuple(ms)

    def gconv(self, g: Geom, inp, h, bias, adjoint: bool, out, stream) -> None:
        self._check(self._dll.ndc_gconv(ctypes.byref(g), inp, h, bias, int(adjoint), out, stream),
                    "ndc_gconv")


    def relayout(self, src: int, dst: int, batch: int, channels: int, spatial: int, dtype: int,
                 to_channels_last: bool, stream) -> None:
        """Channels-last (B, S, C) <-> channel-first (B, C, S) copy of an activation tensor."""
        self._check(self._dll.ndc_relayout(src, dst, batch, channels, spatial, dtype,
                                           int(bool(to_channels_last)), stream), "ndc_relayout")

    def rownorm_workspace_bytes(self, rows: int, n: int) -> int:
        return int(self._dll.ndc_rownorm_workspace_bytes(rows, n))

    def rownorm_forward(self, x: int, y: int, stats: int, rows: int, n: int, dtype: int, eps: float,
                        workspace: int, workspace_bytes: int, stream) -> None:
        """``y = (x - mean) / sqrt(var + eps)`` over each of ``rows`` rows of ``n`` elements;
        ``stats`` receives (mean, rstd) per row."""
        self._check(self._dll.ndc_rownorm_forward(x, y, stats, rows, n, dtype, eps, workspace,
                                                  workspace_bytes, stream), "ndc_rownorm_forward")

    def rownorm_backward(self, gy: int, y: int, stats: int, addend: Optional[int], gx: int, rows: int,
                         n: int, dtype: int, workspace: int, workspace_bytes: int, stream) -> None:
        self._check(self._dll.ndc_rownorm_backward(gy, y, stats, addend, gx, rows, n, dtype, workspace,
                                                   workspace_bytes, stream), "ndc_rownorm_backward")

    def bias_act_parts(self, rows: int, n: int) -> int:
        return int(self._dll.ndc_bias_act_parts(rows, n))

    def bias_act(self, z: int, bias: Optional[int], residual: Optional[int], y: int, batch: int,
                 channels: int, n: int, act: int, dtype: int, stream) -> None:
        """``y = act(z + bias[c]) + residual`` on a channel-first ``(batch, channels, n)`` tensor."""
        self._check(self._dll.ndc_bias_act(z, bias, residual, y, batch, channels, n, act, dtype, stream),
                    "ndc_bias_act")

    def bias_act_backward(self, gy: int, z: int, bias: Optional[int], gz: int, gpart: Optional[int],
                          batch: int, channels: int, n: int, act: int, dtype: int, stream) -> None:
        self._check(self._dll.ndc_bias_act_backward(gy, z, bias, gz, gpart, batch, channels, n, act, dtype,
                                                    stream), "ndc_bias_act_backward")

    def pointwise_gemm_supported(self, cin: int, cout: int, n: int, dtype: int) -> bool:
        return bool(self._dll.ndc_pointwise_gemm_supported(cin, cout, n, dtype))

    def pointwise_weight_bytes(self, cin: int, cout: int) -> int:
        return int(self._dll.ndc_pointwise_weight_bytes(cin, cout))

    def pointwise_pack(self, w: int, w_dtype: int, transposed: bool, wfrag: int, cin: int, cout: int,
                       stream) -> None:
        self._check(self._dll.ndc_pointwise_pack(w, w_dtype, int(transposed), wfrag, cin, cout, stream),
                    "ndc_pointwise_pack")

    def pointwise_gemm(self, x: int, wfrag: int, bias: Optional[int], residual: Optional[int], y: int,
                       zkeep: Optional[int], batch: int, cin: int, cout: int, n: int, act: int, dtype: int,
                       stream) -> None:
        """``y = act(W x + bias) + residual`` on channel-first bf16 ``(batch, c, n)`` tensors."""
        self._check(self._dll.ndc_pointwise_gemm(x, wfrag, bias, residual, y, zkeep, batch, cin, cout, n, act,
                                                 dtype, stream), "ndc_pointwise_gemm")

    def pointwise_gemm_masked(self, x: int, wfrag: int, bias: Optional[int], residual: Optional[int], mask: int,
                              y: int, batch: int, cin: int, cout: int, n: int, dtype: int, stream) -> None:
        """``y = (W x + bias + residual)`` where ``mask > 0``, else 0."""
        self._check(self._dll.ndc_pointwise_gemm_masked(x, wfrag, bias, residual, mask, y, batch, cin, cout, n,
                                                        dtype, stream), "ndc_pointwise_gemm_masked")

    def pointwise_gemm_parts(self) -> int:
        return int(self._dll.ndc_pointwise_gemm_parts())

    def pointwise_gemm_actgrad(self, gy: int, wfrag: int, bias: Optional[int], z: int, gz: int,
                               gpart: Optional[int], batch: int, cin: int, cout: int, n: int, act: int,
                               dtype: int, stream) -> None:
        """``gz = (W gy) * act'(z + bias)`` with per-wavefront sums of ``gz`` in ``gpart``."""
        self._check(self._dll.ndc_pointwise_gemm_actgrad(gy, wfrag, bias, z, gz, gpart, batch, cin, cout, n,
                                                         act, dtype, stream), "ndc_pointwise_gemm_actgrad")

    def chnorm_parts(self, batch: int, n: int, dtype: int) -> int:
        return int(self._dll.ndc_chnorm_parts(batch, n, dtype))

    def chnorm_forward(self, x: int, weight: Optional[int], bias: Optional[int], y: int, stats: int,
                       batch: int, channels: int, n: int, dtype: int, eps: float, stream) -> None:
        """Normalisation over the channels of a channel-first ``(batch, channels, n)`` tensor."""
        self._check(self._dll.ndc_chnorm_forward(x, weight, bias, y, stats, batch, channels, n, dtype, eps,
                                                 stream), "ndc_chnorm_forward")

    def chnorm_backward(self, gy: int, x: int, stats: int, weight: Optional[int], gx: int,
                        partial: Optional[int], batch: int, channels: int, n: int, dtype: int, stream) -> None:
        self._check(self._dll.ndc_chnorm_backward(gy, x, stats, weight, gx, partial, batch, channels, n, dtype,
                                                  stream), "ndc_chnorm_backward")

    def row_sums(self, x: int, partial: int, rows: int, n: int, dtype: int, stream) -> None:
        self._check(self._dll.ndc_row_sums(x, partial, rows, n, dtype, stream), "ndc_row_sums")

    def regroup2(self, src: int, dst: int, bias: Optional[int], rows: int, channels: int, D: int, H: int,
                 W: int, depth2: bool, dtype: int, to_channels: bool, stream) -> None:
        """2 x 2 (x 2) windows of the fine grid (rows, D, H, W) <-> 4 (8) planes per row."""
        self._check(self._dll.ndc_regroup(src, dst, bias, rows, channels, D, H, W, int(bool(depth2)), dtype,
                                           int(bool(to_channels)), stream), "ndc_regroup")


_lock = threading.Lock()
_library: Optional[NdcLibrary] = None


def library_available() -> bool:
    return os.path.exists(LIB_PATH)


def get_library() -> NdcLibrary:
    """The HIP library; raises if it has not been built (there is no other backend)."""
    global _library
    if _library is None:
        with _lock:
            if _library is None:
                if not os.path.exists(LIB_PATH):
                    raise NdcError(
                        f"{LIB_PATH} is missing: build it with `python -m deconver_amd.build` "
                        "(hipcc, gfx950). The NDC update has no CPU or PyTorch fallback.")
                _library = NdcLibrary(LIB_PATH)
                if os.environ.get("DECONVER_NDC_MATRIX", "0") == "1":
                    _library.matrix_kernels(True)
    return _library
