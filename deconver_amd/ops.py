"""Tensor-level wrappers over the C ABI: shape/dtype checks, output allocation, pointers.

These take the library explicitly.  The product passes ``_lib.get_library()`` (HIP) with
CUDA tensors; the CPU test-suite passes the host checker with CPU tensors.  Nothing here
computes anything in PyTorch.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib

_DTYPES = {torch.float32: _lib.NDC_F32, torch.bfloat16: _lib.NDC_BF16}


def dtype_tag(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"NDC kernels store activations as float32 or bfloat16, got {dtype}")


def _stream_of(t: Tensor) -> Optional[int]:
    if t.is_cuda:
        return torch.cuda.current_stream(t.device).cuda_stream
    return None


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_common(x: Tensor, z: Tensor, h: Tensor, bias: Optional[Tensor], groups: int, m: int,
                  sc: int) -> Tuple[int, ...]:
    if x.dim() < 3 or x.dim() > 5:
        raise ValueError(f"expected a (B, C, *S) tensor with 1-3 spatial dims, got {tuple(x.shape)}")
    if x.shape[1] != groups * m:
        raise ValueError(f"x has {x.shape[1]} channels, expected groups*m = {groups * m}")
    if tuple(z.shape) != (x.shape[0], groups * sc, *x.shape[2:]):
        raise ValueError(f"z has shape {tuple(z.shape)}, expected "
                         f"{(x.shape[0], groups * sc, *x.shape[2:])}")
    if h.dim() != x.dim() or h.shape[0] * h.shape[1] != groups * m * sc:
        raise ValueError(f"filter of shape {tuple(h.shape)} does not match groups={groups}, "
                         f"m={m}, sc={sc}")
    if x.dtype != z.dtype:
        raise TypeError(f"x ({x.dtype}) and z ({z.dtype}) must share a dtype")
    if h.dtype != torch.float32 or (bias is not None and bias.dtype != torch.float32):
        raise TypeError("filter and bias must be float32")
    for t in (x, z, h, bias):
        if t is not None and (t.device != x.device or not t.is_contiguous()):
            raise ValueError("all tensors must be contiguous and on one device")
    if bias is not None and bias.numel() != groups * sc:
        raise ValueError(f"bias has {bias.numel()} entries, expected {groups * sc}")
    return tuple(h.shape[2:])


def is_channels_last(t: Optional[Tensor]) -> bool:
    """Whether ``t`` is a (B, C, *S) tensor with 2 or 3 spatial dims laid out channels-last
    (``torch.channels_last`` / ``channels_last_3d``) and not also channel-first contiguous."""
    if t is None or t.dim() not in (4, 5) or t.is_contiguous():
        return False
    fmt = torch.channels_last if t.dim() == 4 else torch.channels_last_3d
    return t.is_contiguous(memory_format=fmt)


def to_channel_first(lib: _lib.NdcLibrary, t: Tensor) -> Tensor:
    """A channel-first contiguous copy of a channels-last tensor, made by the library's tiled
    transposition (``ndc_relayout``) instead of a generic strided copy."""
    if not is_channels_last(t):
        return t.contiguous()
    out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
    lib.relayout(t.data_ptr(), out.data_ptr(), t.shape[0], t.shape[1], t[0, 0].numel(),
                 dtype_tag(t.dtype), False, _stream_of(t))
    return out


def to_channels_last(lib: _lib.NdcLibrary, t: Tensor) -> Tensor:
    """The channels-last copy of a channel-first contiguous (B, C, *S) tensor (2 or 3 spatial
    dims), same shape, by the library's tiled transposition."""
    fmt = torch.channels_last if t.dim() == 4 else torch.channels_last_3d
    out = torch.empty(t.shape, dtype=t.dtype, device=t.device, memory_format=fmt)
    lib.relayout(t.data_ptr(), out.data_ptr(), t.shape[0], t.shape[1], t[0, 0].numel(),
                 dtype_tag(t.dtype), True, _stream_of(t))
    return out


def make_geom_for(x: Tensor, h: Tensor, groups: int, m: int, sc: int, eps: float,
                  relu_input: bool, path: int = _lib.PATH_AUTO) -> _lib.Geom:
    return _lib.make_geom(x.shape[0], groups, m, sc, x.shape[2:], h.shape[2:],
                          dtype_tag(x.dtype), relu_input, eps, path)


def prepare_taps(lib: _lib.NdcLibrary, x: Tensor, h: Tensor, *, groups: int, m: int,
                 sc: int) -> Optional[Tensor]:
    """The filter table the kernels for this geometry read instead of ``h`` (today: the packed
    bfloat16 tap pairs of the 3x3x3 dot2 kernels), or ``None`` if they read ``h`` itself.  One
    small launch; valid for every update with this ``h`` on tensors of ``x``'s shape and
    dtype, forward and backward, until ``h`` changes."""
    g = make_geom_for(x, h, groups, m, sc, 0.0, True)
    nbytes = lib.taps_bytes(g)
    if not nbytes:
        return None
    buf = torch.empty(nbytes + 256, dtype=torch.uint8, device=x.device)
    off = -buf.data_ptr() % 256
    taps = buf[off:off + nbytes]   # 256-byte aligned view
    lib.prepare_taps(g, _ptr(h), _ptr(taps), nbytes, _stream_of(x))
    return taps


def update_forward(lib: _lib.NdcLibrary, x: Tensor, z: Tensor, h: Tensor,
                   bias: Optional[Tensor], *, groups: int, m: int, sc: int, eps: float,
                   relu_input: bool, need_t1: bool = True, save_ratio: bool = False,
                   path: int = _lib.PATH_AUTO, taps: Optional[Tensor] = None):
    """``out = s*(A(x)+eps)/(A(K(s))+eps)`` with ``s = relu?(z+bias)``.

    Returns ``(out, t1)``, or ``(out, t1, (s_over_den, ratio))`` with ``save_ratio``: the two
    extra tensors (shape of ``out``) that let :func:`update_backward` skip re-gathering
    ``A(x)`` and ``A(t1)``."""
    _check_common(x, z, h, bias, groups, m, sc)
    g = make_geom_for(x, h, groups, m, sc, eps, relu_input, path)
    out = torch.empty_like(z)
    want_t1 = need_t1 or not lib.fused_supported(g) or path == _lib.PATH_DIRECT
    t1 = torch.empty_like(x) if want_t1 else None
    s_over_den = torch.empty_like(z) if save_ratio else None
    ratio = torch.empty_like(z) if save_ratio else None
    if taps is not None:
        lib.forward_taps(g, _ptr(x), _ptr(z), _ptr(h), _ptr(taps), _ptr(bias), _ptr(out), _ptr(t1),
                         _ptr(s_over_den), _ptr(ratio), _stream_of(x))
    else:
        nbytes = lib.forward_workspace_bytes(g)
        ws_ptr = None
        if nbytes:
            ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=x.device)
            ws_ptr = (ws.data_ptr() + 255) // 256 * 256
        lib.forward(g, _ptr(x), _ptr(z), _ptr(h), _ptr(bias), _ptr(out), _ptr(t1),
                    _ptr(s_over_den), _ptr(ratio), ws_ptr, nbytes, _stream_of(x))
    if save_ratio:
        return out, t1, (s_over_den, ratio)
    return out, t1


def update_backward(lib: _lib.NdcLibrary, x: Tensor, z: Tensor, t1: Tensor, h: Tensor,
                    bias: Optional[Tensor], gout: Tensor, *, groups: int, m: int, sc: int,
                    eps: float, relu_input: bool, need_x: bool = True, need_z: bool = True,
                    need_h: bool = True, need_b: bool = True,
                    path: int = _lib.PATH_AUTO, pass_times: Optional[list] = None,
                    saved: Optional[Tuple[Tensor, Tensor]] = None,
                    taps: Optional[Tensor] = None):
    """Gradients ``(gx, gz, gh, gb)`` of the update; entries not asked for are ``None``.

    ``saved``: the ``(s_over_den, ratio)`` pair a ``save_ratio`` forward call returned for the
    same inputs.

    ``taps``: the table :func:`prepare_taps` made for this ``h`` (skips packing it again).

    ``pass_times``: a list that, if given, receives the device milliseconds of the three
    backward stages (the call then synchronises)."""
    _check_common(x, z, h, bias, groups, m, sc)
    if gout.shape != z.shape or gout.dtype != z.dtype or not gout.is_contiguous():
        raise ValueError("gout must be contiguous with the shape and dtype of z")
    if t1.shape != x.shape or t1.dtype != x.dtype or not t1.is_contiguous():
        raise ValueError("t1 must be contiguous with the shape and dtype of x")
    s_over_den = ratio = None
    if saved is not None:
        s_over_den, ratio = saved
        for t in (s_over_den, ratio):
            if t.shape != z.shape or t.dtype != z.dtype or not t.is_contiguous():
                raise ValueError("saved tensors must be contiguous with the shape and dtype of z")
    need_b = need_b and bias is not None
    g = make_geom_for(x, h, groups, m, sc, eps, relu_input, path)
    gx = torch.empty_like(x) if need_x else None
    gz = torch.empty_like(z) if need_z else None
    gh = torch.empty_like(h) if need_h else None
    gb = torch.empty(groups * sc, dtype=torch.float32, device=x.device) if need_b else None
    nbytes = lib.backward_workspace_bytes(g, need_x, need_z, need_h, need_b)
    ws = torch.empty(max(nbytes, 1) + 256, dtype=torch.uint8, device=x.device)
    ws_ptr = (ws.data_ptr() + 255) // 256 * 256
    args = (g, _ptr(x), _ptr(z), _ptr(t1), _ptr(s_over_den), _ptr(ratio), _ptr(h), _ptr(bias),
            _ptr(gout), _ptr(gx),
            _ptr(gz), _ptr(gh), _ptr(gb), ws_ptr, nbytes, _stream_of(x))
    if taps is not None and pass_times is None:
        lib.backward_taps(*args[:7], _ptr(taps), *args[7:])
    elif pass_times is None:
        lib.backward(*args)
    else:
        pass_times[:] = lib.backward_profiled(*args)
    return gx, gz, gh, gb


def gconv(lib: _lib.NdcLibrary, inp: Tensor, h: Tensor, *, groups: int, m: int, sc: int,
          adjoint: bool, bias: Optional[Tensor] = None, relu_input: bool = False) -> Tensor:
    """``K(inp)`` (adjoint=False, inp has groups*sc channels) or ``A(inp)`` (groups*m channels)."""
    cin = groups * (m if adjoint else sc)
    cout = groups * (sc if adjoint else m)
    if inp.shape[1] != cin:
        raise ValueError(f"input has {inp.shape[1]} channels, expected {cin}")
    if not inp.is_contiguous() or not h.is_contiguous() or h.dtype != torch.float32:
        raise ValueError("input and filter must be contiguous; filter float32")
    g = _lib.make_geom(inp.shape[0], groups, m, sc, inp.shape[2:], h.shape[2:],
                       dtype_tag(inp.dtype), relu_input, 0.0, _lib.PATH_DIRECT)
    out = torch.empty((inp.shape[0], cout, *inp.shape[2:]), dtype=inp.dtype, device=inp.device)
    lib.gconv(g, _ptr(inp), _ptr(h), _ptr(bias), adjoint, _ptr(out), _stream_of(inp))
    return out


def _rownorm_workspace(lib: _lib.NdcLibrary, rows: int, n: int, device) -> Tensor:
    return torch.empty(max(lib.rownorm_workspace_bytes(rows, n) // 4, 2), dtype=torch.float32, device=device)


def rownorm_forward(lib: _lib.NdcLibrary, x: Tensor, eps: float):
    """Normalises each row of the contiguous matrix ``x`` (rows, n) to zero mean and unit
    (biased) variance.  Returns ``(y, stats)``; ``stats`` (rows, 2) holds (mean, rstd)."""
    if x.dim() != 2 or not x.is_contiguous():
        raise ValueError("rownorm_forward wants a contiguous (rows, n) matrix")
    rows, n = x.shape
    y = torch.empty_like(x)
    stats = torch.empty(rows, 2, dtype=torch.float32, device=x.device)
    ws = _rownorm_workspace(lib, rows, n, x.device)
    lib.rownorm_forward(_ptr(x), _ptr(y), _ptr(stats), rows, n, dtype_tag(x.dtype), eps, _ptr(ws),
                        ws.numel() * 4, _stream_of(x))
    return y, stats


def rownorm_backward(lib: _lib.NdcLibrary, gy: Tensor, y: Tensor, stats: Tensor,
                     addend: Optional[Tensor] = None) -> Tensor:
    """Gradient of :func:`rownorm_forward` with respect to its input, from the gradient of
    its output ``gy``, its output ``y`` and its ``stats``; plus ``addend`` (a tensor like
    ``gy``: the gradient that reaches the input by another way), if given."""
    if gy.shape != y.shape or gy.dtype != y.dtype or not (gy.is_contiguous() and y.is_contiguous()):
        raise ValueError("rownorm_backward wants gy and y contiguous, of one shape and dtype")
    if addend is not None and (addend.shape != y.shape or addend.dtype != y.dtype or not addend.is_contiguous()):
        raise ValueError("addend must be contiguous, of the shape and dtype of gy")
    rows, n = y.shape
    gx = torch.empty_like(y)
    ws = _rownorm_workspace(lib, rows, n, y.device)
    lib.rownorm_backward(_ptr(gy), _ptr(y), _ptr(stats), _ptr(addend), _ptr(gx), rows, n, dtype_tag(y.dtype), _ptr(ws),
                         ws.numel() * 4, _stream_of(y))
    return gx


ACTS = {None: _lib.ACT_NONE, "none": _lib.ACT_NONE, "relu": _lib.ACT_RELU, "gelu": _lib.ACT_GELU}


def bias_act(lib: _lib.NdcLibrary, z: Tensor, bias: Optional[Tensor], residual: Optional[Tensor],
             act: Optional[str], inplace: bool = False) -> Tensor:
    """``act(z + bias[c]) + residual`` for a contiguous channel-first ``z`` of shape (B, C, n);
    ``bias`` float32 of C entries or None, ``residual`` like ``z`` or None.  ``inplace`` writes
    the result over ``z``."""
    if z.dim() != 3 or not z.is_contiguous():
        raise ValueError("bias_act wants a contiguous (B, C, n) tensor")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != z.shape[1] or not bias.is_contiguous()):
        raise ValueError("bias must be float32 with one entry per channel")
    if residual is not None and (residual.shape != z.shape or residual.dtype != z.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous, of the shape and dtype of z")
    y = z if inplace else torch.empty_like(z)
    B, C, n = z.shape
    lib.bias_act(_ptr(z), _ptr(bias), _ptr(residual), _ptr(y), B, C, n, ACTS[act], dtype_tag(z.dtype),
                 _stream_of(z))
    return y


def bias_act_backward(lib: _lib.NdcLibrary, gy: Tensor, z: Tensor, bias: Optional[Tensor], act: str,
                      need_bias_grad: bool = True, inplace: bool = False):
    """``(gz, gbias)`` with ``gz = gy * act'(z + bias)`` and ``gbias`` its sum over batch and
    voxels in float32 (None unless ``need_bias_grad``).  ``inplace`` writes ``gz`` over ``gy``."""
    if gy.shape != z.shape or gy.dtype != z.dtype or not (gy.is_contiguous() and z.is_contiguous()):
        raise ValueError("bias_act_backward wants gy and z contiguous, of one shape and dtype")
    B, C, n = z.shape
    gz = gy if inplace else torch.empty_like(gy)
    parts = lib.bias_act_parts(B * C, n)
    gpart = torch.empty(B, C, parts, dtype=torch.float32, device=z.device) if need_bias_grad else None
    lib.bias_act_backward(_ptr(gy), _ptr(z), _ptr(bias), _ptr(gz), _ptr(gpart), B, C, n, ACTS[act],
                          dtype_tag(z.dtype), _stream_of(z))
    return gz, (gpart.sum((0, 2)) if need_bias_grad else None)


def pointwise_gemm_applies(lib: _lib.NdcLibrary, x: Tensor, cout: int, act: Optional[str] = None,
                           keep_z: bool = False) -> bool:
    """Whether ``pointwise_gemm`` takes the projection of ``x`` (B, cin, n) to ``cout`` channels:
    contiguous bfloat16 on the GPU in the shapes ``ndc_pointwise_gemm_supported`` lists (with
    more than 256 input channels: no activation, nothing kept)."""
    if x.dim() == 3 and x.shape[1] > 256 and (act is not None or keep_z):
        return False
    return (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 3 and x.is_contiguous()
            and lib.pointwise_gemm_supported(x.shape[1], cout, x.shape[2], _lib.NDC_BF16))


def pointwise_pack(lib: _lib.NdcLibrary, weight: Tensor, transposed: bool = False) -> Tensor:
    """The weight of a 1x1 projection in the order ``pointwise_gemm`` reads it (bf16).
    ``weight``: ``(cout, cin)``, contiguous, float32 or bfloat16 (another floating dtype is cast
    to bfloat16 first); with ``transposed`` it is taken as the ``(cin, cout)`` storage of the
    matrix to apply (the input gradient's ``W^T`` from ``W`` as it lies)."""
    if weight.is_floating_point() and weight.dtype not in _DTYPES:
        weight = weight.to(torch.bfloat16)
    if weight.dim() != 2 or not weight.is_contiguous() or weight.dtype not in _DTYPES:
        raise ValueError("pointwise_pack wants a contiguous floating-point matrix")
    cout, cin = (weight.shape[1], weight.shape[0]) if transposed else weight.shape
    wfrag = torch.empty(cout * cin, dtype=torch.bfloat16, device=weight.device)
    lib.pointwise_pack(_ptr(weight), dtype_tag(weight.dtype), transposed, _ptr(wfrag), cin, cout,
                       _stream_of(weight))
    return wfrag


def pointwise_gemm(lib: _lib.NdcLibrary, x: Tensor, wfrag: Tensor, cout: int, bias: Optional[Tensor] = None,
                   residual: Optional[Tensor] = None, act: Optional[str] = None, keep_z: bool = False,
                   mask: Optional[Tensor] = None):
    """``y = act(W x + bias) + residual`` for contiguous bfloat16 ``x`` (B, cin, n) and packed
    ``W`` (``pointwise_pack``); returns ``(y, z)`` with ``z`` the product before bias and
    activation when ``keep_z``, else None.  With ``mask`` (of the output's shape; no activation,
    nothing kept): ``y = W x + bias + residual`` where ``mask > 0``, else 0."""
    B, cin, n = x.shape
    if mask is not None:
        if act is not None or keep_z:
            raise ValueError("the masked form takes no activation and keeps nothing")
        if mask.shape != (B, cout, n) or mask.dtype != x.dtype or not mask.is_contiguous():
            raise ValueError("mask must be contiguous, of the output's shape and dtype")
    if wfrag.numel() != cin * cout or wfrag.dtype != torch.bfloat16:
        raise ValueError("wfrag does not belong to this projection")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != cout or not bias.is_contiguous()):
        raise ValueError("bias must be float32 with one entry per output channel")
    if residual is not None and (residual.shape != (B, cout, n) or residual.dtype != x.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous, of the output's shape and dtype")
    y = x.new_empty(B, cout, n)
    z = x.new_empty(B, cout, n) if keep_z else None
    if mask is not None:
        lib.pointwise_gemm_masked(_ptr(x), _ptr(wfrag), _ptr(bias), _ptr(residual), _ptr(mask), _ptr(y), B, cin,
                                  cout, n, _lib.NDC_BF16, _stream_of(x))
        return y, None
    lib.pointwise_gemm(_ptr(x), _ptr(wfrag), _ptr(bias), _ptr(residual), _ptr(y), _ptr(z), B, cin, cout, n,
                       ACTS[act], _lib.NDC_BF16, _stream_of(x))
    return y, z


def pointwise_gemm_actgrad(lib: _lib.NdcLibrary, gy: Tensor, wfrag: Tensor, cout: int, z: Tensor,
                           bias: Optional[Tensor], act: str, need_bias_grad: bool = True):
    """``(gz, gbias)`` with ``gz = (W gy) * act'(z + bias)`` for contiguous bfloat16 ``gy``
    (B, cin, n), packed ``W`` (cout x cin) and ``z`` (B, cout, n): the input gradient of a
    projection taken through the activation that made its input.  ``gbias``: the sum of ``gz``
    over batch and voxels, float32 (None unless ``need_bias_grad``)."""
    B, cin, n = gy.shape
    if wfrag.numel() != cin * cout or wfrag.dtype != torch.bfloat16:
        raise ValueError("wfrag does not belong to this projection")
    if z.shape != (B, cout, n) or z.dtype != gy.dtype or not z.is_contiguous():
        raise ValueError("z must be contiguous, of the output's shape and dtype")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != cout or not bias.is_contiguous()):
        raise ValueError("bias must be float32 with one entry per output channel")
    if act not in ("relu", "gelu"):
        raise ValueError("act must be 'relu' or 'gelu'")
    gz = torch.empty_like(z)
    gpart = (torch.empty(lib.pointwise_gemm_parts(), cout, dtype=torch.float32, device=gy.device)
             if need_bias_grad else None)
    lib.pointwise_gemm_actgrad(_ptr(gy), _ptr(wfrag), _ptr(bias), _ptr(z), _ptr(gz), _ptr(gpart), B, cin, cout,
                               n, ACTS[act], _lib.NDC_BF16, _stream_of(gy))
    return gz, (gpart.sum(0) if need_bias_grad else None)


def regroup2_applies(fine_shape, dtype, *ptrs) -> bool:
    """Whether ``ndc_regroup`` takes a fine-grid tensor ``(B, C, [D,] H, W)``: float32 or
    bfloat16, even extents, rows of whole 16-byte vectors, 16-byte aligned buffers."""
    if dtype not in _DTYPES or len(fine_shape) not in (4, 5):
        return False
    vn = 16 // (2 if dtype == torch.bfloat16 else 4)
    return (all(v % 2 == 0 and v > 0 for v in fine_shape[2:]) and fine_shape[-1] % vn == 0
            and fine_shape[0] * fine_shape[1] > 0 and all(p % 16 == 0 for p in ptrs))


def windows_to_channels(lib: _lib.NdcLibrary, x: Tensor) -> Tensor:
    """``(B, C, [D,] H, W) -> (B, C * 2^nd, [D/2,] H/2, W/2)``: every 2 x 2 (x 2) window becomes
    2^nd channels, channel-major then window offset.  ``x`` contiguous."""
    B, C = x.shape[:2]
    sp = list(x.shape[2:])
    nd = len(sp)
    out = torch.empty(B, C * 2 ** nd, *[v // 2 for v in sp], dtype=x.dtype, device=x.device)
    D = sp[0] if nd == 3 else 1
    lib.regroup2(_ptr(x), _ptr(out), None, B * C, C, D, sp[-2], sp[-1], nd == 3, dtype_tag(x.dtype), True,
                 _stream_of(x))
    return out


def channels_to_windows(lib: _lib.NdcLibrary, y: Tensor, bias: Optional[Tensor] = None) -> Tensor:
    """Inverse of :func:`windows_to_channels`: ``(B, C * 2^nd, *coarse) -> (B, C, *(2 coarse))``,
    plus ``bias[c]`` (float32, C entries) if given.  ``y`` contiguous."""
    B = y.shape[0]
    sp = [2 * v for v in y.shape[2:]]
    nd = len(sp)
    C = y.shape[1] // 2 ** nd
    out = torch.empty(B, C, *sp, dtype=y.dtype, device=y.device)
    D = sp[0] if nd == 3 else 1
    lib.regroup2(_ptr(y), _ptr(out), _ptr(bias), B * C, C, D, sp[-2], sp[-1], nd == 3, dtype_tag(y.dtype), False,
                 _stream_of(y))
    return out


def channel_sums(lib: _lib.NdcLibrary, g: Tensor) -> Tensor:
    """Sum of a contiguous ``(B, C, n)`` tensor over batch and voxels, float32, ``C`` entries:
    the bias gradient of a projection from its output gradient."""
    if g.dim() != 3 or not g.is_contiguous():
        raise ValueError("channel_sums wants a contiguous (B, C, n) tensor")
    B, C, n = g.shape
    parts = lib.bias_act_parts(B * C, n)
    partial = torch.empty(B, C, parts, dtype=torch.float32, device=g.device)
    lib.row_sums(_ptr(g), _ptr(partial), B * C, n, dtype_tag(g.dtype), _stream_of(g))
    return partial.sum((0, 2))


def chnorm_forward(lib: _lib.NdcLibrary, x: Tensor, weight: Optional[Tensor], bias: Optional[Tensor],
                   eps: float):
    """Normalises a contiguous channel-first ``(B, C, n)`` tensor over its channel axis (per
    voxel), with float32 ``weight`` / ``bias`` of C entries or None.  Returns ``(y, stats)``;
    ``stats`` (B, 2, n) holds mean and rstd per voxel."""
    if x.dim() != 3 or not x.is_contiguous():
        raise ValueError("chnorm_forward wants a contiguous (B, C, n) tensor")
    for p in (weight, bias):
        if p is not None and (p.dtype != torch.float32 or p.numel() != x.shape[1] or not p.is_contiguous()):
            raise ValueError("weight and bias must be float32 with one entry per channel")
    B, C, n = x.shape
    y = torch.empty_like(x)
    stats = torch.empty(B, 2, n, dtype=torch.float32, device=x.device)
    lib.chnorm_forward(_ptr(x), _ptr(weight), _ptr(bias), _ptr(y), _ptr(stats), B, C, n, dtype_tag(x.dtype), eps,
                       _stream_of(x))
    return y, stats


def chnorm_backward(lib: _lib.NdcLibrary, gy: Tensor, x: Tensor, stats: Tensor, weight: Optional[Tensor],
                    need_affine_grads: bool = True):
    """``(gx, gweight, gbias)`` of :func:`chnorm_forward`; the last two float32, or None."""
    if gy.shape != x.shape or gy.dtype != x.dtype or not (gy.is_contiguous() and x.is_contiguous()):
        raise ValueError("chnorm_backward wants gy and x contiguous, of one shape and dtype")
    B, C, n = x.shape
    gx = torch.empty_like(x)
    partial = None
    if need_affine_grads:
        parts = lib.chnorm_parts(B, n, dtype_tag(x.dtype))
        partial = torch.empty(parts, C, 2, dtype=torch.float32, device=x.device)
    lib.chnorm_backward(_ptr(gy), _ptr(x), _ptr(stats), _ptr(weight), _ptr(gx), _ptr(partial), B, C, n,
                        dtype_tag(x.dtype), _stream_of(x))
    if partial is None:
        return gx, None, None
    sums = partial.sum(0)
    return gx, sums[:, 0].contiguous(), sums[:, 1].contiguous()
