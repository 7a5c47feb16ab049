"""ctypes view of the C ABI in include/teletron_norm.h, taking torch tensors.

Thin on purpose: it forwards device pointers, sizes and the current HIP stream
to libteletron_norm.so and raises on a non-zero status.  There is no fallback:
if the library is not built, loading fails with instructions to build it.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

# TELETRON_AMD_LIB=<path> loads another build of the library (a tuning variant from
# `python -m teletron_amd.build --variant`); the extension modules always link the shipped one.
_LIB_PATH = os.environ.get("TELETRON_AMD_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                                                               "libteletron_norm.so")

BF16, F32, F16 = 0, 1, 2
_DTYPES = {torch.bfloat16: BF16, torch.float32: F32, torch.float16: F16}

EXPORTS = (
    "tt_norm_abi_version", "tt_norm_status_string", "tt_norm_last_error", "tt_norm_supported", "tt_norm_tuned",
    "tt_rmsnorm_forward", "tt_rmsnorm_backward_workspace_bytes", "tt_rmsnorm_backward",
    "tt_rmsnorm_backward_from_out", "tt_rmsnorm_forward_strided", "tt_rmsnorm_backward_strided",
    "tt_adaln_forward", "tt_adaln_forward_xnorm", "tt_adaln_backward_workspace_bytes",
    "tt_adaln_backward", "tt_adaln_backward_from_xnorm", "tt_norm_wide_forms_supported",
    "tt_norm_profile_next_row_kernel",
    "tt_gated_residual_adaln_forward", "tt_gated_residual_adaln_backward_workspace_bytes",
    "tt_gated_residual_adaln_backward", "tt_adaln_backward_residual", "tt_adaln_backward_static",
    "tt_rmsnorm_rope_forward_strided", "tt_rmsnorm_rope_backward_strided",
    "tt_adaln_forward_seq_first", "tt_adaln_backward_seq_first", "tt_norm_copy_rows_strided",
)


class NormError(RuntimeError):
    def __init__(self, status: int, what: str, detail: str):
        super().__init__(f"{what}: status {status} ({detail})")
        self.status = status


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(f"{_LIB_PATH} is not built; run `python -m teletron_amd.build`")
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, dbl, ci, sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_double, ctypes.c_int, ctypes.c_size_t
        L.tt_norm_abi_version.restype = ci
        L.tt_norm_status_string.restype = ctypes.c_char_p
        L.tt_norm_status_string.argtypes = [ci]
        L.tt_norm_last_error.restype = ctypes.c_char_p
        L.tt_norm_supported.argtypes = [i64, ci]
        L.tt_norm_tuned.argtypes = [i64, ci]
        L.tt_norm_wide_forms_supported.argtypes = [i64, ci]
        L.tt_rmsnorm_forward.argtypes = [vp, vp, vp, vp, i64, i64, dbl, ci, vp]
        L.tt_rmsnorm_backward_workspace_bytes.restype = sz
        L.tt_rmsnorm_backward_workspace_bytes.argtypes = [i64, i64, ci]
        L.tt_rmsnorm_backward.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, ci, vp, sz, vp]
        L.tt_rmsnorm_backward_from_out.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, ci, vp, sz, vp]
        L.tt_rmsnorm_forward_strided.argtypes = [vp, vp, vp, vp] + [i64] * 7 + [dbl, ci, vp]
        L.tt_rmsnorm_backward_strided.argtypes = [vp] * 6 + [i64] * 10 + [ci, vp, sz, vp]
        L.tt_rmsnorm_rope_forward_strided.argtypes = [vp] * 6 + [i64] * 8 + [dbl, ci, vp]
        L.tt_rmsnorm_rope_backward_strided.argtypes = [vp] * 8 + [i64] * 11 + [ci, vp, sz, vp]
        L.tt_adaln_forward.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, dbl, ci, vp]
        L.tt_adaln_forward_xnorm.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, dbl, ci, vp]
        L.tt_adaln_backward_workspace_bytes.restype = sz
        L.tt_adaln_backward_workspace_bytes.argtypes = [i64, i64, i64, ci]
        L.tt_adaln_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, vp, sz, vp]
        L.tt_adaln_forward_seq_first.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, dbl, ci, vp]
        L.tt_adaln_backward_seq_first.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, vp, sz, vp]
        L.tt_adaln_backward_static.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, vp]
        L.tt_adaln_backward_from_xnorm.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, ci, vp, sz, vp]
        L.tt_gated_residual_adaln_forward.argtypes = [vp] * 9 + [i64, i64, i64, dbl, ci, vp]
        L.tt_gated_residual_adaln_backward_workspace_bytes.restype = sz
        L.tt_gated_residual_adaln_backward_workspace_bytes.argtypes = [i64, i64, i64, ci]
        L.tt_gated_residual_adaln_backward.argtypes = [vp] * 13 + [i64, i64, i64, ci, vp, sz, vp]
        L.tt_adaln_backward_residual.argtypes = [vp] * 9 + [i64, i64, i64, ci, vp, sz, vp]
        L.tt_norm_copy_rows_strided.argtypes = [vp, vp] + [i64] * 7 + [ci, vp]
        L.tt_norm_profile_next_row_kernel.argtypes = [vp, vp]
        _lib = L
    return _lib


def _check(status: int, what: str):
    if status != 0:
        L = lib()
        raise NormError(status, what, (L.tt_norm_last_error() or L.tt_norm_status_string(status)).decode())


def _p(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {t.dtype}")
    return _DTYPES[t.dtype]


def _dense_gpu(*ts):
    for t in ts:
        if not t.is_cuda:
            raise ValueError("tensor must live on the GPU")
        if not t.is_contiguous():
            raise ValueError("tensor must be contiguous")


def _workspace(nbytes: int, like: torch.Tensor) -> torch.Tensor:
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=like.device)


def rmsnorm_forward(x, weight, eps: float, out=None, rstd=None):
    _dense_gpu(x, weight)
    cols = weight.numel()
    rows = x.numel() // cols
    out = torch.empty_like(x) if out is None else out
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device) if rstd is None else rstd
    with torch.cuda.device(x.device):
        _check(lib().tt_rmsnorm_forward(_p(out), _p(rstd), _p(x), _p(weight), rows, cols, eps, _dt(x),
                                        _stream(x)), "tt_rmsnorm_forward")
    return out, rstd


def rmsnorm_backward(dout, x, weight, rstd, from_out: bool = False, dx=None, dweight=None):
    _dense_gpu(dout, x, weight, rstd)
    cols = weight.numel()
    rows = x.numel() // cols
    dx = torch.empty_like(x) if dx is None else dx
    dweight = torch.empty_like(weight) if dweight is None else dweight
    with torch.cuda.device(x.device):
        L = lib()
        n = L.tt_rmsnorm_backward_workspace_bytes(rows, cols, _dt(x))
        ws = _workspace(n, x)
        fn = L.tt_rmsnorm_backward_from_out if from_out else L.tt_rmsnorm_backward
        _check(fn(_p(dx), _p(dweight), _p(dout), _p(x), _p(weight), _p(rstd), rows, cols, _dt(x),
                  _p(ws), n, _stream(x)), fn.__name__)
    return dx, dweight


def _view3(t: torch.Tensor):
    """(sizes, strides) of t's leading dimensions padded to three; last dimension must be contiguous."""
    if t.dim() < 1 or t.dim() > 4 or t.stride(-1) != 1:
        raise ValueError("need a view of at most 4 dimensions with a contiguous last dimension")
    sizes = [1] * (4 - t.dim()) + list(t.shape[:-1])
    strides = [0] * (4 - t.dim()) + list(t.stride()[:-1])
    return sizes, strides


def dense_like_layout(x: torch.Tensor) -> torch.Tensor:
    """An uninitialised tensor of x's shape whose memory order follows x's strides
    (largest stride outermost) but without x's gaps."""
    order = sorted(range(x.dim()), key=lambda d: (-x.stride(d), d))
    buf = torch.empty([x.shape[d] for d in order], dtype=x.dtype, device=x.device)
    inv = [order.index(d) for d in range(x.dim())]
    return buf.permute(inv)


def rmsnorm_forward_strided(x, weight, eps: float):
    """x: any view (<= 4-D, contiguous last dim, 16-byte aligned strides); out is contiguous."""
    if not x.is_cuda or not weight.is_cuda or not weight.is_contiguous():
        raise ValueError("tensors must live on the GPU and weight must be contiguous")
    cols = weight.numel()
    (n0, n1, n2), (s0, s1, s2) = _view3(x)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    rstd = torch.empty(n0 * n1 * n2, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _check(lib().tt_rmsnorm_forward_strided(_p(out), _p(rstd), _p(x), _p(weight), n0, n1, n2, s0, s1, s2,
                                                cols, eps, _dt(x), _stream(x)), "tt_rmsnorm_forward_strided")
    return out, rstd


def rmsnorm_backward_strided(dout, x, weight, rstd, dx=None):
    """dout contiguous; x a view as in rmsnorm_forward_strided; dx (optional) any view of x's shape."""
    _dense_gpu(dout, weight, rstd)
    cols = weight.numel()
    (n0, n1, n2), (s0, s1, s2) = _view3(x)
    dx = dense_like_layout(x) if dx is None else dx
    _, (d0, d1, d2) = _view3(dx)
    dweight = torch.empty_like(weight)
    with torch.cuda.device(x.device):
        L = lib()
        n = L.tt_rmsnorm_backward_workspace_bytes(n0 * n1 * n2, cols, _dt(x))
        ws = _workspace(n, x)
        _check(L.tt_rmsnorm_backward_strided(_p(dx), _p(dweight), _p(dout), _p(x), _p(weight), _p(rstd),
                                             n0, n1, n2, s0, s1, s2, d0, d1, d2, cols, _dt(x), _p(ws), n,
                                             _stream(x)), "tt_rmsnorm_backward_strided")
    return dx, dweight


def copy_rows_strided(dst, src):
    """src contiguous; dst any view (<= 4-D, contiguous last dim, 16-byte aligned strides) of src's shape."""
    _dense_gpu(src)
    if dst.shape != src.shape or dst.dtype != src.dtype or not dst.is_cuda:
        raise ValueError("dst must be a GPU view of src's shape and dtype")
    (n0, n1, n2), (d0, d1, d2) = _view3(dst)
    with torch.cuda.device(src.device):
        _check(lib().tt_norm_copy_rows_strided(_p(dst), _p(src), n0, n1, n2, d0, d1, d2, src.shape[-1], _dt(src),
                                               _stream(src)), "tt_norm_copy_rows_strided")
    return dst


def rmsnorm_rope_forward_strided(x, weight, cos, sin, eps: float):
    """rmsnorm_forward_strided followed by the rotary embedding on tokens < cos.shape[0]; x is [..., S, D]."""
    if not x.is_cuda or not weight.is_cuda or not weight.is_contiguous():
        raise ValueError("tensors must live on the GPU and weight must be contiguous")
    cols = weight.numel()
    (n0, n1, n2), (s0, s1, s2) = _view3(x)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    rstd = torch.empty(n0 * n1 * n2, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _check(lib().tt_rmsnorm_rope_forward_strided(_p(out), _p(rstd), _p(x), _p(weight), _p(cos), _p(sin),
                                                     cos.shape[0], n0, n1, n2, s0, s1, s2, cols, eps, _dt(x),
                                                     _stream(x)), "tt_rmsnorm_rope_forward_strided")
    return out, rstd


def rmsnorm_rope_backward_strided(dout, x, weight, rstd, cos, sin, dx=None):
    """dout: gradient of the rotated output (contiguous); returns (dx, dweight) of the norm."""
    _dense_gpu(dout, weight, rstd)
    cols = weight.numel()
    (n0, n1, n2), (s0, s1, s2) = _view3(x)
    dx = dense_like_layout(x) if dx is None else dx
    _, (d0, d1, d2) = _view3(dx)
    dweight = torch.empty_like(weight)
    with torch.cuda.device(x.device):
        L = lib()
        n = L.tt_rmsnorm_backward_workspace_bytes(n0 * n1 * n2, cols, _dt(x))
        ws = _workspace(n, x)
        _check(L.tt_rmsnorm_rope_backward_strided(_p(dx), _p(dweight), _p(dout), _p(x), _p(weight), _p(rstd),
                                                  _p(cos), _p(sin), cos.shape[0], n0, n1, n2, s0, s1, s2, d0, d1,
                                                  d2, cols, _dt(x), _p(ws), n, _stream(x)),
               "tt_rmsnorm_rope_backward_strided")
    return dx, dweight


def adaln_forward(x, scale, shift, eps: float, want_xnorm: bool = False, seq_first: bool = False):
    """x [B, S, C] (or [rows, C] with scale [1, C]; [S, B, C] with seq_first); returns (out, mean, rstd) or
    (out, x_norm, rstd) when want_xnorm."""
    _dense_gpu(x, scale, shift)
    cols = x.shape[-1]
    batch = scale.numel() // cols
    rows = x.numel() // cols
    if rows % batch:
        raise ValueError("rows not divisible by batch")
    out = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        if want_xnorm:
            xn = torch.empty_like(x)
            _check(lib().tt_adaln_forward_xnorm(_p(out), _p(xn), _p(rstd), _p(x), _p(scale), _p(shift), batch,
                                                rows // batch, cols, eps, _dt(x), _stream(x)),
                   "tt_adaln_forward_xnorm")
            return out, xn, rstd
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        fn = lib().tt_adaln_forward_seq_first if seq_first else lib().tt_adaln_forward
        _check(fn(_p(out), _p(mean), _p(rstd), _p(x), _p(scale), _p(shift), batch,
                  rows // batch, cols, eps, _dt(x), _stream(x)), "tt_adaln_forward")
    return out, mean, rstd


def adaln_backward(dout, x, scale, mean, rstd, from_xnorm: bool = False, seq_first: bool = False):
    _dense_gpu(dout, x, scale, rstd)
    cols = x.shape[-1]
    batch = scale.numel() // cols
    rows = x.numel() // cols
    dx = torch.empty_like(x)
    dscale = torch.empty_like(scale)
    dshift = torch.empty_like(scale)
    with torch.cuda.device(x.device):
        L = lib()
        n = L.tt_adaln_backward_workspace_bytes(batch, rows // batch, cols, _dt(x))
        ws = _workspace(n, x)
        if from_xnorm:
            _check(L.tt_adaln_backward_from_xnorm(_p(dx), _p(dscale), _p(dshift), _p(dout), _p(x), _p(scale),
                                                  _p(rstd), batch, rows // batch, cols, _dt(x), _p(ws), n,
                                                  _stream(x)), "tt_adaln_backward_from_xnorm")
        else:
            fn = L.tt_adaln_backward_seq_first if seq_first else L.tt_adaln_backward
            _check(fn(_p(dx), _p(dscale), _p(dshift), _p(dout), _p(x), _p(scale), _p(mean),
                      _p(rstd), batch, rows // batch, cols, _dt(x), _p(ws), n, _stream(x)),
                   "tt_adaln_backward")
    return dx, dscale, dshift


def adaln_backward_residual(dout, dres, x, scale, mean, rstd):
    """AdaLN backward with the input's other gradient added in: returns (dx + dres, dscale, dshift)."""
    _dense_gpu(dout, dres, x, scale, mean, rstd)
    cols = x.shape[-1]
    batch = scale.numel() // cols
    rows = x.numel() // cols
    dx = torch.empty_like(x)
    dscale = torch.empty_like(scale)
    dshift = torch.empty_like(scale)
    with torch.cuda.device(x.device):
        L = lib()
        n = L.tt_adaln_backward_workspace_bytes(batch, rows // batch, cols, _dt(x))
        ws = _workspace(n, x)
        _check(L.tt_adaln_backward_residual(_p(dx), _p(dscale), _p(dshift), _p(dout), _p(dres), _p(x), _p(scale),
                                            _p(mean), _p(rstd), batch, rows // batch, cols, _dt(x), _p(ws), n,
                                            _stream(x)), "tt_adaln_backward_residual")
    return dx, dscale, dshift


def gated_residual_adaln_forward(h, attn, gate, scale, shift, eps: float):
    """h2 = h + attn*gate[b]; out = AdaLN(h2).  Returns (h2, out, mean, rstd)."""
    _dense_gpu(h, attn, gate, scale, shift)
    cols = h.shape[-1]
    batch = scale.numel() // cols
    rows = h.numel() // cols
    if rows % batch:
        raise ValueError("rows not divisible by batch")
    h2 = torch.empty_like(h)
    out = torch.empty_like(h)
    mean = torch.empty(rows, dtype=torch.float32, device=h.device)
    rstd = torch.empty(rows, dtype=torch.float32, device=h.device)
    with torch.cuda.device(h.device):
        _check(lib().tt_gated_residual_adaln_forward(_p(h2), _p(out), _p(mean), _p(rstd), _p(h), _p(attn),
                                                     _p(gate), _p(scale), _p(shift), batch, rows // batch, cols,
                                                     eps, _dt(h), _stream(h)), "tt_gated_residual_adaln_forward")
    return h2, out, mean, rstd


def gated_residual_adaln_backward(dout, dh2, h2, attn, gate, scale, mean, rstd):
    """Returns (dh, dattn, dgate, dscale, dshift); dh2 may be None."""
    _dense_gpu(dout, h2, attn, gate, scale, mean, rstd)
    if dh2 is not None:
        _dense_gpu(dh2)
    cols = h2.shape[-1]
    batch = scale.numel() // cols
    rows = h2.numel() // cols
    dh = torch.empty_like(h2)
    dattn = torch.empty_like(h2)
    dgate = torch.empty_like(scale)
    dscale = torch.empty_like(scale)
    dshift = torch.empty_like(scale)
    with torch.cuda.device(h2.device):
        L = lib()
        n = L.tt_gated_residual_adaln_backward_workspace_bytes(batch, rows // batch, cols, _dt(h2))
        ws = _workspace(n, h2)
        _check(L.tt_gated_residual_adaln_backward(_p(dh), _p(dattn), _p(dgate), _p(dscale), _p(dshift), _p(dout),
                                                  _p(dh2), _p(h2), _p(attn), _p(gate), _p(scale), _p(mean),
                                                  _p(rstd), batch, rows // batch, cols, _dt(h2), _p(ws), n,
                                                  _stream(h2)), "tt_gated_residual_adaln_backward")
    return dh, dattn, dgate, dscale, dshift
