"""ctypes loader for the scalar C restatement (oracle/norm_oracle_c.c).
TEST INFRASTRUCTURE ONLY -- see the header of norm_oracle.py."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnorm_oracle_c.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "norm_oracle_c.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnorm_oracle_c.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _ptr(t: torch.Tensor):
    assert t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def _sfx(dtype):
    return {torch.bfloat16: "bf16", torch.float32: "f32"}[dtype]


def rmsnorm_fwd(x: torch.Tensor, w: torch.Tensor, eps: float):
    cols = x.shape[-1]
    rows = x.numel() // cols
    out = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32)
    fn = getattr(lib(), f"oc_rmsnorm_fwd_{_sfx(x.dtype)}")
    fn(_ptr(x), _ptr(w), _ptr(out), _ptr(rstd), ctypes.c_long(rows), ctypes.c_long(cols),
       ctypes.c_double(eps))
    return out, rstd


def rmsnorm_bwd(x, w, rstd, g):
    cols = x.shape[-1]
    rows = x.numel() // cols
    dx = torch.empty_like(x)
    dw = torch.empty_like(w)
    acc = np.empty(cols, dtype=np.float64)
    fn = getattr(lib(), f"oc_rmsnorm_bwd_{_sfx(x.dtype)}")
    fn(_ptr(x), _ptr(w), _ptr(rstd), _ptr(g), _ptr(dx), _ptr(dw),
       acc.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(rows), ctypes.c_long(cols))
    return dx, dw


def adaln_fwd(x, scale, shift, eps: float):
    B, S, C = x.shape
    out = torch.empty_like(x)
    mean = torch.empty(B * S, dtype=torch.float32)
    rstd = torch.empty(B * S, dtype=torch.float32)
    fn = getattr(lib(), f"oc_adaln_fwd_{_sfx(x.dtype)}")
    fn(_ptr(x), _ptr(scale), _ptr(shift), _ptr(out), _ptr(mean), _ptr(rstd),
       ctypes.c_long(B), ctypes.c_long(S), ctypes.c_long(C), ctypes.c_double(eps))
    return out, mean, rstd


def adaln_bwd(x, scale, mean, rstd, g):
    B, S, C = x.shape
    dx = torch.empty_like(x)
    dscale = torch.empty_like(scale)
    dshift = torch.empty_like(scale)
    acc = np.empty(2 * C, dtype=np.float64)
    fn = getattr(lib(), f"oc_adaln_bwd_{_sfx(x.dtype)}")
    fn(_ptr(x), _ptr(scale), _ptr(mean), _ptr(rstd), _ptr(g), _ptr(dx), _ptr(dscale), _ptr(dshift),
       acc.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(B), ctypes.c_long(S), ctypes.c_long(C))
    return dx, dscale, dshift


def gated_residual_adaln_fwd(h, attn, gate, scale, shift, eps: float):
    """bf16 only.  Returns (h2, out, mean, rstd)."""
    assert h.dtype == torch.bfloat16
    B, S, C = h.shape
    h2 = torch.empty_like(h)
    lib().oc_gated_residual_fwd_bf16(_ptr(h), _ptr(attn), _ptr(gate), _ptr(h2), ctypes.c_long(B), ctypes.c_long(S),
                                     ctypes.c_long(C))
    out, mean, rstd = adaln_fwd(h2, scale, shift, eps)
    return h2, out, mean, rstd


def gated_residual_adaln_bwd(h2, attn, gate, scale, mean, rstd, grad_out, grad_h2=None):
    """bf16 only.  Returns (dh, dattn, dgate, dscale, dshift)."""
    B, S, C = h2.shape
    dxn, dscale, dshift = adaln_bwd(h2, scale, mean, rstd, grad_out)
    dh, dattn, dgate = torch.empty_like(h2), torch.empty_like(h2), torch.empty_like(gate)
    acc = np.empty(C, dtype=np.float64)
    lib().oc_gated_residual_bwd_bf16(_ptr(dxn), None if grad_h2 is None else _ptr(grad_h2), _ptr(attn), _ptr(gate),
                                     _ptr(dh), _ptr(dattn), _ptr(dgate), acc.ctypes.data_as(ctypes.c_void_p),
                                     ctypes.c_long(B), ctypes.c_long(S), ctypes.c_long(C))
    return dh, dattn, dgate, dscale, dshift
