"""ctypes view of libteletron_probe.so (include/teletron_probe.h): plain streaming kernels for
measurement.  Used by bench.py and by the tests of the probes themselves; the operators
(capi.py, fusedlayers.py, the extension modules) never load it."""
from __future__ import annotations

import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libteletron_probe.so")
EXPORTS = ("tt_probe_abi_version", "tt_probe_last_error", "tt_probe_stream_copy", "tt_probe_stream")

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(f"{_LIB_PATH} is not built; run `python -m teletron_amd.build`")
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.tt_probe_abi_version.restype = ci
        L.tt_probe_last_error.restype = ctypes.c_char_p
        L.tt_probe_stream_copy.argtypes = [vp, vp, sz, vp]
        L.tt_probe_stream.argtypes = [vp, sz, vp, sz, vp, sz, sz, ci, ci, ci, ci, ci, vp]
        _lib = L
    return _lib


class ProbeError(RuntimeError):
    def __init__(self, status: int, what: str):
        super().__init__(f"{what}: status {status} ({lib().tt_probe_last_error().decode()})")
        self.status = status


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _nbytes(t):
    return 0 if t is None else t.numel() * t.element_size()


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def stream_copy(dst: torch.Tensor, src: torch.Tensor):
    """dst[:] = src as a plain 16-byte-per-lane streaming copy (both contiguous, on the GPU)."""
    if not (dst.is_cuda and src.is_cuda and dst.is_contiguous() and src.is_contiguous()):
        raise ValueError("tensors must be contiguous and on the GPU")
    if _nbytes(dst) < _nbytes(src):
        raise ValueError("dst is shorter than src")
    with torch.cuda.device(src.device):
        st = lib().tt_probe_stream_copy(_p(dst), _p(src), _nbytes(src), _stream(src))
    if st != 0:
        raise ProbeError(st, "tt_probe_stream_copy")


def stream(dst, a, b, nbytes: int, reads: int, writes: int, accesses_per_lane: int, persistent_blocks: int = 0,
           write_through: bool = False):
    """One probe launch; dst, a, b are the three allocations (a, b may be None when not read)."""
    with torch.cuda.device(dst.device):
        st = lib().tt_probe_stream(_p(dst), _nbytes(dst), _p(a), _nbytes(a), _p(b), _nbytes(b), nbytes, reads, writes,
                                   accesses_per_lane, persistent_blocks, int(bool(write_through)), _stream(dst))
    if st != 0:
        raise ProbeError(st, "tt_probe_stream")
