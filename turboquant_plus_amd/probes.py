"""Measurement probes for bench.py (libtq_probe.so, csrc/tq_probe.h): plain streaming launches and
back-to-back MFMAs whose sustained rates are set beside the published peaks.  Not part of the codec and
not exported by the package; the reference has no counterpart."""
from __future__ import annotations

import ctypes as C
import os

from . import _lib as L

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtq_probe.so")
MAX_ITERS = 1_000_000
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C turboquant_plus_amd/csrc`")
        h = C.CDLL(LIB_PATH)
        h.tq_probe_stream.restype, h.tq_probe_stream.argtypes = C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                                                          C.c_int64, C.c_void_p]
        h.tq_probe_flat.restype, h.tq_probe_flat.argtypes = C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int,
                                                                      C.c_void_p]
        h.tq_probe_mfma_f16.restype, h.tq_probe_mfma_f16.argtypes = C.c_int64, [C.c_int64, C.c_void_p, C.c_void_p]
        _lib = h
    return _lib


def probe_stream(mode: str, src, dst, chunked: bool = False):
    """One launch of the streaming probe: "read" src, "write" dst or "copy" src to dst, or the same with the
    non-temporal hint ("read_nt", "write_nt", "copy_nt") (uint8 device
    tensors of equal size, a multiple of 16 bytes); chunked gives every workgroup one contiguous slice
    instead of striding all lanes over the buffer.  The caller times it."""
    code = {"read": 0, "write": 1, "copy": 2, "write_nt": 3, "read_nt": 4, "copy_nt": 5}[mode]
    ref = dst if src is None else src
    nbytes = 0 if ref is None else ref.numel()
    rc = lib().tq_probe_stream(code, int(chunked), None if src is None else L.ptr(src),
                               None if dst is None else L.ptr(dst), nbytes, L.stream_ptr())
    if rc:
        raise ValueError(f"tq_probe_stream: bad argument (mode {mode}, {nbytes} bytes)") if rc == -1 else RuntimeError("HIP error")


def probe_flat(src, dst, units: int, write_64ths: int, nontemporal: bool = True):
    """One launch of the flat probe: `units` short-lived workgroups in dispatch order, each reading 16 KB of src
    (None: no reads) and writing write_64ths/64 of 16 KB of dst (0: no writes).  uint8 device tensors of at least
    units * 16 KB and units * 256 * write_64ths bytes.  The caller times it."""
    if src is not None and src.numel() < units * 16384:
        raise ValueError("probe_flat: src too small")
    if write_64ths and (dst is None or dst.numel() < units * 256 * write_64ths):
        raise ValueError("probe_flat: dst too small")
    rc = lib().tq_probe_flat(None if src is None else L.ptr(src), None if dst is None else L.ptr(dst), units, write_64ths,
                             int(nontemporal), L.stream_ptr())
    if rc:
        raise ValueError("tq_probe_flat: bad argument") if rc == -1 else RuntimeError("HIP error")


def probe_mfma_f16(iters: int, sink) -> int:
    """One launch of the MFMA probe (fp16 32x32x16, eight independent accumulators per wavefront on
    every SIMD); returns the floating-point operations launched.  sink: a float32 device tensor."""
    flops = int(lib().tq_probe_mfma_f16(iters, L.ptr(sink), L.stream_ptr()))
    if flops < 0:
        raise ValueError(f"tq_probe_mfma_f16: iters must be in 1..{MAX_ITERS} and sink non-null") if flops == -1 else RuntimeError("HIP error")
    return flops
