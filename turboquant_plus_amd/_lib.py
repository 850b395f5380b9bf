"""ctypes binding of libtq_hip.so (include/tq.h) and the device-buffer plumbing.

There is no CPU implementation behind these calls: when the shared library or
a GPU is missing the entry points raise, they never fall back.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# TQ_HIP_LIBRARY names another build of the same library (the measurement variants that
# `make KNOCKOUT=.. OUT=..` produces); unset, the product library next to this file is loaded.
LIB_PATH = os.environ.get("TQ_HIP_LIBRARY") or os.path.join(_HERE, "libtq_hip.so")

TQ_F16, TQ_F32, TQ_F64 = 0, 1, 2
ROT_DENSE, ROT_WHT = 0, 1
KIND_K, KIND_V = 0, 1
DOMAIN_ROTATED, DOMAIN_ORIGINAL = 0, 1
KFMT_TURBO, KFMT_Q8_0 = 0, 1
ERR_ARG, ERR_UNSUPPORTED, ERR_ALIGN, ERR_HIP = -1, -2, -3, -4


class TQConfig(C.Structure):
    _fields_ = [("d", C.c_int32), ("bits", C.c_int32), ("rotation", C.c_int32), ("norm_correction", C.c_int32),
                ("centroids", C.POINTER(C.c_double)), ("signs1", C.POINTER(C.c_double)),
                ("signs2", C.POINTER(C.c_double)), ("rotation_matrix", C.POINTER(C.c_double)),
                ("projection", C.POINTER(C.c_double)), ("projection_scale", C.c_double)]


class TQAttnParams(C.Structure):
    _fields_ = [("batch", C.c_int32), ("n_q_heads", C.c_int32), ("n_kv_heads", C.c_int32), ("tokens", C.c_int64),
                ("capacity", C.c_int64), ("n_splits", C.c_int32), ("k_format", C.c_int32), ("v_format", C.c_int32),
                ("scale", C.c_float), ("sparse_v_tau", C.c_float), ("tokens_dev", C.c_void_p),
                ("bias_entries", C.c_int32), ("bias_pos", C.c_void_p), ("bias_val", C.c_void_p),
                ("head_dim", C.c_int32)]


_P, _I, _L, _D = C.c_void_p, C.c_int, C.c_int64, C.c_double

# name -> (restype, argtypes); mirrors include/tq.h one to one
PROTOTYPES = {
    "tq_version": (_I, []),
    "tq_last_error": (C.c_char_p, []),
    "tq_device_count": (_I, []),
    "tq_create": (_I, [C.POINTER(_P), C.POINTER(TQConfig)]),
    "tq_destroy": (None, [_P]),
    "tq_fwht": (_I, [_P, _P, _L, C.c_int32, _I, _I, _P]),
    "tq_rotate": (_I, [_P, _P, _P, _L, _I, _I, _I, _P]),
    "tq_nearest_centroid": (_I, [_P, _L, C.POINTER(C.c_double), C.c_int32, _P, _P]),
    "tq_quantize_indices": (_I, [_P, _P, _L, _I, _P, _P, _P, _P]),
    "tq_dequantize_indices": (_I, [_P, _P, _P, _L, _P, _P, _I, _P, _P]),
    "tq_qjl_quantize": (_I, [_P, _P, _L, _I, _P, _P, _P]),
    "tq_qjl_dequantize": (_I, [_P, _P, _P, _D, _L, _P, _P]),
    "tq_pack_bits": (_I, [_P, _L, C.c_int32, _P, _P]),
    "tq_unpack_bits": (_I, [_P, _L, C.c_int32, _P, _P]),
    "tq_pack_indices": (_I, [_P, _L, C.c_int32, _P, _P]),
    "tq_packed_bytes": (_L, [C.c_int32, _L, _L]),
    "tq_store": (_I, [_P, _P, _L, _L, _I, _I, _P, _P]),
    "tq_store_kv": (_I, [_P, _P, _P, _P, _L, _L, _I, _P, _P, _P]),
    "tq_store_kv_cache": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _P, _P, _P]),
    "tq_append": (_I, [_P, _P, _L, _L, _L, _L, _I, _I, _P, _P]),
    "tq_append_kv": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _I, _P, _P, _P]),
    "tq_append_kv_at": (_I, [_P, _P, _P, _P, _L, _P, _L, _L, _I, _P, _P, _P, _P]),
    "tq_append_at": (_I, [_P, _P, _L, _P, _L, _L, _I, _I, _P, _P, _P]),
    "tq_q8_0_append_at": (_I, [_P, _L, _P, _L, _L, _I, _I, _P, _P, _P]),
    "tq_requantize": (_I, [_P, _P, _P, _L, _L, _I, _P, _P]),
    "tq_fork_block_bytes": (_L, [C.c_int32]),
    "tq_export_fork_blocks": (_I, [_P, _P, _L, _L, _I, _P, _P]),
    "tq_import_fork_blocks": (_I, [_P, _P, _L, _L, _I, _P, _P]),
    "tq_fork_row_bytes": (_L, [C.c_int32, C.c_int32]),
    "tq_export_fork_blocks_sized": (_I, [_P, _P, _L, _L, _I, C.c_int32, _P, _P]),
    "tq_import_fork_blocks_sized": (_I, [_P, _P, _L, _L, _I, C.c_int32, _P, _P]),
    "tq_load": (_I, [_P, _P, _L, _L, _I, _P, _I, _I, _P]),
    "tq_load_kv": (_I, [_P, _P, _P, _P, _L, _L, _P, _P, _P]),
    "tq_unpack_codes": (_I, [_P, _P, _L, _L, _I, _P, _P, _P]),
    "tq_store_qjl": (_I, [_P, _P, _L, _L, _I, _P, _P, _P, _P]),
    "tq_q8_0_bytes": (_L, [_L, _L]),
    "tq_q8_0_store": (_I, [_P, _L, _L, _I, _P, _P]),
    "tq_q8_0_unpack": (_I, [_P, _L, _L, _P, _P, _P]),
    "tq_q8_0_store_v": (_I, [_P, _L, _L, _I, _P, _P]),
    "tq_q8_0_unpack_v": (_I, [_P, _L, _L, _P, _P, _P]),
    "tq_q8_0_append": (_I, [_P, _L, _L, _L, _L, _I, _I, _P, _P]),
    "tq_attn_workspace_bytes": (_L, [C.POINTER(TQAttnParams)]),
    "tq_decode_attention": (_I, [_P, _P, C.POINTER(TQAttnParams), _P, _I, _P, _P, _P, _P, _P, _P, _P, _L, _P]),
    "tq_decode_attention_static": (_I, [_P, _P, C.POINTER(TQAttnParams), _P, _I, _P, _P, _P, _P, _P, _P]),
    "tq_score_tile": (_I, [_P, _P, _I, _L, _P, _P, _P, _L, _P, _I, _P, _L, _P]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C turboquant_plus_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().tq_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Map a C return code to the exception the reference API raises."""
    if rc == 0:
        return
    msg = last_error()
    if rc in (ERR_ARG, ERR_ALIGN):
        raise ValueError(msg)
    if rc == ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(f"HIP error: {msg}")


_torch = None


def torch():
    global _torch
    if _torch is None:
        import torch as _t
        _torch = _t
    return _torch


def require_gpu():
    if lib().tq_device_count() < 1:
        raise RuntimeError("no HIP device visible: the TurboQuant kernels need an MI355X (no CPU path exists)")
    return torch().device("cuda")


def dtype_code(t) -> int:
    tt = torch()
    if t.dtype == tt.float16:
        return TQ_F16
    if t.dtype == tt.float32:
        return TQ_F32
    if t.dtype == tt.float64:
        return TQ_F64
    raise TypeError(f"unsupported dtype {t.dtype}")


def torch_dtype(code: int):
    tt = torch()
    return {TQ_F16: tt.float16, TQ_F32: tt.float32, TQ_F64: tt.float64}[code]


def to_device(x, float_ok=(np.float16, np.float32, np.float64)):
    """NumPy array or torch tensor -> contiguous CUDA tensor (floats keep their
    width, everything else becomes float64 as NumPy promotion would)."""
    tt = torch()
    dev = require_gpu()
    if isinstance(x, tt.Tensor):
        t = x.to(dev)
        if t.dtype not in (tt.float16, tt.float32, tt.float64):
            t = t.to(tt.float64)
        return t.contiguous()
    a = np.asarray(x)
    if a.dtype not in [np.dtype(f) for f in float_ok]:
        a = a.astype(np.float64)
    return tt.from_numpy(np.ascontiguousarray(a)).to(dev)


def stream_ptr():
    return C.c_void_p(torch().cuda.current_stream().cuda_stream)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def dbl_ptr(a):
    return a.ctypes.data_as(C.POINTER(C.c_double)) if a is not None else None


class Handle:
    """Owns a tq_handle*; the NumPy tables it was built from stay referenced."""

    def __init__(self, d, bits, centroids, *, signs1=None, signs2=None, rotation=None, projection=None,
                 projection_scale=0.0, norm_correction=True):
        require_gpu()
        keep = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float64)
        self._tables = [keep(centroids), keep(signs1), keep(signs2), keep(rotation), keep(projection)]
        cfg = TQConfig(d=d, bits=bits, rotation=ROT_DENSE if rotation is not None else ROT_WHT,
                       norm_correction=int(bool(norm_correction)),
                       centroids=dbl_ptr(self._tables[0]), signs1=dbl_ptr(self._tables[1]),
                       signs2=dbl_ptr(self._tables[2]), rotation_matrix=dbl_ptr(self._tables[3]),
                       projection=dbl_ptr(self._tables[4]), projection_scale=float(projection_scale))
        h = C.c_void_p()
        check(lib().tq_create(C.byref(h), C.byref(cfg)))
        self.h = h

    def __del__(self):
        h, self.h = getattr(self, "h", None), None
        if h and _lib is not None:
            _lib.tq_destroy(h)
