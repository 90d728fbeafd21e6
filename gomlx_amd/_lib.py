"""ctypes binding of libgomlx_hipq.so (the C ABI declared in include/gomlx_hipq.h).

There is no fallback: if the shared library has not been built, importing symbols from it
raises.  Build it with ``python -m gomlx_amd.build``.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgomlx_hipq.so")


def use_library(path: str) -> None:
    """Loads `path` instead of the in-tree product library; only before the first call of lib().  For the benchmark's
    timing-only ablation builds, which export the same symbols."""
    global LIB_PATH
    if _lib is not None:
        raise RuntimeError("the library is already loaded")
    LIB_PATH = path

OK, ERR_INVALID, ERR_NOT_IMPLEMENTED, ERR_HIP, ERR_NO_DEVICE, ERR_OOM = range(6)
F32, BF16 = 0, 1

# Every symbol include/gomlx_hipq.h declares: (name, restype, argtypes).
_vp, _i64, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
_pint = ctypes.POINTER(ctypes.c_int)
SIGNATURES = [
    ("gq_abi_version", _int, []),
    ("gq_bytes_per_block", _int, [_int]),
    ("gq_values_per_block", _int, [_int]),
    ("gq_row_bytes", _sz, [_int, _i64]),
    ("gq_qdense_check", _int, [_int, _int, _i64, _i64, _i64, _i64, _i64, _int, ctypes.POINTER(_i64)]),
    ("gq_device_count", _int, [_pint]),
    ("gq_init", _int, [_int]),
    ("gq_device_name", _int, [ctypes.c_char_p, _sz]),
    ("gq_malloc", _int, [ctypes.POINTER(_vp), _sz]),
    ("gq_free", _int, [_vp]),
    ("gq_h2d", _int, [_vp, _vp, _sz, _vp]),
    ("gq_d2h", _int, [_vp, _vp, _sz, _vp]),
    ("gq_stream_create", _int, [ctypes.POINTER(_vp)]),
    ("gq_stream_destroy", _int, [_vp]),
    ("gq_sync", _int, [_vp]),
    ("gq_dequantize", _int, [_int, _vp, _i64, _i64, _vp, _vp]),
    ("gq_qdense_f32", _int, [_int, _vp, _i64, _i64, _vp, _i64, _vp, _int, _vp, _vp]),
    ("gq_qdense_f32_static", _int, [_int, _vp, _i64, _i64, _vp, _i64, _vp, _int, _vp, _vp]),
    ("gq_qdense_f32_batch", _int, [_int, _vp, _vp]),
    ("gq_qdense_bf16", _int, [_int, _vp, _i64, _i64, _vp, _i64, _vp, _int, _vp, _vp]),
    ("gq_rmsnorm_f32", _int, [_vp, _i64, _i64, _vp, ctypes.c_float, ctypes.c_float, _vp, _vp]),
    ("gq_qdense_block_f32", _int, [_int, _vp, _i64, _i64, _vp, _vp, _i64, _vp, _int, _vp, _vp, _vp]),
    ("gq_qdense_norm_f32_batch", _int, [_int, _vp, _vp, _vp]),
    ("gq_qdense_gated_f32", _int, [_int, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp, _vp]),
    ("gq_qdense_block_bf16", _int, [_int, _vp, _i64, _i64, _vp, _vp, _i64, _vp, _int, _vp, _vp, _vp]),
    ("gq_qdense_norm_bf16_batch", _int, [_int, _vp, _vp, _vp]),
    ("gq_qdense_gated_bf16", _int, [_int, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp, _vp]),
    ("gq_embedding_lookup", _int, [_int, _vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
    ("gq_graph_begin", _int, [_vp]),
    ("gq_graph_end", _int, [_vp, ctypes.POINTER(_vp)]),
    ("gq_graph_launch", _int, [_vp, _vp]),
    ("gq_graph_destroy", _int, [_vp]),
    ("gq_profile_begin", _int, []),
    ("gq_profile_end", _int, [_pint, ctypes.POINTER(ctypes.c_double)]),
    ("gq_workspace_stats", _int, [ctypes.POINTER(_sz), _pint]),
    ("gq_last_error", ctypes.c_char_p, []),
]


class DenseDesc(ctypes.Structure):
    """gq_dense_desc of include/gomlx_hipq.h."""
    _fields_ = [("type", _int), ("act", _int), ("dX", _vp), ("M", _i64), ("K", _i64), ("dW", _vp), ("N", _i64),
                ("dBias", _vp), ("dY", _vp)]


class RmsNormDesc(ctypes.Structure):
    """gq_rmsnorm of include/gomlx_hipq.h."""
    _fields_ = [("dGain", _vp), ("eps", ctypes.c_float), ("gain_offset", ctypes.c_float)]


class HipqError(RuntimeError):
    """A hard failure reported by the library (anything but NOT_IMPLEMENTED)."""

    def __init__(self, status: int, message: str):
        super().__init__(f"gomlx_hipq status {status}: {message}")
        self.status = status


class NotImplementedByBackend(HipqError):
    """Counterpart of compute.ErrNotImplemented: callers may fall back to a decomposed path
    (core/graph/fused_ops.go:357-363 of the reference)."""


_lib = None
_initialised = False


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP library first (python -m gomlx_amd.build); "
                "there is no CPU fallback")
        L = ctypes.CDLL(LIB_PATH)
        for name, restype, argtypes in SIGNATURES:
            fn = getattr(L, name)  # raises AttributeError if the symbol is not exported
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


def check(status: int) -> None:
    if status == OK:
        return
    msg = lib().gq_last_error().decode("utf-8", "replace")
    if status == ERR_NOT_IMPLEMENTED:
        raise NotImplementedByBackend(status, msg)
    raise HipqError(status, msg)


def init(device: int = 0) -> None:
    """gq_init once per process; raises if there is no gfx950 device."""
    global _initialised
    if not _initialised:
        check(lib().gq_init(device))
        _initialised = True
