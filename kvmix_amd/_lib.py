"""ctypes loader for libkvmix_hip.so (the C ABI declared in include/kvmix_hip.h).

There is no fallback: if the shared library is missing the import of the operators
fails with an error that says how to build it."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkvmix_hip.so")

OK = 0
F16, F32 = 0, 1
FMT_REF, FMT_DENSE3, FMT_REF3_WRAP = 0, 1, 2
SCALE_RECIPROCAL, SCALE_DIVIDE = 0, 1

EXPORTS = (
    "kvmix_version",
    "kvmix_strerror",
    "kvmix_quant_pack_last_dim",
    "kvmix_quant_pack_key_tokens",
    "kvmix_quant_pack_kv_flush",
    "kvmix_gemv_workspace_bytes",
    "kvmix_quantized_gemv",
)

_lib = None


class KeyFlush(ctypes.Structure):
    """kvmix_key_flush_t"""
    _fields_ = [("k", ctypes.c_void_p), ("outer", ctypes.c_int64), ("n", ctypes.c_int64), ("D", ctypes.c_int64),
                ("k_outer_stride", ctypes.c_int64), ("k_token_stride", ctypes.c_int64),
                ("group", ctypes.c_int), ("bits", ctypes.c_int), ("fmt", ctypes.c_int), ("scale_mode", ctypes.c_int),
                ("code", ctypes.c_void_p), ("code_outer_stride", ctypes.c_int64), ("code_inner_stride", ctypes.c_int64),
                ("scale", ctypes.c_void_p), ("zero", ctypes.c_void_p),
                ("sz_outer_stride", ctypes.c_int64), ("sz_inner_stride", ctypes.c_int64)]


class ValueFlush(ctypes.Structure):
    """kvmix_value_flush_t"""
    _fields_ = [("x", ctypes.c_void_p), ("outer", ctypes.c_int64), ("inner", ctypes.c_int64), ("steps", ctypes.c_int64),
                ("x_outer_stride", ctypes.c_int64), ("x_inner_stride", ctypes.c_int64),
                ("group", ctypes.c_int), ("bits", ctypes.c_int), ("fmt", ctypes.c_int), ("scale_mode", ctypes.c_int),
                ("code", ctypes.c_void_p), ("code_outer_stride", ctypes.c_int64), ("code_inner_stride", ctypes.c_int64),
                ("scale", ctypes.c_void_p), ("zero", ctypes.c_void_p),
                ("sz_outer_stride", ctypes.c_int64), ("sz_inner_stride", ctypes.c_int64)]


class KVmixLibraryMissing(ImportError):
    pass


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KVmixLibraryMissing(
            f"{LIB_PATH} is not built; run `python -m kvmix_amd.build_ext` (needs hipcc). "
            "The KVmix operators have no CPU or PyTorch fallback."
        )
    L = ctypes.CDLL(LIB_PATH)
    i64, i32, vp, sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
    L.kvmix_version.restype = i32
    L.kvmix_strerror.restype = ctypes.c_char_p
    L.kvmix_strerror.argtypes = [i32]
    L.kvmix_quant_pack_last_dim.restype = i32
    L.kvmix_quant_pack_last_dim.argtypes = [vp, i32, i64, i64, i64, i64, i64, i32, i32, i32, i32,
                                            vp, i64, i64, vp, vp, i64, i64, vp]
    L.kvmix_quant_pack_key_tokens.restype = i32
    L.kvmix_quant_pack_key_tokens.argtypes = [vp, i64, i64, i64, i64, i64, i32, i32, i32, i32,
                                              vp, i64, i64, vp, vp, i64, i64, vp]
    L.kvmix_quant_pack_kv_flush.restype = i32
    L.kvmix_quant_pack_kv_flush.argtypes = [ctypes.POINTER(KeyFlush), ctypes.POINTER(ValueFlush), vp]
    L.kvmix_gemv_workspace_bytes.restype = sz
    L.kvmix_gemv_workspace_bytes.argtypes = [i64, i64, i64, i64]
    L.kvmix_quantized_gemv.restype = i32
    L.kvmix_quantized_gemv.argtypes = [i32, vp, i64, i64, vp, i64, i64, vp, vp, i64, i64, i32, i32,
                                       i64, i32, i64, i64, i64, vp, i64, i64, vp, sz, vp]
    _lib = L
    return L


def strerror(code: int) -> str:
    return load().kvmix_strerror(code).decode()


def check(code: int) -> None:
    """Turn a non-zero C-ABI return code into the RuntimeError the reference raises."""
    if code != OK:
        raise RuntimeError(strerror(code))
