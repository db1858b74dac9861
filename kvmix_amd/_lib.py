"""ctypes loader for libkvmix_hip.so (the C ABI declared in include/kvmix_hip.h).

There is no fallback: if the shared library is missing the import of the operators
fails with an error that says how to build it."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# KVMIX_HIP_LIB names another build of the same library (a build under test: its dispatch can be checked on the
# CPU with tests/test_gemv_plan_cpu.py before it is run on a GPU)
LIB_PATH = os.environ.get("KVMIX_HIP_LIB") or os.path.join(_HERE, "libkvmix_hip.so")

OK = 0
F16, F32 = 0, 1
FMT_REF, FMT_DENSE3, FMT_REF3_WRAP = 0, 1, 2
SCALE_RECIPROCAL, SCALE_DIVIDE = 0, 1
GEMV_STATIC_SCRATCH_BYTES = 2 << 20  # KVMIX_GEMV_STATIC_SCRATCH_BYTES

EXPORTS = (
    "kvmix_version",
    "kvmix_strerror",
    "kvmix_quant_pack_last_dim",
    "kvmix_quant_pack_key_tokens",
    "kvmix_quant_pack_kv_flush",
    "kvmix_quant_pack_kv_flush_batch",
    "kvmix_gemv_workspace_bytes",
    "kvmix_quantized_gemv",
    "kvmix_quantized_gemv_static",
    "kvmix_quantized_gemv_plan",
    "kvmix_decode_attention_workspace_bytes",
    "kvmix_decode_attention",
    "kvmix_decode_attention_fused_supported",
    "kvmix_decode_attention_fused_workspace_bytes",
    "kvmix_decode_attention_fused",
    "kvmix_decode_attention_fused_plan",
    "kvmix_rope_append",
    "kvmix_probe_stream_read",
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


class DecodeAttn(ctypes.Structure):
    """kvmix_decode_attn_t"""
    _i64, _i32, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    _fields_ = [("q", _vp), ("q_stride", _i64),
                ("k_code", _vp), ("k_code_batch_stride", _i64), ("k_code_row_stride", _i64),
                ("k_scale", _vp), ("k_zero", _vp), ("k_sz_batch_stride", _i64), ("k_sz_row_stride", _i64),
                ("k_bits", _i32), ("k_fmt", _i32), ("k_group", _i32), ("k_tokens", _i64),
                ("v_code", _vp), ("v_code_batch_stride", _i64), ("v_code_row_stride", _i64),
                ("v_scale", _vp), ("v_zero", _vp), ("v_sz_batch_stride", _i64), ("v_sz_row_stride", _i64),
                ("v_bits", _i32), ("v_fmt", _i32), ("v_group", _i32), ("v_tokens", _i64),
                ("k_tail", _vp), ("k_tail_batch_stride", _i64), ("k_tail_token_stride", _i64),
                ("k_tail_slots", _i64), ("k_tail_len", _i64), ("k_tail_len_dev", _vp),
                ("v_tail", _vp), ("v_tail_batch_stride", _i64), ("v_tail_token_stride", _i64),
                ("v_tail_slots", _i64), ("v_tail_len", _i64), ("v_tail_len_dev", _vp),
                ("mask", _vp), ("mask_stride", _i64),
                ("samples", _i64), ("heads", _i32), ("heads_per_kv", _i32), ("D", _i64),
                ("probs", _vp), ("probs_stride", _i64), ("out", _vp), ("out_stride", _i64)]


class RopeAppend(ctypes.Structure):
    """kvmix_rope_append_t"""
    _i64, _i32, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    _fields_ = [("qkv", _vp), ("qkv_batch_stride", _i64), ("cos", _vp), ("sin", _vp),
                ("q_out", _vp), ("q_batch_stride", _i64),
                ("k_tail", _vp), ("k_tail_batch_stride", _i64), ("k_tail_head_stride", _i64),
                ("k_tail_token_stride", _i64), ("k_tail_slots", _i64), ("k_slot", _i64), ("k_slot_dev", _vp),
                ("v_tail", _vp), ("v_tail_batch_stride", _i64), ("v_tail_head_stride", _i64),
                ("v_tail_token_stride", _i64), ("v_tail_slots", _i64), ("v_slot", _i64), ("v_slot_dev", _vp),
                ("batch", _i64), ("heads", _i32), ("kv_heads", _i32), ("D", _i64)]


class GemvPlan(ctypes.Structure):
    """kvmix_gemv_plan_t"""
    _fields_ = [("kernel", ctypes.c_char * 64), ("grid", ctypes.c_uint * 3), ("block", ctypes.c_uint * 3),
                ("lds_bytes", ctypes.c_uint64), ("splits", ctypes.c_int), ("ksplit", ctypes.c_int),
                ("launches", ctypes.c_int)]


class AttnPlan(ctypes.Structure):
    """kvmix_attn_plan_t"""
    _fields_ = [("matrix", ctypes.c_int), ("recommended", ctypes.c_int), ("launches", ctypes.c_int), ("matrix_tiles", ctypes.c_int64),
                ("matrix_tile_waves", ctypes.c_int), ("slab_positions", ctypes.c_int64), ("slab_begin", ctypes.c_int64), ("slabs", ctypes.c_int64),
                ("slab_blocks", ctypes.c_int64), ("matrix_grid", ctypes.c_uint * 3), ("matrix_block", ctypes.c_uint * 3)]


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
    L.kvmix_quant_pack_kv_flush_batch.restype = i32
    L.kvmix_quant_pack_kv_flush_batch.argtypes = [ctypes.POINTER(ctypes.POINTER(KeyFlush)),
                                                  ctypes.POINTER(ctypes.POINTER(ValueFlush)), ctypes.c_int, vp]
    L.kvmix_gemv_workspace_bytes.restype = sz
    L.kvmix_gemv_workspace_bytes.argtypes = [i64, i64, i64, i64]
    L.kvmix_quantized_gemv.restype = i32
    L.kvmix_quantized_gemv.argtypes = [i32, vp, i64, i64, vp, i64, i64, vp, vp, i64, i64, i32, i32,
                                       i64, i32, i64, i64, i64, vp, i64, i64, vp, sz, vp]
    L.kvmix_quantized_gemv_static.restype = i32
    L.kvmix_quantized_gemv_static.argtypes = [i32, vp, i64, i64, vp, i64, i64, vp, vp, i64, i64, i32, i32,
                                              i64, i32, i64, i64, i64, vp, i64, i64, vp]
    L.kvmix_quantized_gemv_plan.restype = i32
    L.kvmix_quantized_gemv_plan.argtypes = [i32, i32, i32, i64, i32, i64, i64, i64, i64, i64, ctypes.POINTER(GemvPlan)]
    L.kvmix_decode_attention_workspace_bytes.restype = sz
    L.kvmix_decode_attention_workspace_bytes.argtypes = [ctypes.POINTER(DecodeAttn)]
    L.kvmix_decode_attention.restype = i32
    L.kvmix_decode_attention.argtypes = [ctypes.POINTER(DecodeAttn), vp, sz, vp]
    L.kvmix_decode_attention_fused_supported.restype = i32
    L.kvmix_decode_attention_fused_supported.argtypes = [ctypes.POINTER(DecodeAttn)]
    L.kvmix_decode_attention_fused_workspace_bytes.restype = sz
    L.kvmix_decode_attention_fused_workspace_bytes.argtypes = [ctypes.POINTER(DecodeAttn)]
    L.kvmix_decode_attention_fused.restype = i32
    L.kvmix_decode_attention_fused.argtypes = [ctypes.POINTER(DecodeAttn), vp, sz, vp]
    L.kvmix_decode_attention_fused_plan.restype = i32
    L.kvmix_decode_attention_fused_plan.argtypes = [ctypes.POINTER(DecodeAttn), ctypes.POINTER(AttnPlan)]
    L.kvmix_rope_append.restype = i32
    L.kvmix_rope_append.argtypes = [ctypes.POINTER(RopeAppend), vp]
    L.kvmix_probe_stream_read.restype = i32
    L.kvmix_probe_stream_read.argtypes = [vp, i32, i64, i64, i32, i32, i32, i32, i32, vp, vp]
    _lib = L
    return L


def gemv_plan(group: int, bits: int, fmt: int, samples: int, heads_per_kv: int, M: int, K: int, N: int,
              code_row_stride: int = None, sz_row_stride: int = None) -> dict:
    """kvmix_quantized_gemv_plan for dense rows (or the given row strides): the kernel a call of these
    sizes gets, as a dict.  Needs no GPU."""
    if code_row_stride is None:
        code_row_stride = N * 3 // 32 if (bits == 3 and fmt == FMT_DENSE3) else (N // 11 if bits == 3 else N * bits // 32)
    if sz_row_stride is None:
        sz_row_stride = N // group
    plan = GemvPlan()
    check(load().kvmix_quantized_gemv_plan(group, bits, fmt, samples, heads_per_kv, M, K, N, code_row_stride,
                                           sz_row_stride, ctypes.byref(plan)))
    return {"kernel": plan.kernel.decode(), "grid": tuple(plan.grid), "block": tuple(plan.block),
            "lds_bytes": plan.lds_bytes, "splits": plan.splits, "ksplit": plan.ksplit, "launches": plan.launches}


def attn_step_descriptor(batch: int, heads: int, kv_heads: int, head_dim: int, k_bits: int, k_fmt: int, k_group: int,
                         k_tokens: int, v_bits: int, v_fmt: int, v_group: int, v_tokens: int, k_tail_slots: int,
                         v_tail_slots: int, k_code_row_stride: int = None, v_code_row_stride: int = None) -> DecodeAttn:
    """A kvmix_decode_attn_t that carries the sizes of a step over dense operands and no pointers: what the
    plan and support queries read."""
    st = DecodeAttn()
    D = head_dim
    st.samples, st.heads, st.heads_per_kv, st.D = batch * heads, heads, heads // kv_heads, D
    st.q_stride = st.out_stride = D
    st.k_bits, st.k_fmt, st.k_group, st.k_tokens = k_bits, k_fmt, k_group, k_tokens
    ref3 = k_bits == 3 and k_fmt == FMT_REF
    words = k_tokens // 11 if ref3 else k_tokens * k_bits // 32
    st.k_code_row_stride = words if k_code_row_stride is None else k_code_row_stride
    st.k_code_batch_stride = D * st.k_code_row_stride
    st.k_sz_row_stride = k_tokens // (11 if ref3 else max(k_group, 1))
    st.k_sz_batch_stride = D * st.k_sz_row_stride
    st.v_bits, st.v_fmt, st.v_group, st.v_tokens = v_bits, v_fmt, v_group, v_tokens
    st.v_code_row_stride = D * v_bits // 32 if v_code_row_stride is None else v_code_row_stride
    st.v_code_batch_stride = v_tokens * st.v_code_row_stride
    st.v_sz_row_stride = D // max(v_group, 1)
    st.v_sz_batch_stride = v_tokens * st.v_sz_row_stride
    for prefix, slots in (("k", k_tail_slots), ("v", v_tail_slots)):
        setattr(st, prefix + "_tail_slots", slots)
        setattr(st, prefix + "_tail_len", slots)
        setattr(st, prefix + "_tail_token_stride", D)
        setattr(st, prefix + "_tail_batch_stride", slots * D)
    return st


def attn_plan(step: DecodeAttn) -> dict:
    """kvmix_decode_attention_fused_plan as a dict (raises on the codes the step itself would return).  Needs no GPU."""
    plan = AttnPlan()
    check(load().kvmix_decode_attention_fused_plan(ctypes.byref(step), ctypes.byref(plan)))
    return {"matrix": bool(plan.matrix), "recommended": bool(plan.recommended), "launches": plan.launches, "matrix_tiles": plan.matrix_tiles,
            "matrix_tile_waves": plan.matrix_tile_waves,
            "slab_positions": plan.slab_positions, "slab_begin": plan.slab_begin, "slabs": plan.slabs,
            "slab_blocks": plan.slab_blocks, "matrix_grid": tuple(plan.matrix_grid),
            "matrix_block": tuple(plan.matrix_block)}


def flush_batch(keys, values, stream) -> int:
    """kvmix_quant_pack_kv_flush_batch over sequences of KeyFlush / ValueFlush descriptors; returns the library's code."""
    n = len(keys)
    if n != len(values):
        raise ValueError("as many key as value descriptors")
    ka = (ctypes.POINTER(KeyFlush) * n)(*[ctypes.pointer(k) for k in keys])
    va = (ctypes.POINTER(ValueFlush) * n)(*[ctypes.pointer(v) for v in values])
    return load().kvmix_quant_pack_kv_flush_batch(ka, va, n, stream)


def strerror(code: int) -> str:
    return load().kvmix_strerror(code).decode()


def check(code: int) -> None:
    """Turn a non-zero C-ABI return code into the RuntimeError the reference raises."""
    if code != OK:
        raise RuntimeError(strerror(code))
