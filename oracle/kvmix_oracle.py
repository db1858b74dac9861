"""CPU oracle for the KVmix KV-cache hot path -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the product package never does.  Two independent restatements of the
reference arithmetic live here:

* ctypes bindings to ``libkvmix_oracle.so`` (``kvmix_oracle.c``: scalar C, IEEE
  binary32), the primary checker and the timed CPU baseline;
* a vectorised numpy twin of the quantizer / packer / dequantizer
  (``*_np`` functions), written separately so that a slip in one of the two is
  caught by the other.

Reference files followed (relative to the reference tree):
  quant_cuda/csrc/quantization_cuda.cu:540-721        quantize_pack_last_dim
  quant_cuda/csrc/quantization_cuda.cu:298-411        process_key_quantization
  quant_cuda/csrc/quantization_cuda.cu:413-537        process_value_quantization
  quant_cuda/csrc/dequantization_gemv_cuda.cu:7-248   quantized_gemm
  models/modeling_llama_KVmix.py:19-28,68-75,105-211  decode-step attention glue
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkvmix_oracle.so")
_lib = None

SCALE_RECIPROCAL = 0  # (mx-mn) * fp32(1/qmax): ATen CUDA division by a scalar
SCALE_DIVIDE = 1      # (mx-mn) / qmax

_ERRORS = {
    -1: "Supported quantization bits: 1, 2, 3, 4",
    -2: "For 3-bit quantization, group_length must be 11",
    -3: "length must be divisible by group_length / values per word",
    -4: "Total heads must be divisible by KV heads",
    -5: "allocation failed",
}


def build(force: bool = False) -> str:
    """Compile the C oracle next to this file (gcc, a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        L.kvo_quantize_pack_last_dim.argtypes = [vp, i64, i64, i32, i32, i32, vp, vp, vp]
        L.kvo_quantize_pack_last_dim_f16.argtypes = [vp, i64, i64, i32, i32, i32, vp, vp, vp]
        L.kvo_process_key.argtypes = [vp, i64, i64, vp, i64, vp, vp, i64, i32, i32, vp, vp, vp]
        L.kvo_process_value.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, i32, i32, vp, vp, vp]
        L.kvo_quantized_gemm.argtypes = [i32, vp, i64, i64, vp, vp, vp, i32, i64, i32, i64, i64, i64,
                                         i32, vp, vp, vp]
        L.kvo_dequantize.argtypes = [vp, vp, vp, i32, i32, i64, i64, vp]
        L.kvo_unpack_row.argtypes = [vp, i64, i32, vp]
        L.kvo_half_to_float_n.argtypes = [vp, vp, i64]
        L.kvo_float_to_half_n.argtypes = [vp, vp, i64]
        L.kvo_half_to_float.restype = ctypes.c_float
        L.kvo_half_to_float.argtypes = [ctypes.c_uint16]
        L.kvo_float_to_half.restype = ctypes.c_uint16
        L.kvo_float_to_half.argtypes = [ctypes.c_float]
        L.kvo_set_num_threads.argtypes = [i32]
        L.kvo_quantize_pack_dense3.argtypes = [vp, i64, i64, i32, i32, vp, vp, vp]
        L.kvo_unpack_dense3_row.argtypes = [vp, i64, vp]
        L.kvo_quantized_gemm_dense3.argtypes = [i32, vp, i64, i64, vp, vp, vp, i64, i32, i64, i64, i64,
                                                vp, vp, vp]
        _lib = L
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(_ERRORS.get(rc, f"oracle error {rc}"))


def values_per_word(bits: int) -> int:
    return 11 if bits == 3 else 32 // bits


def num_threads() -> int:
    return lib().kvo_num_threads()


def set_num_threads(n: int) -> None:
    lib().kvo_set_num_threads(n)


# ---------------------------------------------------------------------------
# fp16 conversion (exposed so the tests can pin the C routines against numpy)
# ---------------------------------------------------------------------------

def half_to_float(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h).view(np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().kvo_half_to_float_n(_p(h), _p(out), h.size)
    return out


def float_to_half(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().kvo_float_to_half_n(_p(f), _p(out), f.size)
    return out.view(np.float16)


# ---------------------------------------------------------------------------
# quantize_pack_last_dim   (quantization_cuda.cu:631-721)
# ---------------------------------------------------------------------------

def quantize_pack_last_dim(x: np.ndarray, group_length: int, quant_bits: int,
                           scale_mode: int = SCALE_RECIPROCAL
                           ) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """x: 4-D float16 or float32.  Returns (code int32 [..., S/vpw], scale, min) with
    scale/min in x's dtype, as the reference does (fp16 inputs are computed in fp32
    and only the returned scale/min are rounded to fp16)."""
    if quant_bits == 3 and group_length != 11:
        raise RuntimeError(_ERRORS[-2])
    if x.ndim != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    is_half = x.dtype == np.float16
    xf = np.ascontiguousarray(x, dtype=np.float32)
    B, H, R, S = xf.shape
    rows = B * H * R
    vpw = values_per_word(quant_bits) if quant_bits in (1, 2, 3, 4) else 1
    g = max(group_length, 1)
    code = np.zeros((B, H, R, S // vpw), np.int32)
    scale = np.zeros((B, H, R, S // g), np.float32)
    mn = np.zeros((B, H, R, S // g), np.float32)
    _check(lib().kvo_quantize_pack_last_dim(_p(xf), rows, S, group_length, quant_bits, scale_mode,
                                            _p(code), _p(scale), _p(mn)))
    if is_half:
        with np.errstate(over="ignore"):
            scale, mn = scale.astype(np.float16), mn.astype(np.float16)
    return code, scale, mn


def quantize_pack_last_dim_f16_timed(x: np.ndarray, group_length: int, quant_bits: int):
    """All-C fp16 path (up-cast, quantize, pack, down-cast) for CPU-baseline timing."""
    assert x.dtype == np.float16 and x.ndim == 4 and x.flags.c_contiguous
    B, H, R, S = x.shape
    vpw = values_per_word(quant_bits)
    code = np.empty((B, H, R, S // vpw), np.int32)
    scale = np.empty((B, H, R, S // group_length), np.float16)
    mn = np.empty((B, H, R, S // group_length), np.float16)
    _check(lib().kvo_quantize_pack_last_dim_f16(_p(x), B * H * R, S, group_length, quant_bits,
                                                SCALE_RECIPROCAL, _p(code), _p(scale), _p(mn)))
    return code, scale, mn


def round_half_away(v: np.ndarray) -> np.ndarray:
    """roundf(): nearest, ties away from zero, for float32 arrays (NaN stays NaN)."""
    v = np.asarray(v, np.float32)
    t = np.trunc(v)
    frac = np.abs(v - t)  # exact in fp32
    return np.where(frac >= np.float32(0.5), t + np.sign(v).astype(np.float32), t).astype(np.float32)


def pack_np(q: np.ndarray, bits: int) -> np.ndarray:
    """Pack integer codes [..., S] into words [..., S/vpw], value 0 in the low bits.
    3-bit: ten codes at bits 0..29 and the 11th at bits 30..31
    (quantization_cuda.cu:617-625)."""
    vpw = values_per_word(bits)
    q = np.asarray(q).astype(np.uint64)
    q = q.reshape(q.shape[:-1] + (q.shape[-1] // vpw, vpw))
    if bits == 3:
        shifts = np.array([3 * i for i in range(10)] + [30], np.uint64)
    else:
        shifts = (np.arange(vpw) * bits).astype(np.uint64)
    words = np.bitwise_or.reduce(q << shifts, axis=-1) & np.uint64(0xFFFFFFFF)
    return words.astype(np.uint32).view(np.int32)


def unpack_np(code: np.ndarray, bits: int) -> np.ndarray:
    """Inverse of pack_np (unpack order of dequantization_gemv_cuda.cu:81-105)."""
    vpw = values_per_word(bits)
    w = np.ascontiguousarray(code).view(np.uint32).astype(np.uint64)[..., None]
    if bits == 3:
        shifts = np.array([3 * i for i in range(10)] + [30], np.uint64)
        masks = np.array([7] * 10 + [3], np.uint64)
    else:
        shifts = (np.arange(vpw) * bits).astype(np.uint64)
        masks = np.full(vpw, (1 << bits) - 1, np.uint64)
    vals = (w >> shifts) & masks
    return vals.reshape(code.shape[:-1] + (code.shape[-1] * vpw,)).astype(np.int32)


def quantize_pack_last_dim_np(x: np.ndarray, group_length: int, quant_bits: int,
                              scale_mode: int = SCALE_RECIPROCAL):
    """numpy twin of quantize_pack_last_dim (independent of the C code)."""
    if quant_bits == 3 and group_length != 11:
        raise RuntimeError(_ERRORS[-2])
    if x.ndim != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    is_half = x.dtype == np.float16
    xf = x.astype(np.float32)
    B, H, R, S = xf.shape
    if S % group_length or (quant_bits != 3 and S % (32 // quant_bits)):
        raise RuntimeError(_ERRORS[-3])
    qmax = np.float32((1 << quant_bits) - 1)
    xg = xf.reshape(B, H, R, S // group_length, group_length)
    with np.errstate(all="ignore"):
        mn = np.fmin.reduce(xg, axis=-1)
        mx = np.fmax.reduce(xg, axis=-1)
        scale = ((mx - mn) / qmax).astype(np.float32)
        normalized = ((xg - mn[..., None]) / scale[..., None]).astype(np.float32)
        r = round_half_away(normalized)
        r = np.where(np.isnan(r), np.float32(0), r)
        hi = np.full(group_length, qmax, np.float32)
        if quant_bits == 3:
            hi[10] = 3
        q = np.clip(r, 0, hi).astype(np.int64).reshape(B, H, R, S)
        if scale_mode == SCALE_RECIPROCAL:
            scale_out = ((mx - mn) * (np.float32(1.0) / qmax)).astype(np.float32)
        else:
            scale_out = scale
    code = pack_np(q, quant_bits)
    if is_half:
        with np.errstate(over="ignore"):
            scale_out, mn = scale_out.astype(np.float16), mn.astype(np.float16)
    return code, scale_out, mn


# ---------------------------------------------------------------------------
# dense 3-bit stream (extension; no reference counterpart)
# ---------------------------------------------------------------------------

def quantize_pack_dense3(x: np.ndarray, group_length: int = 32, scale_mode: int = SCALE_RECIPROCAL):
    """3-bit codes (qmax 7 everywhere) as a little-endian bit stream: 32 codes in 3 words."""
    if x.ndim != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    is_half = x.dtype == np.float16
    xf = np.ascontiguousarray(x, dtype=np.float32)
    B, H, R, S = xf.shape
    g = max(group_length, 1)
    code = np.zeros((B, H, R, S * 3 // 32), np.int32)
    scale = np.zeros((B, H, R, S // g), np.float32)
    mn = np.zeros_like(scale)
    _check(lib().kvo_quantize_pack_dense3(_p(xf), B * H * R, S, group_length, scale_mode, _p(code),
                                          _p(scale), _p(mn)))
    if is_half:
        scale, mn = scale.astype(np.float16), mn.astype(np.float16)
    return code, scale, mn


def pack_dense3_np(q: np.ndarray) -> np.ndarray:
    """codes [..., S] (0..7) -> words [..., 3S/32]: code i at stream bits [3i, 3i+3)."""
    q = np.asarray(q).astype(np.uint8)
    bits = ((q[..., None] >> np.arange(3, dtype=np.uint8)) & 1).reshape(q.shape[:-1] + (q.shape[-1] * 3,))
    by = np.packbits(bits, axis=-1, bitorder="little")
    return np.ascontiguousarray(by).view(np.uint32).view(np.int32)


def unpack_dense3_np(code: np.ndarray) -> np.ndarray:
    by = np.ascontiguousarray(code).view(np.uint8)
    bits = np.unpackbits(by, axis=-1, bitorder="little")
    bits = bits.reshape(bits.shape[:-1] + (bits.shape[-1] // 3, 3)).astype(np.int32)
    return bits[..., 0] | (bits[..., 1] << 1) | (bits[..., 2] << 2)


def dequantize_dense3_np(code, scales, zeros, group_size=32) -> np.ndarray:
    q = unpack_dense3_np(code).astype(np.float32)
    s = np.repeat(scales.astype(np.float32), group_size, axis=-1)
    z = np.repeat(zeros.astype(np.float32), group_size, axis=-1)
    return (s * q).astype(np.float32) + z


def quantized_gemm_dense3(group_size, fA, qB, scales, zeros, want_f64=False):
    B, nh, M, K = fA.shape
    nh_kv = qB.shape[1]
    if nh % nh_kv:
        raise RuntimeError(_ERRORS[-4])
    N = zeros.shape[-1] * group_size
    a = np.ascontiguousarray(fA, np.float16)
    q = np.ascontiguousarray(qB, np.int32)
    s = np.ascontiguousarray(scales, np.float16)
    z = np.ascontiguousarray(zeros, np.float16)
    out = np.zeros((B, nh, M, N), np.float16)
    o64 = np.zeros((B, nh, M, N), np.float64) if want_f64 else None
    a64 = np.zeros((B, nh, M, N), np.float64) if want_f64 else None
    _check(lib().kvo_quantized_gemm_dense3(group_size, _p(a), M * K, K, _p(q), _p(s), _p(z), B * nh,
                                           nh // nh_kv, M, K, N, _p(out), _p(o64), _p(a64)))
    return (out, o64, a64) if want_f64 else out


# ---------------------------------------------------------------------------
# append variants
# ---------------------------------------------------------------------------

def process_key_quantization(x_new, prev_code, prev_scale, prev_min, group_length, quant_bits):
    """quantization_cuda.cu:298-411.  x_new [B,H,D,n]; prev_* [B,H,D,old]."""
    is_half = x_new.dtype == np.float16
    xf = np.ascontiguousarray(x_new, np.float32)
    ps = np.ascontiguousarray(prev_scale, np.float32)
    pm = np.ascontiguousarray(prev_min, np.float32)
    pc = np.ascontiguousarray(prev_code, np.int32)
    B, H, D, n = xf.shape
    if quant_bits == 3 and group_length != 11:
        raise RuntimeError(_ERRORS[-2])
    vpw = values_per_word(quant_bits)
    ow, og = pc.shape[3], ps.shape[3]
    code = np.zeros((B, H, D, ow + n // vpw), np.int32)
    scale = np.zeros((B, H, D, og + n // group_length), np.float32)
    mn = np.zeros_like(scale)
    _check(lib().kvo_process_key(_p(xf), B * H * D, n, _p(pc), ow, _p(ps), _p(pm), og, group_length,
                                 quant_bits, _p(code), _p(scale), _p(mn)))
    if is_half:
        scale, mn = scale.astype(np.float16), mn.astype(np.float16)
    return code, scale, mn


def process_value_quantization(x_new, prev_code, prev_scale, prev_min, group_length, quant_bits):
    """quantization_cuda.cu:413-537.  x_new [B,H,n,D]; prev_* [B,H,old,...]."""
    is_half = x_new.dtype == np.float16
    xf = np.ascontiguousarray(x_new, np.float32)
    ps = np.ascontiguousarray(prev_scale, np.float32)
    pm = np.ascontiguousarray(prev_min, np.float32)
    pc = np.ascontiguousarray(prev_code, np.int32)
    B, H, n, D = xf.shape
    if quant_bits == 3 and group_length != 11:
        raise RuntimeError(_ERRORS[-2])
    vpw = values_per_word(quant_bits)
    old = pc.shape[2]
    code = np.zeros((B, H, old + n, D // vpw), np.int32)
    scale = np.zeros((B, H, old + n, D // group_length), np.float32)
    mn = np.zeros_like(scale)
    _check(lib().kvo_process_value(_p(xf), B * H, n, D, _p(pc), _p(ps), _p(pm), old, group_length,
                                   quant_bits, _p(code), _p(scale), _p(mn)))
    if is_half:
        scale, mn = scale.astype(np.float16), mn.astype(np.float16)
    return code, scale, mn


# ---------------------------------------------------------------------------
# quantized_gemm   (dequantization_gemv_cuda.cu:127-248)
# ---------------------------------------------------------------------------

GEMM_REFERENCE_ORDER = 0   # 32-lane partial sums + shuffle tree, fma contraction
GEMM_SEQUENTIAL = 1        # dequantize then accumulate k = 0..K-1 in fp32


def quantized_gemm(group_size: int, fA: np.ndarray, qB: np.ndarray, scales: np.ndarray,
                   zeros: np.ndarray, bits: int, mode: int = GEMM_REFERENCE_ORDER,
                   want_f64: bool = False):
    """fA [B,nh,M,K] f16; qB [B,nh_kv,K,N/vpw] i32; scales/zeros [B,nh_kv,K,N/g] f16.
    Returns out f16 [B,nh,M,N]; with want_f64 also (sum in float64, sum of |terms|)."""
    if fA.ndim != 4 or qB.ndim != 4:
        raise RuntimeError("Input tensors must be 4-dimensional")
    if bits not in (1, 2, 3, 4):
        raise RuntimeError(_ERRORS[-1])
    B, nh, M, K = fA.shape
    nh_kv = qB.shape[1]
    if nh % nh_kv:
        raise RuntimeError(_ERRORS[-4])
    if bits == 3 and group_size != 11:
        raise RuntimeError("For 3-bit quantization, group size must be 11")
    N = zeros.shape[-1] * group_size  # dequantization_gemv_cuda.cu:184
    a = np.ascontiguousarray(fA, np.float16)
    q = np.ascontiguousarray(qB, np.int32)
    s = np.ascontiguousarray(scales, np.float16)
    z = np.ascontiguousarray(zeros, np.float16)
    out = np.zeros((B, nh, M, N), np.float16)
    o64 = np.zeros((B, nh, M, N), np.float64) if want_f64 else None
    a64 = np.zeros((B, nh, M, N), np.float64) if want_f64 else None
    _check(lib().kvo_quantized_gemm(group_size, _p(a), M * K, K, _p(q), _p(s), _p(z), bits, B * nh,
                                    nh // nh_kv, M, K, N, mode, _p(out), _p(o64), _p(a64)))
    return (out, o64, a64) if want_f64 else out


def dequantize(qB: np.ndarray, scales: np.ndarray, zeros: np.ndarray, bits: int,
               group_size: int) -> np.ndarray:
    """fp32 weights w[..., n] = fp32(scale[..., grp]) * code + fp32(zero[..., grp])."""
    q = np.ascontiguousarray(qB, np.int32)
    s = np.ascontiguousarray(scales, np.float16)
    z = np.ascontiguousarray(zeros, np.float16)
    N = z.shape[-1] * group_size
    rows = int(np.prod(q.shape[:-1]))
    out = np.zeros(q.shape[:-1] + (N,), np.float32)
    _check(lib().kvo_dequantize(_p(q), _p(s), _p(z), bits, group_size, rows, N, _p(out)))
    return out


def dequantize_np(qB, scales, zeros, bits, group_size) -> np.ndarray:
    """numpy twin of dequantize for group sizes that are multiples of the word size."""
    codes = unpack_np(qB, bits).astype(np.float32)
    s = np.repeat(scales.astype(np.float32), group_size, axis=-1)
    z = np.repeat(zeros.astype(np.float32), group_size, axis=-1)
    return (s * codes).astype(np.float32) + z


# ---------------------------------------------------------------------------
# decode-step attention glue   (models/modeling_llama_KVmix.py:105-211)
# ---------------------------------------------------------------------------

def repeat_kv(x: Optional[np.ndarray], n_rep: int) -> Optional[np.ndarray]:
    """models/modeling_llama_KVmix.py:19-28"""
    if x is None or n_rep == 1:
        return x
    return np.repeat(x, n_rep, axis=1)


def flush_length(tail_len: int, ratio: float, group: int) -> int:
    """How many of the oldest fp16 tail tokens get quantized now
    (models/modeling_llama_KVmix.py:119-127,152-155)."""
    keep = int(ratio * tail_len)
    if tail_len > keep and keep >= 0:
        return ((tail_len - keep) // group) * group
    return 0


def _softmax_f32(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.float32)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m, dtype=np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def _matmul_f16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """fp16 x fp16 -> fp16 with fp32 accumulation (what a GPU half GEMM returns)."""
    return np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)


def attention_prompt(q, k, v, attention_mask=None):
    """The dense attention of the prompt branch (models/modeling_llama_KVmix.py:253-264):
    fp16 logits q.K^T / sqrt(D) (a half tensor divided by a Python number stays half), the mask added
    in the promoted dtype of the two (a half mask: the sum is rounded to half, so a fully masked row
    ends with every entry at the lowest finite half and its softmax is uniform; a float mask: the sum
    is float), clamped to that dtype's lowest finite value, softmax in fp32, probabilities rounded to
    fp16, fp16 product with V.  q [B,nh,T,D], k, v [B,nh_kv,T,D] f16; mask None or [B,1,T,T] f16/f32.
    Returns (attn_output [B,nh,T,D] f16, probs f16)."""
    B, nh, T, D = q.shape
    rep = nh // k.shape[1]
    w = _matmul_f16(q, repeat_kv(k, rep).transpose(0, 1, 3, 2))
    w = (w.astype(np.float32) / np.float32(math.sqrt(D))).astype(np.float16)
    if attention_mask is None:
        w = w.astype(np.float32)
    elif attention_mask.dtype == np.float16:
        with np.errstate(over="ignore"):
            w = (w.astype(np.float32) + attention_mask.astype(np.float32)).astype(np.float16)
        w = np.maximum(w, np.finfo(np.float16).min).astype(np.float32)
    else:
        w = np.maximum(w.astype(np.float32) + attention_mask.astype(np.float32), np.finfo(np.float32).min)
    p = _softmax_f32(w).astype(np.float16)
    return _matmul_f16(p, repeat_kv(v, rep)), p


def attention_decode_step(q, k_new, v_new, cache, k_bits, v_bits, k_ratio, v_ratio,
                          group_size=32, attention_mask=None, fixed_window=None,
                          k_dense3=False, v_dense3=False, compute_output=True):
    """One decode step of LlamaAttention_KVmix.forward after RoPE.

    q [B,nh,1,D] f16; k_new, v_new [B,nh_kv,1,D] f16; cache = the reference's 9-tuple
    (Kcode, K_tail, Kscale, Kmin, Vcode, V_tail, Vscale, Vmin, kv_seq_len), entries may
    be None.  Returns (attn_output [B,nh,1,D] f16, probs f16, new cache).
    fixed_window=R replaces the ratio rule by: when the tail holds more than R tokens, flush
    floor(R/g)*g of the oldest ones (the benchmark's fixed residual window).
    k_dense3 / v_dense3 (with 3 bits): that side is kept in the dense 3-bit stream -- an
    extension without reference counterpart -- in groups of group_size; the flow around the
    quantizer and the product is the reference's.
    compute_output=False only brings the cache up to date (append + flush) and returns
    (None, None, new cache): the cache never depends on the attention arithmetic."""
    kc, k_tail, ks, km, vc, v_tail, vs, vm, seen = cache
    B, nh, _, D = q.shape
    n_rep = nh // k_new.shape[1]
    k_dense3 = bool(k_dense3) and k_bits == 3
    v_dense3 = bool(v_dense3) and v_bits == 3
    kg = 11 if (k_bits == 3 and not k_dense3) else group_size
    vg = group_size

    def quant(chunk, g, bits, dense3):
        return quantize_pack_dense3(chunk, g) if dense3 else quantize_pack_last_dim(chunk, g, bits)

    def gemm(g, x, c, s, m, bits, dense3):
        return quantized_gemm_dense3(g, x, c, s, m) if dense3 else quantized_gemm(g, x, c, s, m, bits)
    k_tail = k_new if k_tail is None else np.concatenate([k_tail, k_new], axis=2)
    v_tail = v_new if v_tail is None else np.concatenate([v_tail, v_new], axis=2)

    def n_flush(tail_len, ratio, g):
        if fixed_window is not None:
            return (fixed_window // g) * g if tail_len > fixed_window else 0
        return flush_length(tail_len, ratio, g)

    nk = n_flush(k_tail.shape[2], k_ratio, kg)
    if nk > 0:
        chunk = np.ascontiguousarray(k_tail[:, :, :nk, :].transpose(0, 1, 3, 2))
        k_tail = k_tail[:, :, nk:, :]
        c, s, m = quant(chunk, kg, k_bits, k_dense3)
        kc = c if kc is None else np.concatenate([kc, c], axis=3)
        ks = s if ks is None else np.concatenate([ks, s], axis=3)
        km = m if km is None else np.concatenate([km, m], axis=3)
    nv = n_flush(v_tail.shape[2], v_ratio, vg)
    if nv > 0:
        chunk = np.ascontiguousarray(v_tail[:, :, :nv, :])
        v_tail = v_tail[:, :, nv:, :]
        c, s, m = quant(chunk, vg, v_bits, v_dense3)
        vc = c if vc is None else np.concatenate([vc, c], axis=2)
        vs = s if vs is None else np.concatenate([vs, s], axis=2)
        vm = m if vm is None else np.concatenate([vm, m], axis=2)

    if not compute_output:
        return None, None, (kc, k_tail, ks, km, vc, v_tail, vs, vm, seen + 1)
    att_q = None
    if kc is not None:
        att_q = gemm(kg, q, repeat_kv(kc, n_rep), repeat_kv(ks, n_rep), repeat_kv(km, n_rep), k_bits, k_dense3)
    att_f = _matmul_f16(q, repeat_kv(k_tail, n_rep).transpose(0, 1, 3, 2))
    if att_q is not None:
        w = np.concatenate([att_q.astype(np.float32), att_f.astype(np.float32)], axis=-1)
    else:
        w = att_f.astype(np.float32)
    w = (w / np.float32(math.sqrt(D))).astype(np.float32)
    if attention_mask is not None:
        w = np.maximum(w + attention_mask.astype(np.float32), np.finfo(np.float32).min)
    p = _softmax_f32(w).astype(np.float16)
    if vc is None:
        out = _matmul_f16(p, repeat_kv(v_tail, n_rep))
    else:
        lv = v_tail.shape[2]
        out_q = gemm(vg, np.ascontiguousarray(p[..., : p.shape[-1] - lv]),
                     repeat_kv(vc, n_rep), repeat_kv(vs, n_rep), repeat_kv(vm, n_rep), v_bits, v_dense3)
        out_f = _matmul_f16(p[..., p.shape[-1] - lv:], repeat_kv(v_tail, n_rep))
        out = (out_q.astype(np.float32) + out_f.astype(np.float32)).astype(np.float16)
    return out, p, (kc, k_tail, ks, km, vc, v_tail, vs, vm, seen + 1)
