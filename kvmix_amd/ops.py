"""The reference's four operators (module `KVmix`, quant_cuda/csrc/pybind.cpp:6-15) on top of
the gfx950 C ABI.  Names, positional argument order, return types and error texts follow the
reference; the tensors are torch ROCm tensors, everything else is the HIP library.

    quantize_pack_last_dim_cuda(input, group_length, quant_bits) -> (code, scale, min)
    quantized_gemm(group_size, fA, qB, scales, zeros, bits) -> out
    process_key_quantization_cuda(input, prev_code, prev_scale, prev_min, group_length, quant_bits)
    process_value_quantization_cuda(input, prev_code, prev_scale, prev_min, group_length, quant_bits)

All four launch on torch's current stream of the input's device and do not synchronise.
"""
from __future__ import annotations

from typing import Tuple

import functools

import torch

from . import _lib

_DT = {torch.float16: _lib.F16, torch.float32: _lib.F32}


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("KVmix operators run on the GPU only: got a tensor on " + str(t.device))


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _values_per_word(bits: int) -> int:
    return 11 if bits == 3 else 32 // bits


def _check_bits(bits: int) -> None:
    if bits not in (1, 2, 3, 4):
        raise RuntimeError("Supported quantization bits: 1, 2, 3, 4")


def _rows3(t: torch.Tensor) -> Tuple[torch.Tensor, int, int]:
    """View a 4-D tensor [B, H, R, S] as [B*H, R, S] without copying when its strides allow it;
    returns (tensor, outer_stride, inner_stride) in elements."""
    B, H, R, S = t.shape
    ok = (S <= 1 or t.stride(3) == 1) and (B <= 1 or t.stride(0) == H * t.stride(1))
    if ok and R > 1 and t.stride(2) < S:
        ok = False
    if ok and H > 1 and t.stride(1) < t.stride(2):
        ok = False
    if not ok:
        t = t.contiguous()
    return t, (t.stride(1) if B * H > 1 else max(R * t.stride(2), 1)), (t.stride(2) if R > 1 else max(S, 1))


def _quantize_into(x: torch.Tensor, group: int, bits: int, fmt: int, scale_mode: int,
                   code: torch.Tensor, scale: torch.Tensor, mn: torch.Tensor) -> None:
    """x [B,H,R,S]; code/scale/mn 4-D views (possibly slices of larger buffers) to fill."""
    L = _lib.load()
    B, H, R, S = x.shape
    x, xo, xi = _rows3(x)
    with torch.cuda.device(x.device):
        _lib.check(L.kvmix_quant_pack_last_dim(
            x.data_ptr(), _DT[x.dtype], B * H, R, S, xo, xi, group, bits, fmt, scale_mode,
            code.data_ptr(), code.stride(1), code.stride(2),
            scale.data_ptr(), mn.data_ptr(), scale.stride(1), scale.stride(2), _stream(x)))


def quantize_pack_last_dim_cuda(input: torch.Tensor, group_length: int, quant_bits: int):
    """Group-quantize the last dimension of a 4-D fp16/fp32 tensor and bit-pack the codes.

    Reference: quantize_pack_last_dim_cuda, quant_cuda/csrc/quantization_cuda.cu:631-721.
    Returns (code int32 [B,H,R,S/vpw], scale [B,H,R,S/g], min [B,H,R,S/g]); scale and min have the
    input's dtype.  3-bit uses the reference's 11-codes-per-word layout and needs group_length 11."""
    if quant_bits == 3 and group_length != 11:
        raise RuntimeError("For 3-bit quantization, group_length must be 11")
    if input.dtype not in _DT:
        raise RuntimeError(f"expected scalar type Float or Half but found {input.dtype}")
    if input.dim() != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    _check_bits(quant_bits)
    B, H, R, S = input.shape
    if quant_bits == 3:
        if S % 11 != 0:
            raise RuntimeError("For 3-bit quantization, steps must be divisible by 11")
    else:
        if group_length <= 0 or S % group_length != 0:
            raise RuntimeError("steps must be divisible by group_length")
        if S % (32 // quant_bits) != 0:
            raise RuntimeError("steps must be divisible by (32 / quant_bits)")
    _need_gpu(input)
    vpw = _values_per_word(quant_bits)
    code = torch.empty((B, H, R, S // vpw), dtype=torch.int32, device=input.device)
    scale = torch.empty((B, H, R, S // group_length), dtype=input.dtype, device=input.device)
    mn = torch.empty_like(scale)
    _quantize_into(input, group_length, quant_bits, _lib.FMT_REF, _lib.SCALE_RECIPROCAL, code, scale, mn)
    return code, scale, mn


def quantize_pack_dense3(input: torch.Tensor, group_length: int = 32):
    """Extension (no reference counterpart): 3-bit codes with qmax 7 for every value, stored as a
    little-endian bit stream (32 codes in three uint32), group a multiple of 32.  Same min / max /
    scale / rounding arithmetic as quantize_pack_last_dim_cuda.  Pair with
    quantized_gemm(..., bits=3, fmt=FMT_DENSE3).
    Returns (code int32 [B,H,R,3S/32], scale [B,H,R,S/g], min [B,H,R,S/g])."""
    if input.dtype not in _DT:
        raise RuntimeError(f"expected scalar type Float or Half but found {input.dtype}")
    if input.dim() != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    B, H, R, S = input.shape
    if group_length <= 0 or group_length % 32 != 0:
        raise RuntimeError("dense 3-bit needs a group_length that is a multiple of 32")
    if S % group_length != 0:
        raise RuntimeError("steps must be divisible by group_length")
    _need_gpu(input)
    code = torch.empty((B, H, R, S * 3 // 32), dtype=torch.int32, device=input.device)
    scale = torch.empty((B, H, R, S // group_length), dtype=input.dtype, device=input.device)
    mn = torch.empty_like(scale)
    _quantize_into(input, group_length, 3, _lib.FMT_DENSE3, _lib.SCALE_RECIPROCAL, code, scale, mn)
    return code, scale, mn


FMT_REF = _lib.FMT_REF
FMT_DENSE3 = _lib.FMT_DENSE3


def quantize_kv_flush(k_chunk: torch.Tensor, k_group: int, k_bits: int, v_chunk: torch.Tensor, v_group: int,
                      v_bits: int, k_fmt: int = _lib.FMT_REF, v_fmt: int = _lib.FMT_REF):
    """Extension (no reference counterpart): both flushes of a decode step in ONE launch.

    k_chunk [B,H,n,D] fp16 are the oldest n tokens of the key tail, token-major as the tail is
    stored; the result is what quantize_pack_last_dim_cuda(k_chunk.transpose(2, 3).contiguous(),
    k_group, k_bits) returns (models/modeling_llama_KVmix.py:131-133), without the transpose copy.
    v_chunk [B,H,nv,D] fp16 is quantized along D as quantize_pack_last_dim_cuda(v_chunk, v_group,
    v_bits) does (:157-159).  Bit-identical to the two separate operators.
    Returns (k_code [B,H,D,n/vpw], k_scale, k_min [B,H,D,n/g], v_code [B,H,nv,D/vpw], v_scale, v_min)."""
    for t in (k_chunk, v_chunk):
        if t.dim() != 4:
            raise RuntimeError("input_tensor must be a 4D tensor")
        if t.dtype != torch.float16:
            raise RuntimeError(f"expected scalar type Half but found {t.dtype}")
    _check_bits(k_bits)
    _check_bits(v_bits)
    _need_gpu(k_chunk, v_chunk)
    L = _lib.load()
    B, H, n, D = k_chunk.shape
    Bv, Hv, nv, Dv = v_chunk.shape
    dev = k_chunk.device

    def words(steps, bits, fmt):
        return steps * 3 // 32 if (bits == 3 and fmt == _lib.FMT_DENSE3) else steps // _values_per_word(bits)

    kc = torch.empty((B, H, D, words(n, k_bits, k_fmt)), dtype=torch.int32, device=dev)
    ks = torch.empty((B, H, D, n // k_group if k_group > 0 else 0), dtype=torch.float16, device=dev)
    km = torch.empty_like(ks)
    vc = torch.empty((Bv, Hv, nv, words(Dv, v_bits, v_fmt)), dtype=torch.int32, device=dev)
    vs = torch.empty((Bv, Hv, nv, Dv // v_group if v_group > 0 else 0), dtype=torch.float16, device=dev)
    vm = torch.empty_like(vs)
    quantize_kv_flush_into(k_chunk, k_group, k_bits, (kc, ks, km), v_chunk, v_group, v_bits, (vc, vs, vm), k_fmt, v_fmt)
    return kc, ks, km, vc, vs, vm


def _flush_descriptors(k_chunk, k_group: int, k_bits: int, k_out, v_chunk, v_group: int, v_bits: int, v_out,
                       k_fmt: int = _lib.FMT_REF, v_fmt: int = _lib.FMT_REF):
    """The (KeyFlush, ValueFlush, tensors to keep alive) of one flush, or None when there is nothing to do.  Keys in
    groups the token-major key kernel does not take (other than 32, or 11 for the reference's 3 bits) are quantized
    here and now through the one-shot quantizer; the key descriptor then stays empty."""
    kf, vf = _lib.KeyFlush(), _lib.ValueFlush()
    kf.group, kf.bits, kf.fmt, kf.scale_mode = max(k_group, 1), k_bits, k_fmt, _lib.SCALE_RECIPROCAL
    vf.group, vf.bits, vf.fmt, vf.scale_mode = max(v_group, 1), v_bits, v_fmt, _lib.SCALE_RECIPROCAL
    ref = k_chunk if k_chunk is not None else v_chunk
    if ref is None:
        return None
    _need_gpu(ref)
    keep = [ref]

    def out_strides(code, scale, mn, B, H):
        for t in (code, scale, mn):
            if t.dim() != 4 or (t.shape[3] > 1 and t.stride(3) != 1) or (B > 1 and t.stride(0) != H * t.stride(1)):
                raise RuntimeError("output views must be 4-D, unit-stride along the last dimension, (B, H) collapsible")
        if (scale.stride(1), scale.stride(2)) != (mn.stride(1), mn.stride(2)):
            raise RuntimeError("scale and min outputs must share their strides")

    if k_chunk is not None and k_chunk.shape[2] > 0:
        B, H, n, D = k_chunk.shape
        ref3 = k_bits == 3 and k_fmt == _lib.FMT_REF
        if not ref3 and k_group != 32:
            # the token-major key kernel is built for group 32 (and the reference's 3-bit group 11)
            _quantize_into(k_chunk.transpose(2, 3).contiguous(), k_group, k_bits, k_fmt, _lib.SCALE_RECIPROCAL, *k_out)
        else:
            if k_chunk.stride(3) != 1 or (B > 1 and k_chunk.stride(0) != H * k_chunk.stride(1)):
                k_chunk = k_chunk.contiguous()
            kc, ks, km = k_out
            out_strides(kc, ks, km, B, H)
            kf.k, kf.outer, kf.n, kf.D = k_chunk.data_ptr(), B * H, n, D
            kf.k_outer_stride, kf.k_token_stride = k_chunk.stride(1), k_chunk.stride(2)
            kf.code, kf.code_outer_stride, kf.code_inner_stride = kc.data_ptr(), kc.stride(1), kc.stride(2)
            kf.scale, kf.zero = ks.data_ptr(), km.data_ptr()
            kf.sz_outer_stride, kf.sz_inner_stride = ks.stride(1), ks.stride(2)
            keep += [k_chunk, kc, ks, km]
    if v_chunk is not None and v_chunk.shape[2] > 0:
        Bv, Hv, nv, Dv = v_chunk.shape
        v_chunk, vo, vi = _rows3(v_chunk)
        vc, vs, vm = v_out
        out_strides(vc, vs, vm, Bv, Hv)
        vf.x, vf.outer, vf.inner, vf.steps = v_chunk.data_ptr(), Bv * Hv, nv, Dv
        vf.x_outer_stride, vf.x_inner_stride = vo, vi
        vf.code, vf.code_outer_stride, vf.code_inner_stride = vc.data_ptr(), vc.stride(1), vc.stride(2)
        vf.scale, vf.zero = vs.data_ptr(), vm.data_ptr()
        vf.sz_outer_stride, vf.sz_inner_stride = vs.stride(1), vs.stride(2)
        keep += [v_chunk, vc, vs, vm]
    return kf, vf, keep


def quantize_kv_flush_into(k_chunk, k_group: int, k_bits: int, k_out, v_chunk, v_group: int, v_bits: int, v_out,
                           k_fmt: int = _lib.FMT_REF, v_fmt: int = _lib.FMT_REF) -> None:
    """quantize_kv_flush writing into tensors the caller owns: k_out = (code [B,H,D,n/vpw],
    scale, min [B,H,D,n/g]) and v_out = (code [B,H,nv,D/vpw], scale, min [B,H,nv,D/g]) may be
    slices of larger pre-allocated cache buffers (unit stride along the last dimension, (B, H)
    collapsible).  Either half may be None (k_chunk and k_out, or v_chunk and v_out)."""
    import ctypes

    d = _flush_descriptors(k_chunk, k_group, k_bits, k_out, v_chunk, v_group, v_bits, v_out, k_fmt, v_fmt)
    if d is None:
        return
    kf, vf, keep = d
    with torch.cuda.device(keep[0].device):
        _lib.check(_lib.load().kvmix_quant_pack_kv_flush(ctypes.byref(kf), ctypes.byref(vf), _stream(keep[0])))


def quantize_kv_flush_batch(flushes) -> None:
    """The flushes of several caches at once (kvmix_quant_pack_kv_flush_batch: eight to a launch): `flushes` is a
    sequence of argument tuples of quantize_kv_flush_into, all on one device; the results are those of calling it
    on each tuple, bit for bit.  What a decode step flushes are the oldest tokens of the fp16 tails
    (models/modeling_llama_KVmix.py:122-127,152-156), so a caller can issue the flushes of all layers of a step
    together before its first layer runs."""
    ds = [d for d in (_flush_descriptors(*f) for f in flushes) if d is not None]
    if not ds:
        return
    dev = ds[0][2][0].device
    if any(d[2][0].device != dev for d in ds):
        raise RuntimeError("the flushes of one batch must be on one device")
    with torch.cuda.device(dev):
        _lib.check(_lib.flush_batch([d[0] for d in ds], [d[1] for d in ds], _stream(ds[0][2][0])))


def _batched3(t: torch.Tensor) -> Tuple[torch.Tensor, int, int]:
    """[B, H, R, S] -> (tensor, batch stride, row stride) with (B, H) collapsible, unit last stride."""
    B, H, R, S = t.shape
    ok = (S <= 1 or t.stride(3) == 1) and (B <= 1 or t.stride(0) == H * t.stride(1))
    ok = ok and (R <= 1 or t.stride(2) >= S) and (H <= 1 or t.stride(1) >= t.stride(2))
    if not ok:
        t = t.contiguous()
    bs = t.stride(1) if B * H > 1 else max(R * max(t.stride(2), S), 1)
    rs = t.stride(2) if R > 1 else max(S, 1)
    return t, bs, rs


def quantized_gemm(group_size: int, fA: torch.Tensor, qB: torch.Tensor, scales: torch.Tensor,
                   zeros: torch.Tensor, bits: int, fmt: int = _lib.FMT_REF) -> torch.Tensor:
    """out[b,h,m,:] = fA[b,h,m,:] @ dequant(qB[b,h',:,:]) with h' = h // (nh // nh_kv).

    Reference: quantized_gemm, quant_cuda/csrc/dequantization_gemv_cuda.cu:127-248.
    fA [B,nh,M,K] f16; qB [B,nh_kv,K,N/vpw] i32; scales, zeros [B,nh_kv,K,N/g] f16 -> [B,nh,M,N] f16.
    The packed operands are read in place (views of a larger cache buffer are fine); GQA inputs
    may be passed un-repeated.  `fmt` is an extension (dense 3-bit); the default is the reference's."""
    if fA.dim() != 4 or qB.dim() != 4:
        raise RuntimeError("Input tensors must be 4-dimensional")
    _check_bits(bits)
    B, nh, M, K = fA.shape
    nh_kv = qB.shape[1]
    if nh_kv == 0 or nh % nh_kv != 0:
        raise RuntimeError("Total heads must be divisible by KV heads")
    if bits == 3 and fmt == _lib.FMT_REF and group_size != 11:
        raise RuntimeError("For 3-bit quantization, group size must be 11")
    if fA.dtype != torch.float16 or scales.dtype != torch.float16 or zeros.dtype != torch.float16:
        raise RuntimeError("expected scalar type Half for fA, scales and zeros")
    if qB.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int for qB")
    _need_gpu(fA, qB, scales, zeros)
    if scales.dim() != 4 or zeros.dim() != 4 or scales.shape != zeros.shape:
        raise RuntimeError("scales and zeros must be 4-dimensional and of equal shape")
    if qB.shape[0] != B or qB.shape[2] != K or scales.shape[:3] != qB.shape[:3]:
        raise RuntimeError("shape mismatch between fA, qB and scales")
    N = zeros.shape[-1] * group_size  # dequantization_gemv_cuda.cu:184
    L = _lib.load()
    fA, x_bs, x_rs = _batched3(fA)
    qB, c_bs, c_rs = _batched3(qB)
    scales, s_bs, s_rs = _batched3(scales)
    zeros, z_bs, z_rs = _batched3(zeros)
    if (z_bs, z_rs) != (s_bs, s_rs):
        zeros = zeros.contiguous()
        scales = scales.contiguous()
        scales, s_bs, s_rs = _batched3(scales)
        zeros, z_bs, z_rs = _batched3(zeros)
    out = torch.empty((B, nh, M, N), dtype=torch.float16, device=fA.device)
    ws_bytes = L.kvmix_gemv_workspace_bytes(B * nh, M, K, N)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=fA.device) if ws_bytes else None
    with torch.cuda.device(fA.device):
        _lib.check(L.kvmix_quantized_gemv(
            group_size, fA.data_ptr(), x_bs, x_rs, qB.data_ptr(), c_bs, c_rs,
            scales.data_ptr(), zeros.data_ptr(), s_bs, s_rs, bits, fmt, B * nh, nh // nh_kv,
            M, K, N, out.data_ptr(), M * N, N, ws.data_ptr() if ws is not None else None,
            ws_bytes, _stream(fA)))
    return out


def prefer_single_pass(batch: int, heads: int, kv_heads: int, head_dim: int, width: int, k_bits: int, k_fmt: int,
                       k_group: int, v_bits: int, v_fmt: int, v_group: int, k_tokens: int = None,
                       v_tokens: int = None) -> bool:
    """Policy for callers that do not need the probabilities: whether the single-pass step is both
    available for this layout and the faster of the two at this size.  The library holds the measured rule
    (kvmix_decode_attention_fused_plan: `recommended`); k_tokens / v_tokens are the quantized lengths, where the
    caller knows them (they decide whether a large step can use the matrix cores; without them a step is
    taken to have nothing quantized on both sides)."""
    if kv_heads <= 0 or heads % kv_heads != 0:
        return False
    if not single_pass_supported(head_dim, heads // kv_heads, k_bits, k_fmt, k_group, v_bits, v_fmt, v_group):
        return False
    if k_tokens is None or v_tokens is None or width < max(k_tokens, v_tokens):
        k_tokens = v_tokens = 0
    step = _lib.attn_step_descriptor(batch, heads, kv_heads, head_dim, k_bits, k_fmt, k_group, k_tokens, v_bits, v_fmt,
                                     v_group, v_tokens, width - k_tokens, width - v_tokens)
    try:
        return _lib.attn_plan(step)["recommended"]
    except RuntimeError:
        return False


def rope_append(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, heads: int, kv_heads: int,
                k_tail: torch.Tensor, v_tail: torch.Tensor, k_slot, v_slot) -> torch.Tensor:
    """Rotary embedding of the new token's query and key heads and the append of its key and value
    heads to the cache tails, in one launch (models/modeling_llama_KVmix.py:102-112 for one token).

    qkv [B, 1, (heads + 2 kv_heads) * D] or [B, heads + 2 kv_heads, D] fp16: query, key, value heads
    of the new token; cos, sin: D fp16 values for its position (any shape with D elements);
    k_tail, v_tail [B, kv_heads, slots, D] fp16 windows, written in place at slot k_slot / v_slot
    (ints, or one-element int64 device tensors read when the kernel runs).
    Returns the rotated queries [B, heads, 1, D].  Bit-identical to x * cos + rotate_half(x) * sin
    in fp16 tensor arithmetic."""
    import ctypes

    for t in (qkv, cos, sin, k_tail, v_tail):
        if t.dtype != torch.float16:
            raise RuntimeError(f"expected scalar type Half but found {t.dtype}")
    _need_gpu(qkv, cos, sin, k_tail, v_tail)
    B, D = qkv.shape[0], k_tail.shape[-1]
    total = heads + 2 * kv_heads
    if qkv.numel() != B * total * D or cos.numel() != D or sin.numel() != D:
        raise RuntimeError("rope_append: qkv must hold heads + 2 * kv_heads rows of D values per batch element, cos and sin D values")
    if k_tail.dim() != 4 or v_tail.dim() != 4 or k_tail.shape[:2] != (B, kv_heads) or v_tail.shape[:2] != (B, kv_heads) \
            or v_tail.shape[-1] != D or k_tail.stride(3) != 1 or v_tail.stride(3) != 1:
        raise RuntimeError("rope_append: tails must be [B, kv_heads, slots, D] with unit stride along D")
    qkv = qkv.reshape(B, total * D)
    if qkv.stride(1) != 1:
        qkv = qkv.contiguous()
    cos, sin = cos.reshape(D).contiguous(), sin.reshape(D).contiguous()
    q_out = torch.empty((B, heads, 1, D), dtype=torch.float16, device=qkv.device)
    st = _lib.RopeAppend()
    st.qkv, st.qkv_batch_stride, st.cos, st.sin = qkv.data_ptr(), qkv.stride(0) if B > 1 else total * D, cos.data_ptr(), sin.data_ptr()
    st.q_out, st.q_batch_stride = q_out.data_ptr(), heads * D
    for prefix, tail, slot in (("k", k_tail, k_slot), ("v", v_tail, v_slot)):
        setattr(st, prefix + "_tail", tail.data_ptr())
        setattr(st, prefix + "_tail_batch_stride", tail.stride(0))
        setattr(st, prefix + "_tail_head_stride", tail.stride(1))
        setattr(st, prefix + "_tail_token_stride", tail.stride(2))
        setattr(st, prefix + "_tail_slots", tail.shape[2])
        if torch.is_tensor(slot):
            if slot.dtype != torch.int64 or slot.numel() != 1 or not slot.is_cuda:
                raise RuntimeError("a device-side slot must be one int64 element on the GPU")
            setattr(st, prefix + "_slot_dev", slot.data_ptr())
        else:
            setattr(st, prefix + "_slot", int(slot))
    st.batch, st.heads, st.kv_heads, st.D = B, heads, kv_heads, D
    with torch.cuda.device(qkv.device):
        _lib.check(_lib.load().kvmix_rope_append(ctypes.byref(st), _stream(qkv)))
    return q_out


@functools.lru_cache(maxsize=None)
def single_pass_supported(head_dim: int, heads_per_kv: int, k_bits: int, k_fmt: int, k_group: int, v_bits: int,
                          v_fmt: int, v_group: int) -> bool:
    """Whether decode_attention(single_pass=True) takes a cache of this layout (asks the library)."""
    import ctypes

    st = _lib.DecodeAttn()
    st.D, st.heads_per_kv, st.heads, st.samples = head_dim, heads_per_kv, heads_per_kv, heads_per_kv
    st.k_bits, st.k_fmt, st.k_group, st.k_tokens = k_bits, k_fmt, k_group, (11 if k_group == 11 else 32) * 32
    st.v_bits, st.v_fmt, st.v_group, st.v_tokens = v_bits, v_fmt, v_group, 32
    return bool(_lib.load().kvmix_decode_attention_fused_supported(ctypes.byref(st)))


def decode_attention(q: torch.Tensor, k_packed, v_packed, k_tail: torch.Tensor, v_tail: torch.Tensor,
                     k_group: int, k_bits: int, v_group: int, v_bits: int, k_fmt: int = _lib.FMT_REF,
                     v_fmt: int = _lib.FMT_REF, attention_mask=None, k_tail_len=None, v_tail_len=None,
                     single_pass: bool = False):
    """One decode step of attention over the packed cache plus its fp16 tails, in four or five
    launches (no reference operator: it is what models/modeling_llama_KVmix.py:180-211 composes
    from quantized_gemm, matmul, cat and softmax).

    single_pass=True runs the step as one pass over the positions instead (two launches, logits and
    probabilities stay on chip); no probabilities are returned (probs is None) and the roundings
    after the softmax are not the reference's (see the header).  Layouts the single-pass kernels do
    not take raise RuntimeError; `single_pass_supported` tells beforehand.

    q [B,nh,1,D] fp16; k_packed = (code [B,Hkv,D,Tk/vpw], scale, min) or None; v_packed =
    (code [B,Hkv,Tv,D/vpw], scale, min) or None; k_tail, v_tail [B,Hkv,slots,D] fp16.
    *_tail_len: None (every slot holds a token), an int, or a device int64 tensor of one element
    read when the kernels run (for steps replayed from a captured graph).
    attention_mask: None or fp32 [B,1,1,width].
    Returns (out [B,nh,1,D] fp16, probs [B,nh,1,width] fp16), width = max(Tk + key slots, Tv + value slots)."""
    import ctypes

    if q.dim() != 4 or q.shape[2] != 1:
        raise RuntimeError("decode_attention takes one query position: q must be [B, nh, 1, D]")
    for t in (q, k_tail, v_tail):
        if t.dtype != torch.float16:
            raise RuntimeError(f"expected scalar type Half but found {t.dtype}")
    _need_gpu(q, k_tail, v_tail)
    _check_bits(k_bits)
    _check_bits(v_bits)
    L = _lib.load()
    B, nh, _, D = q.shape
    nkv = k_tail.shape[1]
    if nkv == 0 or nh % nkv != 0:
        raise RuntimeError("Total heads must be divisible by KV heads")
    st = _lib.DecodeAttn()
    q, q_bs, _ = _batched3(q)
    st.q, st.q_stride = q.data_ptr(), q_bs
    keep = [q]

    def packed(prefix, triple, tokens_of):
        if triple is None or triple[0] is None:
            setattr(st, prefix + "_tokens", 0)
            return
        code, scale, zero = triple
        code, c_bs, c_rs = _batched3(code)
        scale, s_bs, s_rs = _batched3(scale)
        zero, z_bs, z_rs = _batched3(zero)
        if (z_bs, z_rs) != (s_bs, s_rs):
            scale, zero = scale.contiguous(), zero.contiguous()
            scale, s_bs, s_rs = _batched3(scale)
            zero, z_bs, z_rs = _batched3(zero)
        keep.extend((code, scale, zero))
        setattr(st, prefix + "_code", code.data_ptr())
        setattr(st, prefix + "_code_batch_stride", c_bs)
        setattr(st, prefix + "_code_row_stride", c_rs)
        setattr(st, prefix + "_scale", scale.data_ptr())
        setattr(st, prefix + "_zero", zero.data_ptr())
        setattr(st, prefix + "_sz_batch_stride", s_bs)
        setattr(st, prefix + "_sz_row_stride", s_rs)
        setattr(st, prefix + "_tokens", tokens_of(code, zero))

    packed("k", k_packed, lambda code, zero: zero.shape[-1] * k_group)
    packed("v", v_packed, lambda code, zero: code.shape[2])
    st.k_bits, st.k_fmt, st.k_group = k_bits, k_fmt, k_group
    st.v_bits, st.v_fmt, st.v_group = v_bits, v_fmt, v_group

    def tail(prefix, t, length):
        t, t_bs, t_ts = _batched3(t)
        keep.append(t)
        setattr(st, prefix + "_tail", t.data_ptr())
        setattr(st, prefix + "_tail_batch_stride", t_bs)
        setattr(st, prefix + "_tail_token_stride", t_ts)
        setattr(st, prefix + "_tail_slots", t.shape[2])
        if torch.is_tensor(length):
            if length.dtype != torch.int64 or length.numel() != 1 or not length.is_cuda:
                raise RuntimeError("a device-side tail length must be one int64 element on the GPU")
            setattr(st, prefix + "_tail_len_dev", length.data_ptr())
        else:
            setattr(st, prefix + "_tail_len", t.shape[2] if length is None else int(length))

    tail("k", k_tail, k_tail_len)
    tail("v", v_tail, v_tail_len)
    width = max(st.k_tokens + st.k_tail_slots, st.v_tokens + st.v_tail_slots)
    if attention_mask is not None:
        if attention_mask.dtype != torch.float32 or tuple(attention_mask.shape) != (B, 1, 1, width):
            raise RuntimeError(f"attention_mask must be fp32 of shape {(B, 1, 1, width)}")
        if attention_mask.stride(3) != 1:
            attention_mask = attention_mask.contiguous()
        keep.append(attention_mask)
        st.mask, st.mask_stride = attention_mask.data_ptr(), attention_mask.stride(0) if B > 1 else width
    st.samples, st.heads, st.heads_per_kv, st.D = B * nh, nh, nh // nkv, D
    out = torch.empty((B, nh, 1, D), dtype=torch.float16, device=q.device)
    if single_pass:
        st.out, st.out_stride = out.data_ptr(), D
        if not L.kvmix_decode_attention_fused_supported(ctypes.byref(st)):
            raise RuntimeError("the single-pass attention step does not take this layout (head_dim 128, keys 1/2/4-bit or "
                               "dense 3-bit group 32 or reference 3-bit, values 1/2/4-bit or dense 3-bit group 32)")
        ws_bytes = L.kvmix_decode_attention_fused_workspace_bytes(ctypes.byref(st))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        with torch.cuda.device(q.device):
            _lib.check(L.kvmix_decode_attention_fused(ctypes.byref(st), ws.data_ptr(), ws_bytes, _stream(q)))
        return out, None
    probs = torch.empty((B, nh, 1, width), dtype=torch.float16, device=q.device)
    st.probs, st.probs_stride, st.out, st.out_stride = probs.data_ptr(), width, out.data_ptr(), D
    ws_bytes = L.kvmix_decode_attention_workspace_bytes(ctypes.byref(st))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    with torch.cuda.device(q.device):
        _lib.check(L.kvmix_decode_attention(ctypes.byref(st), ws.data_ptr() if ws is not None else None, ws_bytes,
                                            _stream(q)))
    return out, probs


def _append_checks(input, prev_scale, prev_min):
    if input.dim() != 4:
        raise RuntimeError("input_tensor must be a 4D tensor")
    if input.dtype not in _DT:
        raise RuntimeError(f"expected scalar type Float or Half but found {input.dtype}")
    if prev_scale.dtype != input.dtype or prev_min.dtype != input.dtype:
        raise RuntimeError("previous_scale / previous_min must have the input's dtype")


def process_key_quantization_cuda(input: torch.Tensor, previous_code: torch.Tensor,
                                  previous_scale: torch.Tensor, previous_min: torch.Tensor,
                                  group_length: int, quant_bits: int):
    """Append form for keys: input [B,H,D,n] (groups along n) is quantized and returned
    concatenated after previous_* along the last dimension.

    Reference: process_key_quantization_cuda, quant_cuda/csrc/quantization_cuda.cu:298-411.
    The returned scale is (max-min)/qmax rounded to the input dtype (the reference's append
    kernels divide in-kernel, :49-51,:149-151)."""
    _append_checks(input, previous_scale, previous_min)
    _check_bits(quant_bits)
    B, H, D, n = input.shape
    if quant_bits == 3:
        if group_length != 11:
            raise RuntimeError("For 3-bit quantization, group_length must be 11")
        if n % 11 != 0:
            raise RuntimeError("new_steps must be divisible by 11 for 3-bit quantization")
    elif group_length <= 0 or n % group_length != 0:
        raise RuntimeError("new_steps must be divisible by group_length")
    _need_gpu(input, previous_code, previous_scale, previous_min)
    vpw = _values_per_word(quant_bits)
    if quant_bits != 3 and (group_length % vpw != 0 or n % vpw != 0):
        raise RuntimeError(_lib.strerror(-9))
    ow, og = previous_code.shape[3], previous_scale.shape[3]
    code = torch.empty((B, H, D, ow + n // vpw), dtype=torch.int32, device=input.device)
    scale = torch.empty((B, H, D, og + n // group_length), dtype=input.dtype, device=input.device)
    mn = torch.empty_like(scale)
    code[..., :ow].copy_(previous_code.reshape(B, H, D, ow))
    scale[..., :og].copy_(previous_scale.reshape(B, H, D, og))
    mn[..., :og].copy_(previous_min.reshape(B, H, D, og))
    if n > 0:
        _quantize_into(input, group_length, quant_bits, _lib.FMT_REF, _lib.SCALE_DIVIDE,
                       code[..., ow:], scale[..., og:], mn[..., og:])
    return code, scale, mn


def process_value_quantization_cuda(input: torch.Tensor, previous_code: torch.Tensor,
                                    previous_scale: torch.Tensor, previous_min: torch.Tensor,
                                    group_length: int, quant_bits: int):
    """Append form for values: input [B,H,n,D] (groups along D) is quantized and returned
    concatenated after previous_* along the token dimension.

    Reference: process_value_quantization_cuda, quant_cuda/csrc/quantization_cuda.cu:413-537.
    3-bit follows the reference's placeholder branch literally (plain 3*j shifts, so the
    eleventh code of a word keeps only its low two bits)."""
    _append_checks(input, previous_scale, previous_min)
    _check_bits(quant_bits)
    B, H, n, D = input.shape
    if quant_bits == 3:
        if group_length != 11:
            raise RuntimeError("For 3-bit quantization, group_length must be 11")
        if D % 11 != 0:
            raise RuntimeError("head_dim must be divisible by 11 for 3-bit quantization")
    elif group_length <= 0 or D % group_length != 0:
        raise RuntimeError("head_dim must be divisible by group_length")
    _need_gpu(input, previous_code, previous_scale, previous_min)
    vpw = _values_per_word(quant_bits)
    if quant_bits != 3 and (group_length % vpw != 0 or D % vpw != 0):
        raise RuntimeError(_lib.strerror(-9))
    old = previous_code.shape[2]
    wpt, gpt = D // vpw, D // group_length
    code = torch.empty((B, H, old + n, wpt), dtype=torch.int32, device=input.device)
    scale = torch.empty((B, H, old + n, gpt), dtype=input.dtype, device=input.device)
    mn = torch.empty_like(scale)
    code[:, :, :old].copy_(previous_code.reshape(B, H, old, wpt))
    scale[:, :, :old].copy_(previous_scale.reshape(B, H, old, gpt))
    mn[:, :, :old].copy_(previous_min.reshape(B, H, old, gpt))
    if n > 0:
        fmt = _lib.FMT_REF3_WRAP if quant_bits == 3 else _lib.FMT_REF
        _quantize_into(input, group_length, quant_bits, fmt, _lib.SCALE_DIVIDE,
                       code[:, :, old:], scale[:, :, old:], mn[:, :, old:])
    return code, scale, mn
