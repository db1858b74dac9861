"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol
declared in include/kvmix_hip.h, maps error codes to the reference's messages, and the
Python operators reject bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from kvmix_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from kvmix_amd import build_ext

        build_ext.build()
    return _lib.load()


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "kvmix_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(kvmix_[a-z_0-9]+)\s*\(", header))
    assert declared >= {"kvmix_version", "kvmix_strerror", "kvmix_quant_pack_last_dim",
                        "kvmix_quant_pack_key_tokens", "kvmix_gemv_workspace_bytes",
                        "kvmix_quantized_gemv"}
    for name in declared:
        assert hasattr(lib, name), name
    from kvmix_amd import _lib
    assert set(_lib.EXPORTS) == declared


def test_version_and_error_text(lib):
    from kvmix_amd import _lib

    assert lib.kvmix_version() >= 100
    assert _lib.strerror(0) == "ok"
    assert "1, 2, 3, 4" in _lib.strerror(-1)
    assert "group_length must be 11" in _lib.strerror(-2)
    assert "divisible by group_length" in _lib.strerror(-3)
    assert "32 / quant_bits" in _lib.strerror(-4)
    assert "divisible by KV heads" in _lib.strerror(-5)
    codes = {_lib.strerror(c) for c in range(-14, 0)}
    assert len(codes) == 14  # distinct text per code
    assert "built-in buffer" in _lib.strerror(-13) and "hipGetSymbolAddress" in _lib.strerror(-14)
    with pytest.raises(RuntimeError, match="KV heads"):
        _lib.check(-5)


def test_host_validation_needs_no_gpu(lib):
    """Argument errors are detected on the host before any launch (safe without a GPU)."""
    q = lib.kvmix_quant_pack_last_dim
    one = ctypes.c_void_p(16)
    args = lambda **kw: [kw.get("x", one), kw.get("dt", 0), 1, 1, kw.get("steps", 64), 64, 64,
                         kw.get("g", 32), kw.get("bits", 4), kw.get("fmt", 0), 0, one, 8, 8, one, one, 2, 2, None]
    assert q(*args(bits=5)) == -1
    assert q(*args(bits=3, g=32)) == -2
    assert q(*args(g=48)) == -3
    assert q(*args(bits=1, g=16, steps=48)) == -4
    assert q(*args(dt=7)) == -6
    assert q(*args(x=None)) == -7
    assert q(*args(fmt=9)) == -10
    g = lib.kvmix_quantized_gemv
    gargs = lambda **kw: [kw.get("g", 32), one, 128, 128, one, 1024, 16, one, one, 512, 4, kw.get("bits", 4), 0,
                          kw.get("samples", 4), kw.get("hpk", 1), 1, kw.get("K", 8), 128, one, 128, 128,
                          None, 0, None]
    assert g(*gargs(bits=0)) == -1
    assert g(*gargs(samples=3, hpk=2)) == -5
    assert g(*gargs(bits=3)) == -2
    assert g(*gargs(g=48)) == -3
    assert g(*gargs(g=4)) == -9     # a word of eight 4-bit codes would straddle two groups
    assert lib.kvmix_gemv_workspace_bytes(32, 1, 4096, 128) > 0
    assert lib.kvmix_gemv_workspace_bytes(0, 1, 4096, 128) == 0
    # the batched flush: every pair is checked before anything is launched
    from kvmix_amd import _lib

    fb = lib.kvmix_quant_pack_kv_flush_batch
    assert fb(None, None, 0, None) == 0 and fb(None, None, -1, None) == -8 and fb(None, None, 2, None) == -7
    good_k = _lib.KeyFlush(16, 1, 32, 128, 4096, 128, 32, 4, 0, 0, 16, 512, 4, 16, 16, 128, 1)
    good_v = _lib.ValueFlush(16, 1, 32, 128, 4096, 128, 32, 4, 0, 0, 16, 512, 16, 16, 16, 128, 4)
    bad_v = _lib.ValueFlush(16, 1, 32, 128, 4096, 128, 32, 5, 0, 0, 16, 512, 16, 16, 16, 128, 4)   # 5 bits
    assert _lib.flush_batch([good_k, good_k], [good_v, bad_v], None) == -1
    ka = (ctypes.POINTER(_lib.KeyFlush) * 2)(ctypes.pointer(good_k), None)
    va = (ctypes.POINTER(_lib.ValueFlush) * 2)(ctypes.pointer(good_v), ctypes.pointer(good_v))
    assert fb(ka, va, 2, None) == -7                                                                 # a pair without its key half


def test_decode_attention_host_validation_needs_no_gpu(lib):
    """kvmix_decode_attention checks its descriptor on the host before the first launch."""
    from kvmix_amd import _lib

    def desc(**kw):
        st = _lib.DecodeAttn()
        st.q, st.q_stride, st.probs, st.out = 16, 128, 16, 16
        st.k_tail, st.v_tail = 16, 16
        st.k_tail_batch_stride = st.v_tail_batch_stride = 8 * 128
        st.k_tail_token_stride = st.v_tail_token_stride = 128
        st.k_tail_slots = st.v_tail_slots = st.k_tail_len = st.v_tail_len = 8
        st.samples, st.heads, st.heads_per_kv, st.D = 4, 4, 1, 128
        st.probs_stride, st.out_stride = 8, 128
        st.k_bits = st.v_bits = 4
        st.k_group = st.v_group = 32
        for k, v in kw.items():
            setattr(st, k, v)
        return st

    call = lambda st: lib.kvmix_decode_attention(ctypes.byref(st), None, 0, None)
    assert lib.kvmix_decode_attention(None, None, 0, None) == -7
    assert call(desc(heads_per_kv=3)) == -5          # 4 rows are not a multiple of 3 heads per kv head
    assert call(desc(heads=3)) == -5
    assert call(desc(D=100)) == -9                   # head dimension must be a multiple of 8
    assert call(desc(k_tail_len=9)) == -8            # more live tokens than slots
    assert call(desc(v_tail_len=5)) == -8            # keys and values must cover the same positions
    assert call(desc(probs_stride=7)) == -8          # a probability row is 8 wide here
    assert call(desc(q=None)) == -7
    assert call(desc(k_tail=None)) == -7
    assert call(desc(samples=0)) == 0                # nothing to do
    assert lib.kvmix_decode_attention_workspace_bytes(ctypes.byref(desc())) == 0  # no quantized values: no scratch
    big = desc(v_tokens=4096)
    assert lib.kvmix_decode_attention_workspace_bytes(ctypes.byref(big)) == lib.kvmix_gemv_workspace_bytes(4, 1, 4096, 128)


def test_single_pass_attention_host_validation_needs_no_gpu(lib):
    """kvmix_decode_attention_fused: what it takes, what it refuses, how much scratch it asks for."""
    from kvmix_amd import _lib

    def desc(**kw):
        st = _lib.DecodeAttn()
        st.q, st.q_stride, st.out, st.out_stride = 16, 128, 16, 128
        st.k_tail, st.v_tail = 16, 16
        st.k_tail_batch_stride = st.v_tail_batch_stride = 8 * 128
        st.k_tail_token_stride = st.v_tail_token_stride = 128
        st.k_tail_slots = st.v_tail_slots = st.k_tail_len = st.v_tail_len = 8
        st.samples, st.heads, st.heads_per_kv, st.D = 4, 4, 1, 128
        st.k_bits = st.v_bits = 4
        st.k_group = st.v_group = 32
        for k, v in kw.items():
            setattr(st, k, v)
        return st

    sup = lambda st: lib.kvmix_decode_attention_fused_supported(ctypes.byref(st))
    call = lambda st, ws=None, n=0: lib.kvmix_decode_attention_fused(ctypes.byref(st), ws, n, None)
    assert sup(desc()) == 1
    assert sup(desc(D=64)) == 0
    assert sup(desc(heads_per_kv=3)) == 0
    assert sup(desc(k_tokens=64, k_group=64)) == 0                       # key groups other than 32
    assert sup(desc(k_tokens=64, k_bits=3, k_group=32, k_fmt=_lib.FMT_DENSE3)) == 1   # dense 3-bit keys
    assert sup(desc(k_tokens=64, k_bits=4, k_group=32, k_fmt=_lib.FMT_DENSE3)) == 0
    assert sup(desc(k_tokens=66, k_bits=3, k_group=11)) == 1             # the reference's 3-bit words
    assert sup(desc(v_tokens=32, v_bits=3)) == 0                         # 3-bit values only in the dense format
    assert sup(desc(v_tokens=32, v_bits=3, v_fmt=_lib.FMT_DENSE3)) == 1
    assert lib.kvmix_decode_attention_fused(None, None, 0, None) == -7
    assert call(desc(D=64)) == -9
    assert call(desc(heads=3)) == -5
    assert call(desc(k_tail_len=9)) == -8
    assert call(desc(v_tail_len=5)) == -8
    assert call(desc(samples=0)) == 0
    assert call(desc(k_tokens=48, k_code=16, k_scale=16, k_zero=16, k_code_row_stride=6, k_sz_row_stride=2,
                     k_tail_len=8, v_tail_slots=56, v_tail_len=56)) == -8   # 48 key tokens are not whole groups of 32
    assert call(desc(k_tokens=64, k_code=16, k_scale=16, k_zero=16, k_code_row_stride=7, k_sz_row_stride=2,
                     v_tail_slots=72, v_tail_len=72)) == -8               # a key row of 64 4-bit codes is 8 words
    assert call(desc(k_tokens=64, v_tail_slots=72, v_tail_len=72)) == -7  # quantized keys without their pointers
    # scratch: (D + 2) floats per row and slab of 512 positions (704 with the reference's 3-bit keys)
    assert lib.kvmix_decode_attention_fused_workspace_bytes(ctypes.byref(desc())) == 4 * 1 * 130 * 4
    long = desc(k_tokens=2048, v_tokens=2048)
    assert lib.kvmix_decode_attention_fused_workspace_bytes(ctypes.byref(long)) == 4 * 5 * 130 * 4
    ref3 = desc(k_tokens=2046, k_bits=3, k_group=11, v_tokens=2048)
    assert lib.kvmix_decode_attention_fused_workspace_bytes(ctypes.byref(ref3)) == 4 * 3 * 130 * 4
    assert call(long, None, 0) in (-7, -11)                               # pointers / scratch missing: refused before any launch


def test_rope_append_host_validation_needs_no_gpu(lib):
    from kvmix_amd import _lib

    def desc(**kw):
        st = _lib.RopeAppend()
        st.qkv, st.cos, st.sin, st.q_out, st.k_tail, st.v_tail = 16, 16, 16, 16, 16, 16
        st.batch, st.heads, st.kv_heads, st.D = 2, 8, 2, 128
        st.qkv_batch_stride, st.q_batch_stride = 12 * 128, 8 * 128
        st.k_tail_batch_stride = st.v_tail_batch_stride = 2 * 16 * 128
        st.k_tail_head_stride = st.v_tail_head_stride = 16 * 128
        st.k_tail_token_stride = st.v_tail_token_stride = 128
        st.k_tail_slots = st.v_tail_slots = 16
        for k, v in kw.items():
            setattr(st, k, v)
        return st

    call = lambda st: lib.kvmix_rope_append(ctypes.byref(st), None)
    assert lib.kvmix_rope_append(None, None) == -7
    assert call(desc(kv_heads=3)) == -5               # 8 query heads over 3 kv heads
    assert call(desc(D=72)) == -9                     # the head dimension must be a multiple of 16
    assert call(desc(qkv_batch_stride=11 * 128)) == -8
    assert call(desc(k_slot=16)) == -8                # host-side slot outside the window
    assert call(desc(v_slot=-1)) == -8
    assert call(desc(k_tail_token_stride=64)) == -8
    assert call(desc(cos=None)) == -7
    assert call(desc(batch=0)) == 0


def test_python_ops_reject_bad_arguments_like_the_reference():
    import KVmix

    x = torch.zeros(1, 1, 2, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="For 3-bit quantization, group_length must be 11"):
        KVmix.quantize_pack_last_dim_cuda(x, 32, 3)
    with pytest.raises(RuntimeError, match="input_tensor must be a 4D tensor"):
        KVmix.quantize_pack_last_dim_cuda(x[0], 32, 4)
    with pytest.raises(RuntimeError, match="steps must be divisible by group_length"):
        KVmix.quantize_pack_last_dim_cuda(x, 48, 4)
    with pytest.raises(RuntimeError, match="steps must be divisible by 11"):
        KVmix.quantize_pack_last_dim_cuda(x, 11, 3)
    with pytest.raises(RuntimeError, match="GPU only"):
        KVmix.quantize_pack_last_dim_cuda(x, 32, 4)  # CPU tensors are refused: there is no CPU fallback
    q = torch.zeros(1, 2, 64, 4, dtype=torch.int32)
    s = torch.zeros(1, 2, 64, 1, dtype=torch.float16)
    a = torch.zeros(1, 3, 1, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="Total heads must be divisible by KV heads"):
        KVmix.quantized_gemm(32, a, q, s, s, 4)
    with pytest.raises(RuntimeError, match="Supported quantization bits: 1, 2, 3, 4"):
        KVmix.quantized_gemm(32, a[:, :2], q, s, s, 8)
    with pytest.raises(RuntimeError, match="For 3-bit quantization, group size must be 11"):
        KVmix.quantized_gemm(32, a[:, :2], q, s, s, 3)
    with pytest.raises(RuntimeError, match="Input tensors must be 4-dimensional"):
        KVmix.quantized_gemm(32, a[0], q, s, s, 4)
    with pytest.raises(RuntimeError, match="new_steps must be divisible by group_length"):
        KVmix.process_key_quantization_cuda(x, q[..., :0], s[..., :0], s[..., :0], 48, 4)
    with pytest.raises(RuntimeError, match="head_dim must be divisible by 11"):
        KVmix.process_value_quantization_cuda(x, q[..., :0], s[..., :0], s[..., :0], 11, 3)
    assert sorted(KVmix.__all__) == sorted(["quantized_gemm", "quantize_pack_last_dim_cuda",
                                            "process_value_quantization_cuda", "process_key_quantization_cuda"])


def test_single_pass_policy_knows_the_matrix_core_steps():
    """prefer_single_pass: small steps always; large ones only where the library can run the quantized
    positions on the matrix cores (needs the quantized lengths)."""
    from kvmix_amd import ops

    small = ops.prefer_single_pass(4, 32, 32, 128, 2304, 4, 0, 32, 4, 0, 32)
    large_unknown = ops.prefer_single_pass(16, 32, 32, 128, 8192, 4, 0, 32, 4, 0, 32)
    large = ops.prefer_single_pass(16, 32, 32, 128, 8192, 4, 0, 32, 4, 0, 32, k_tokens=8064, v_tokens=8064)
    uneven = ops.prefer_single_pass(16, 32, 32, 128, 8192, 4, 0, 32, 4, 0, 32, k_tokens=8064, v_tokens=8032)
    ref3 = ops.prefer_single_pass(16, 32, 32, 128, 8192, 3, 0, 11, 4, 0, 32, k_tokens=8063, v_tokens=8064)
    few = ops.prefer_single_pass(2, 32, 32, 128, 16384, 4, 0, 32, 4, 0, 32, k_tokens=2048, v_tokens=2048)
    # (keys and values quantized to different lengths take the matrix cores over the positions both sides have
    # quantized; the reference's 3-bit keys can, but the four launches are the faster form at that size)
    assert (small, large_unknown, large, uneven, ref3, few) == (True, False, True, True, False, False)
    from kvmix_amd import _lib
    plan = _lib.attn_plan(_lib.attn_step_descriptor(16, 32, 32, 128, 3, 0, 11, 8063, 4, 0, 32, 8064, 129, 128))
    assert plan["matrix"] and not plan["recommended"]
