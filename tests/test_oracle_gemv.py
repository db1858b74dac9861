"""Pins the CPU oracle's dequant-GEMV, append variants and decode-step glue against
library routines (float64 matmul), special cases with closed forms, and identities.
Reference: quant_cuda/csrc/dequantization_gemv_cuda.cu:7-248,
quant_cuda/csrc/quantization_cuda.cu:298-537, models/modeling_llama_KVmix.py:105-211."""
import math

import numpy as np
import pytest

from helpers import gemv_close, kv_like, same_bits

CASES = [(4, 32), (2, 32), (1, 32), (3, 11), (4, 8), (2, 16), (1, 64)]


def make_packed(oracle, rng, B, Hkv, K, N, bits, g, along_n=True):
    """Quantize a random weight [B,Hkv,K,N] along N -> (w_fp16, code, scale, zero)."""
    w = kv_like(rng, (B, Hkv, K, N), outlier_axis=2, n_outliers=2)
    code, scale, zero = oracle.quantize_pack_last_dim(w, g, bits)
    return w, code, scale, zero


@pytest.mark.parametrize("bits,g", CASES)
@pytest.mark.parametrize("shape", ["qk", "pv"])
def test_gemv_equals_float64_matmul_of_dequantized(oracle, bits, g, shape):
    rng = np.random.default_rng(bits * 31 + g)
    unit = int(np.lcm(g, oracle.values_per_word(bits)))
    if shape == "qk":
        K, N = 64, unit * 12
    else:
        K, N = 300, unit * (2 if bits == 3 else 4)
    B, nh, nkv = 2, 4, 2
    w, code, scale, zero = make_packed(oracle, rng, B, nkv, K, N, bits, g)
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    deq = oracle.dequantize_np(code, scale, zero, bits, g).astype(np.float64)  # numpy twin
    assert same_bits(oracle.dequantize(code, scale, zero, bits, g), deq.astype(np.float32))
    want64 = np.einsum("bhmk,bhkn->bhmn", x.astype(np.float64), np.repeat(deq, nh // nkv, axis=1))
    abs64 = np.einsum("bhmk,bhkn->bhmn", np.abs(x.astype(np.float64)), np.abs(np.repeat(deq, nh // nkv, axis=1)))
    for mode in (oracle.GEMM_REFERENCE_ORDER, oracle.GEMM_SEQUENTIAL):
        out, o64, a64 = oracle.quantized_gemm(g, x, code, scale, zero, bits, mode=mode, want_f64=True)
        assert out.dtype == np.float16 and out.shape == (B, nh, 1, N)
        np.testing.assert_allclose(o64, want64, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(a64, abs64, rtol=1e-12, atol=1e-12)
        ok, worst = gemv_close(out, want64, abs64)
        assert ok, worst


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32), (3, 11)])
def test_gemv_special_cases(oracle, bits, g):
    rng = np.random.default_rng(bits)
    B, nh, K = 1, 2, 40
    N = int(np.lcm(g, oracle.values_per_word(bits))) * 3
    qmax = (1 << bits) - 1
    q = rng.integers(0, qmax + 1, size=(B, nh, K, N))
    if bits == 3:
        q[..., 10::11] &= 3
    code = oracle.pack_np(q, bits)
    ones = np.ones((B, nh, K, N // g), np.float16)
    zero = rng.standard_normal((B, nh, K, N // g)).astype(np.float16)
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    # scale = 0: out[n] = sum_k x[k] * zero[k, n/g]
    out = oracle.quantized_gemm(g, x, code, np.zeros_like(ones), zero, bits, mode=oracle.GEMM_SEQUENTIAL,
                                want_f64=True)[1]
    want = np.einsum("bhmk,bhkg->bhmg", x.astype(np.float64), zero.astype(np.float64))
    np.testing.assert_allclose(out, np.repeat(want, g, axis=-1), rtol=1e-12, atol=1e-12)
    # all-ones x, scale 1, zero 0: column sums of the integer codes, exactly
    out = oracle.quantized_gemm(g, np.ones_like(x), code, ones, np.zeros_like(ones), bits)
    assert np.array_equal(out.astype(np.int64)[:, :, 0], q.sum(axis=2))
    # one-hot x: the dequantized row, rounded to fp16
    scale = (rng.random((B, nh, K, N // g)) + 0.5).astype(np.float16)
    e = np.zeros_like(x)
    e[..., 7] = 1
    out = oracle.quantized_gemm(g, e, code, scale, zero, bits)
    row = (np.repeat(scale.astype(np.float32), g, -1) * q + np.repeat(zero.astype(np.float32), g, -1))[:, :, 7]
    assert same_bits(out[:, :, 0], row.astype(np.float16))


def test_gemv_gqa_equals_repeated_mha(oracle):
    rng = np.random.default_rng(11)
    B, nh, nkv, K, N = 2, 8, 2, 32, 128
    _, code, scale, zero = make_packed(oracle, rng, B, nkv, K, N, 4, 32)
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    a = oracle.quantized_gemm(32, x, code, scale, zero, 4)
    rep = nh // nkv
    b = oracle.quantized_gemm(32, x, oracle.repeat_kv(code, rep), oracle.repeat_kv(scale, rep),
                              oracle.repeat_kv(zero, rep), 4)
    assert same_bits(a, b)


def test_gemv_errors(oracle):
    x = np.zeros((1, 3, 1, 8), np.float16)
    code = np.zeros((1, 2, 8, 4), np.int32)
    sz = np.zeros((1, 2, 8, 1), np.float16)
    with pytest.raises(RuntimeError, match="divisible by KV heads"):
        oracle.quantized_gemm(32, x, code, sz, sz, 4)
    with pytest.raises(RuntimeError, match="1, 2, 3, 4"):
        oracle.quantized_gemm(32, x[:, :2], code, sz, sz, 5)
    with pytest.raises(RuntimeError, match="group size must be 11"):
        oracle.quantized_gemm(32, x[:, :2], code, sz, sz, 3)
    with pytest.raises(RuntimeError, match="4-dimensional"):
        oracle.quantized_gemm(32, x[0], code, sz, sz, 4)


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32), (3, 11), (4, 8)])
def test_key_append_is_one_shot_on_the_new_chunk(oracle, bits, g):
    rng = np.random.default_rng(bits + 40)
    unit = int(np.lcm(g, oracle.values_per_word(bits)))
    B, H, D = 1, 2, 6
    old = kv_like(rng, (B, H, D, unit * 2))
    new = kv_like(rng, (B, H, D, unit * 3))
    c0, s0, z0 = oracle.quantize_pack_last_dim(old, g, bits, oracle.SCALE_DIVIDE)
    c1, s1, z1 = oracle.quantize_pack_last_dim(new, g, bits, oracle.SCALE_DIVIDE)
    c, s, z = oracle.process_key_quantization(new, c0, s0, z0, g, bits)
    assert same_bits(c, np.concatenate([c0, c1], -1))
    assert same_bits(s, np.concatenate([s0, s1], -1))
    assert same_bits(z, np.concatenate([z0, z1], -1))
    # empty history
    e = oracle.process_key_quantization(new, c0[..., :0], s0[..., :0], z0[..., :0], g, bits)
    assert same_bits(e[0], c1) and same_bits(e[1], s1) and same_bits(e[2], z1)


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32), (4, 16)])
def test_value_append_is_one_shot_on_the_new_chunk(oracle, bits, g):
    rng = np.random.default_rng(bits + 50)
    B, H, D = 2, 2, 64
    old = kv_like(rng, (B, H, 5, D))
    new = kv_like(rng, (B, H, 7, D))
    c0, s0, z0 = oracle.quantize_pack_last_dim(old, g, bits, oracle.SCALE_DIVIDE)
    c1, s1, z1 = oracle.quantize_pack_last_dim(new, g, bits, oracle.SCALE_DIVIDE)
    c, s, z = oracle.process_value_quantization(new, c0, s0, z0, g, bits)
    assert same_bits(c, np.concatenate([c0, c1], 2))
    assert same_bits(s, np.concatenate([s0, s1], 2))
    assert same_bits(z, np.concatenate([z0, z1], 2))


def test_value_append_3bit_placeholder_keeps_low_two_bits(oracle):
    """quantization_cuda.cu:282-289 with j == 10: code clamped to 0..7, shifted by 30."""
    D = 22
    x = np.zeros((1, 1, 1, D), np.float32)
    x[0, 0, 0, :11] = [0, 7, 1, 2, 3, 4, 5, 6, 7, 0, 6]    # 11th code 6 -> 6 & 3 = 2
    x[0, 0, 0, 11:] = [0, 7, 0, 0, 0, 0, 0, 0, 0, 0, 5]    # 11th code 5 -> 1
    e = np.zeros((1, 1, 0, 2), np.int32)
    ef = np.zeros((1, 1, 0, 2), np.float32)
    c, s, z = oracle.process_value_quantization(x, e, ef, ef, 11, 3)
    w = np.ascontiguousarray(c).view(np.uint32)[0, 0, 0]
    hand0 = sum(v << (3 * i) for i, v in enumerate([0, 7, 1, 2, 3, 4, 5, 6, 7, 0])) | (2 << 30)
    hand1 = (7 << 3) | (1 << 30)
    assert int(w[0]) == hand0 and int(w[1]) == hand1
    assert np.all(s == 1.0) and np.all(z == 0.0)


def dense_attention(q, K, V):
    """fp64 softmax attention; q [B,nh,1,D], K,V [B,nh,T,D]."""
    w = np.einsum("bhqd,bhtd->bhqt", q, K) / math.sqrt(q.shape[-1])
    w = w - w.max(-1, keepdims=True)
    p = np.exp(w)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqt,bhtd->bhqd", p, V), p


@pytest.mark.parametrize("k_bits,v_bits,nkv", [(4, 4, 4), (3, 2, 2), (2, 4, 1), (1, 1, 4)])
def test_decode_steps_match_dense_attention_on_dequantized_cache(oracle, k_bits, v_bits, nkv):
    rng = np.random.default_rng(k_bits * 7 + v_bits)
    B, nh, D, g = 1, 4, 64, 32
    rep = nh // nkv
    cache = (None,) * 8 + (0,)
    hist_k, hist_v = [], []
    ratios = {4: 0.3, 3: 0.2, 2: 0.2, 1: 0.1}
    for step in range(90):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        hist_k.append(k)
        hist_v.append(v)
        out, p, cache = oracle.attention_decode_step(q, k, v, cache, k_bits, v_bits, ratios[k_bits],
                                                     ratios[v_bits], group_size=g)
        kc, k_tail, ks, km, vc, v_tail, vs, vm, seen = cache
        assert seen == step + 1
        kg = 11 if k_bits == 3 else g
        nqk = 0 if kc is None else ks.shape[-1] * kg
        nqv = 0 if vc is None else vc.shape[2]
        assert nqk + k_tail.shape[2] == step + 1 and nqv + v_tail.shape[2] == step + 1
        assert nqk % kg == 0 and nqv % g == 0
        # rebuild K, V as the cache represents them
        Kd = k_tail.astype(np.float64)
        if kc is not None:
            kq = oracle.dequantize_np(kc, ks, km, k_bits, kg).astype(np.float64).transpose(0, 1, 3, 2)
            Kd = np.concatenate([kq, Kd], 2)
        Vd = v_tail.astype(np.float64)
        if vc is not None:
            Vd = np.concatenate([oracle.dequantize_np(vc, vs, vm, v_bits, g).astype(np.float64), Vd], 2)
        want, pw = dense_attention(q.astype(np.float64), np.repeat(Kd, rep, 1), np.repeat(Vd, rep, 1))
        np.testing.assert_allclose(p.astype(np.float64), pw, rtol=4e-3, atol=2e-4)
        np.testing.assert_allclose(out.astype(np.float64), want, rtol=4e-3, atol=4e-3)
    assert cache[0] is not None and cache[4] is not None  # both sides did flush at some point
    # and the quantized part really is the quantization of the oldest tokens
    allk = np.concatenate(hist_k, 2)
    kg = 11 if k_bits == 3 else g
    nqk = cache[2].shape[-1] * kg
    c, s, m = oracle.quantize_pack_last_dim(np.ascontiguousarray(allk[:, :, :kg].transpose(0, 1, 3, 2)), kg, k_bits)
    assert same_bits(cache[0][..., : c.shape[-1]], c)


def test_flush_rule(oracle):
    # models/modeling_llama_KVmix.py:119-127: keep=int(ratio*L); flush floor((L-keep)/g)*g
    assert oracle.flush_length(39, 0.2, 32) == 32
    assert oracle.flush_length(38, 0.2, 32) == 0
    assert oracle.flush_length(416, 0.2, 32) == 320
    assert oracle.flush_length(13, 0.2, 11) == 11
    assert oracle.flush_length(5, 0.3, 32) == 0


def test_prompt_attention_against_float64_and_fully_masked_rows(oracle):
    """attention_prompt: causal rows against dense float64 attention; a row whose every position is
    masked gives the plain mean of V when the mask is half (every fp16 logit ends at the lowest finite
    half) or holds the lowest finite float (the logit is absorbed), but keeps its logits' differences
    when a float mask holds -65504 -- the three cases of models/modeling_llama_KVmix.py:259-262."""
    rng = np.random.default_rng(12)
    B, nh, nkv, T, D, pad = 2, 4, 2, 40, 64, 9
    q = rng.standard_normal((B, nh, T, D)).astype(np.float16)
    k = rng.standard_normal((B, nkv, T, D)).astype(np.float16)
    v = rng.standard_normal((B, nkv, T, D)).astype(np.float16)
    rep = nh // nkv
    mean_v = np.repeat(v.astype(np.float64), rep, 1).mean(2)                       # [B, nh, D]
    for dtype, low in ((np.float16, np.finfo(np.float16).min), (np.float32, np.finfo(np.float32).min),
                       (np.float32, np.float32(np.finfo(np.float16).min))):
        mask = np.triu(np.full((T, T), low, dtype), 1)[None, None].repeat(B, 0)
        mask[1, :, :, :pad] = low
        out, p = oracle.attention_prompt(q, k, v, mask)
        assert out.dtype == np.float16 and p.dtype == np.float16 and p.shape == (B, nh, T, T)
        # rows with at least one open position: dense float64 attention over the open positions
        m64 = np.where(mask.astype(np.float64) < -1e4, -np.inf, 0.0)
        w = np.einsum("bhqd,bhtd->bhqt", q.astype(np.float64), np.repeat(k.astype(np.float64), rep, 1)) / np.sqrt(D) + m64
        with np.errstate(invalid="ignore"):
            e = np.exp(w - w.max(-1, keepdims=True))
            want = np.einsum("bhqt,bhtd->bhqd", e / e.sum(-1, keepdims=True), np.repeat(v.astype(np.float64), rep, 1))
        live = np.ones((B, T), bool)
        live[1, :pad] = False
        np.testing.assert_allclose(out.astype(np.float64)[live.nonzero()[0], :, live.nonzero()[1]],
                                   want[live.nonzero()[0], :, live.nonzero()[1]], rtol=1e-2, atol=1e-2)
        dead = out[1, :, :pad].astype(np.float64)
        uniform = np.allclose(dead, mean_v[1][:, None, :], rtol=1e-2, atol=1e-2)
        absorbed = dtype == np.float16 or low == np.finfo(np.float32).min
        assert uniform == absorbed, (dtype, low)


@pytest.mark.parametrize("k_dense3,v_dense3", [(True, True), (False, True), (True, False)])
def test_decode_steps_with_dense3_sides_match_dense_attention(oracle, k_dense3, v_dense3):
    """The decode step with 3-bit sides kept in the dense stream: the cache holds what one-shot dense
    3-bit quantization of the flushed tokens gives, and the step equals dense float64 attention over
    the dequantized cache (the same pin as for the reference's formats)."""
    rng = np.random.default_rng(13)
    B, nh, nkv, D, g, window = 1, 4, 2, 128, 32, 64
    rep = nh // nkv
    cache = (None,) * 8 + (0,)
    hist_k, hist_v = [], []
    for step in range(140):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        hist_k.append(k)
        hist_v.append(v)
        out, p, cache = oracle.attention_decode_step(q, k, v, cache, 3, 3 if v_dense3 else 4, 0.0, 0.0, group_size=g,
                                                     fixed_window=window, k_dense3=k_dense3, v_dense3=v_dense3)
        kc, k_tail, ks, km, vc, v_tail, vs, vm, seen = cache
        kg = g if k_dense3 else 11
        Kd = k_tail.astype(np.float64)
        if kc is not None:
            kq = oracle.dequantize_dense3_np(kc, ks, km, g) if k_dense3 else oracle.dequantize_np(kc, ks, km, 3, 11)
            Kd = np.concatenate([kq.astype(np.float64).transpose(0, 1, 3, 2), Kd], 2)
        Vd = v_tail.astype(np.float64)
        if vc is not None:
            vq = oracle.dequantize_dense3_np(vc, vs, vm, g) if v_dense3 else oracle.dequantize_np(vc, vs, vm, 4, g)
            Vd = np.concatenate([vq.astype(np.float64), Vd], 2)
        assert Kd.shape[2] == step + 1 and Vd.shape[2] == step + 1
        want, pw = dense_attention(q.astype(np.float64), np.repeat(Kd, rep, 1), np.repeat(Vd, rep, 1))
        np.testing.assert_allclose(p.astype(np.float64), pw, rtol=4e-3, atol=2e-4)
        np.testing.assert_allclose(out.astype(np.float64), want, rtol=4e-3, atol=4e-3)
    kc, _, ks, km, vc, _, vs, vm, _ = cache
    assert kc is not None and vc is not None
    allk, allv = np.concatenate(hist_k, 2), np.concatenate(hist_v, 2)
    if k_dense3:
        c, s, m = oracle.quantize_pack_dense3(np.ascontiguousarray(allk[:, :, :64].transpose(0, 1, 3, 2)), g)
        assert same_bits(kc[..., : c.shape[-1]], c) and same_bits(ks[..., :2], s) and same_bits(km[..., :2], m)
    if v_dense3:
        c, s, m = oracle.quantize_pack_dense3(np.ascontiguousarray(allv[:, :, :64]), g)
        assert same_bits(vc[:, :, :64], c) and same_bits(vs[:, :, :64], s) and same_bits(vm[:, :, :64], m)
    # compute_output=False leaves the cache exactly as the full step does
    a = oracle.attention_decode_step(q, k, v, cache, 3, 3 if v_dense3 else 4, 0.0, 0.0, group_size=g, fixed_window=window,
                                     k_dense3=k_dense3, v_dense3=v_dense3)[2]
    b = oracle.attention_decode_step(q, k, v, cache, 3, 3 if v_dense3 else 4, 0.0, 0.0, group_size=g, fixed_window=window,
                                     k_dense3=k_dense3, v_dense3=v_dense3, compute_output=False)
    assert b[0] is None and b[1] is None
    for x, y in zip(a, b[2]):
        assert (x is None and y is None) or (isinstance(x, int) and x == y) or same_bits(x, y)
