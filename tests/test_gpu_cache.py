"""The in-place pre-allocated cache (kvmix_amd.cache.PackedKVCache) on the GPU: every step it must
hold exactly what the reference's concatenated 9-tuple holds (models/modeling_llama_KVmix.py:
105-273, restated by the oracle), through buffer growth and tail compaction, and attention over
its views must give what attention over the tuple gives."""
import numpy as np
import pytest
import torch

from helpers import kv_like, same_bits
from test_gpu_attention import cache_np, same_cache, to_t

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k_bits,v_bits,nkv,window,capacity", [(4, 4, 4, None, 4096), (3, 2, 2, None, 16),
                                                               (2, 4, 1, None, 40), (1, 1, 4, 64, 4096),
                                                               (3, 4, 4, 48, 1)])
def test_inplace_decode_follows_the_oracle(oracle, dev, k_bits, v_bits, nkv, window, capacity):
    """100 decode steps from an empty cache; small capacities force the packed buffers to grow."""
    from kvmix_amd.attention import RESIDUAL_RATIO_BY_BITS, KVmixAttention

    rng = np.random.default_rng(k_bits * 10 + v_bits)
    B, nh, D, g = 2, 4, 128, 32
    att = KVmixAttention(k_bits, v_bits, group_size=g, residual_length=window)
    cache_o = (None,) * 8 + (0,)
    cache_t = (None,) * 8 + (0,)
    cache_i = att.new_cache(capacity=capacity)
    kr, vr = RESIDUAL_RATIO_BY_BITS[k_bits], RESIDUAL_RATIO_BY_BITS[v_bits]
    for step in range(100):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, k_bits, v_bits, kr, vr, group_size=g,
                                                           fixed_window=window)
        out_t, p_t, cache_t = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_t)
        if step == 0:
            # decode branch on an empty cache (the oracle's and the tuple path's first step)
            cache_i.append(to_t(k, dev), to_t(v, dev))
            continue
        out_i, p_i, back = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_i)
        assert back is cache_i
        same_cache(cache_i.as_tuple(), cache_o)
        assert cache_i[-1] == cache_o[-1] and len(cache_i) == 9
        # same packed bits, same kernels; torch's fp16 tail matmul may pick another routine for the views
        torch.testing.assert_close(p_i, p_t, rtol=2e-3, atol=1e-6)
        torch.testing.assert_close(out_i, out_t, rtol=2e-3, atol=2e-3)
        np.testing.assert_allclose(out_i.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3)
    assert cache_o[0] is not None and cache_o[4] is not None


@pytest.mark.parametrize("k_bits,v_bits,g", [(4, 2, 64), (2, 4, 128), (3, 1, 64)])
def test_inplace_decode_with_other_group_sizes(oracle, dev, k_bits, v_bits, g):
    """config.group_size other than 32 (the reference takes any): the flushes go through the generic
    quantizer, also in the steps where both tails flush at once, and the products through the
    generic kernel; cache bit for bit, outputs within tolerance, 300 steps."""
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(g + k_bits)
    B, nh, nkv, D, window = 2, 4, 2, 128, 2 * g
    att = KVmixAttention(k_bits, v_bits, group_size=g, residual_length=window)
    cache_o = (None,) * 8 + (0,)
    cache_i = att.new_cache(capacity=256)
    both = 0
    for step in range(300):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        before = (cache_o[0], cache_o[4])
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, k_bits, v_bits, 0.0, 0.0, group_size=g,
                                                           fixed_window=window)
        both += (cache_o[0] is not before[0]) and (cache_o[4] is not before[1])
        if step == 0:
            cache_i.append(to_t(k, dev), to_t(v, dev))
            continue
        out_i, p_i, _ = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_i)
        same_cache(cache_i.as_tuple(), cache_o)
        np.testing.assert_allclose(out_i.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3)
    assert both >= 1 or k_bits == 3  # (group-11 keys and group-64 values rarely flush in the same step)


@pytest.mark.parametrize("k_dense3,nkv", [(False, 4), (True, 2)])
def test_inplace_dense3_values_follow_the_oracle_glue(oracle, dev, k_dense3, nkv):
    """3-bit values in the dense stream (and 3-bit keys in either format) against the oracle's decode
    step carrying the same formats: cache bit for bit and outputs, 150 steps with a 64-token window."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(31 + nkv)
    B, nh, D, g, window = 2, 4, 128, 32, 64
    att = KVmixAttention(3, 3, group_size=g, residual_length=window)
    cache_i = att.new_cache(capacity=64, k_fmt=ops.FMT_DENSE3 if k_dense3 else ops.FMT_REF, v_fmt=ops.FMT_DENSE3)
    cache_o = (None,) * 8 + (0,)
    for step in range(150):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, 3, 3, 0.0, 0.0, group_size=g,
                                                           fixed_window=window, k_dense3=k_dense3, v_dense3=True)
        if step == 0:
            cache_i.append(to_t(k, dev), to_t(v, dev))
            continue
        out_i, p_i, _ = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_i)
        same_cache(cache_i.as_tuple(), cache_o)
        np.testing.assert_allclose(p_i.cpu().numpy().astype(np.float64), p_o.astype(np.float64), rtol=5e-3, atol=2e-5)
        np.testing.assert_allclose(out_i.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3)
    assert cache_o[0] is not None and cache_o[4] is not None


def test_inplace_prompt_then_decode(oracle, dev):
    """Prompt through an empty in-place cache, then decode steps whose first flush covers several
    groups; tail buffers wrap and compact on the way."""
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(5)
    B, nh, nkv, D, T, g = 1, 8, 2, 128, 300, 32
    att = KVmixAttention(3, 2, group_size=g)
    K = kv_like(rng, (B, nkv, T, D), outlier_axis=3)
    V = kv_like(rng, (B, nkv, T, D), outlier_axis=3)
    Q = rng.standard_normal((B, nh, T, D)).astype(np.float16)
    mask = np.triu(np.full((T, T), np.finfo(np.float32).min, np.float32), 1)[None, None]
    out_t, _, cache_t = att(to_t(Q, dev), to_t(K, dev), to_t(V, dev), None, attention_mask=to_t(mask, dev))
    cache_i = att.new_cache(capacity=512)
    out_i, _, back = att(to_t(Q, dev), to_t(K, dev), to_t(V, dev), cache_i, attention_mask=to_t(mask, dev))
    assert back is cache_i and torch.equal(out_i, out_t)  # the prompt branch computes on the inputs alone
    same_cache(cache_i.as_tuple(), cache_np(cache_t))
    cache_o = cache_np(cache_t)
    for step in range(200):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, 3, 2, 0.2, 0.2, group_size=g)
        out_i, p_i, _ = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_i)
        same_cache(cache_i.as_tuple(), cache_o)
        # the quantized and the fp16-tail halves of the output are rounded to fp16 before they are added
        # and may cancel; with |V| up to ~40 in the outlier channels one fp16 ulp of a half is 0.0078
        np.testing.assert_allclose(out_i.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=1.6e-2)


def test_inplace_dense3_formats(oracle, dev):
    """3-bit group-32 keys and values (the dense bit stream): the cache holds what one-shot
    quantization of the flushed tokens gives, and attention over it matches dense attention over
    the dequantized cache."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(9)
    B, nh, nkv, D, g, R = 2, 8, 2, 128, 32, 64
    att = KVmixAttention(3, 3, group_size=g, residual_length=R)
    cache = att.new_cache(capacity=128, k_fmt=ops.FMT_DENSE3, v_fmt=ops.FMT_DENSE3)
    assert cache.Kgroup_size == 32
    Ks, Vs = [], []
    for step in range(200):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        Ks.append(k)
        Vs.append(v)
        if step == 0:
            cache.append(to_t(k, dev), to_t(v, dev))
            continue
        out, p, _ = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache)
    Kall, Vall = np.concatenate(Ks, 2), np.concatenate(Vs, 2)
    kc, k_tail, ks, km, vc, v_tail, vs, vm, n = cache.as_tuple()
    assert n == 200 and cache.k_tokens == cache.v_tokens == 192  # three flushes of 64
    tq = cache.k_tokens
    okc, oks, okm = oracle.quantize_pack_dense3(np.ascontiguousarray(Kall[:, :, :tq].transpose(0, 1, 3, 2)), 32)
    ovc, ovs, ovm = oracle.quantize_pack_dense3(np.ascontiguousarray(Vall[:, :, :tq]), 32)
    # flushes of 64 tokens = two groups per flush: group boundaries equal the one-shot ones
    for got, want in ((kc, okc), (ks, oks), (km, okm), (vc, ovc), (vs, ovs), (vm, ovm)):
        assert same_bits(got.cpu().numpy(), want)
    assert same_bits(k_tail.cpu().numpy(), Kall[:, :, tq:]) and same_bits(v_tail.cpu().numpy(), Vall[:, :, tq:])
    # last step's output against float64 attention over the dequantized cache
    Kd = np.concatenate([oracle.dequantize_dense3_np(okc, oks, okm).transpose(0, 1, 3, 2), Kall[:, :, tq:].astype(np.float64)], 2)
    Vd = np.concatenate([oracle.dequantize_dense3_np(ovc, ovs, ovm), Vall[:, :, tq:].astype(np.float64)], 2)
    rep = nh // nkv
    w = np.einsum("bhqd,bhtd->bhqt", q.astype(np.float64), np.repeat(Kd, rep, 1)) / np.sqrt(D)
    w = np.exp(w - w.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    want = np.einsum("bhqt,bhtd->bhqd", w, np.repeat(Vd, rep, 1))
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want, rtol=1e-2, atol=1e-2)


def test_append_costs_no_reallocation_within_capacity(dev):
    """Within the stated capacity the packed buffers never move (appends are in place)."""
    from kvmix_amd.cache import PackedKVCache

    cache = PackedKVCache(4, 2, residual_length=32, capacity=1024)
    g = torch.Generator(device="cpu").manual_seed(0)
    ptrs = set()
    for step in range(700):
        k = torch.randn(1, 2, 1, 128, generator=g).to(torch.float16).to(dev)
        cache.append(k, k)
        if cache.k_tokens:
            ptrs.add((cache._k[0].data_ptr(), cache._v[0].data_ptr()))
    assert cache.k_tokens == 672 and cache.kv_seq_len == 700 and len(ptrs) == 1


def test_cache_argument_errors(dev):
    from kvmix_amd import ops
    from kvmix_amd.cache import PackedKVCache

    with pytest.raises(RuntimeError, match="Supported quantization bits"):
        PackedKVCache(5, 2)
    with pytest.raises(RuntimeError, match="FMT_DENSE3"):
        PackedKVCache(4, 3)
    PackedKVCache(4, 3, v_fmt=ops.FMT_DENSE3)
    c = PackedKVCache(4, 4)
    x = torch.zeros(1, 1, 1, 128, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        c.append(x, x)
    with pytest.raises(RuntimeError, match="Half"):
        c.append(x.to(dev).float(), x.to(dev).float())
    with pytest.raises(RuntimeError, match="equal shape"):
        c.append(x.to(dev), x.to(dev)[:, :, :, :64])


def test_a_prompt_does_not_size_the_tails(dev):
    """The fp16 tails hold what the policy keeps, not the prompt: a long prompt is quantized straight
    from the incoming tensors (the cache would otherwise be larger than the fp16 cache it replaces)."""
    from kvmix_amd.cache import PackedKVCache

    gen = torch.Generator(device=dev).manual_seed(3)
    k = torch.randn(2, 2, 1500, 128, device=dev, generator=gen).half()
    v = torch.randn(2, 2, 1500, 128, device=dev, generator=gen).half()
    fixed = PackedKVCache(4, 2, residual_length=128, capacity=2048)
    fixed.append(k.transpose(1, 2).contiguous().transpose(1, 2), v, prompt=True)  # (a strided view, as a model hands it over)
    assert fixed.k_tokens == 1344 and fixed.v_tokens == 1344 and len(fixed.as_tuple()[1][0, 0]) == 156
    assert fixed._k_tail.buf.shape[2] <= 128 + 32 + 64 and fixed._v_tail.buf.shape[2] <= 128 + 32 + 64
    for _ in range(300):  # decode steps through several flushes and compactions: the buffers stay that size
        fixed.append(k[:, :, :1], v[:, :, :1])
    assert fixed.kv_seq_len == 1800 and fixed._k_tail.buf.shape[2] <= 128 + 32 + 64
    ratio = PackedKVCache(4, 2, k_residual_ratio=0.2, v_residual_ratio=0.1, capacity=2048)
    ratio.append(k, v, prompt=True)
    assert ratio._k_tail.len == 1500 - ratio.k_tokens and ratio._k_tail.buf.shape[2] <= ratio._k_tail.len + 64
