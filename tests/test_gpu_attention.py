"""The attention glue (kvmix_amd.attention.KVmixAttention) on the GPU against the oracle's
restatement of models/modeling_llama_KVmix.py:105-283: same flush decisions, bit-exact cache
contents, outputs within tolerance, for MHA and GQA, ratio and fixed-window policies."""
import numpy as np
import pytest
import torch

from helpers import kv_like, same_bits

pytestmark = pytest.mark.gpu


def to_t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def cache_np(c):
    return tuple(x.cpu().numpy() if torch.is_tensor(x) else x for x in c)


def same_cache(got, want):
    for i, (g, w) in enumerate(zip(cache_np(got), want)):
        if w is None or isinstance(w, int):
            assert g == w or (g is None and w is None), i
        else:
            assert same_bits(g, w), i


@pytest.mark.parametrize("k_bits,v_bits,nkv,window", [(4, 4, 4, None), (3, 2, 2, None), (2, 4, 1, None),
                                                      (1, 1, 4, None), (4, 2, 2, 64), (3, 4, 4, 48)])
def test_decode_steps_follow_the_oracle(oracle, dev, k_bits, v_bits, nkv, window):
    from kvmix_amd.attention import RESIDUAL_RATIO_BY_BITS, KVmixAttention

    rng = np.random.default_rng(k_bits * 10 + v_bits)
    B, nh, D, g = 2, 4, 128, 32
    att = KVmixAttention(k_bits, v_bits, group_size=g, residual_length=window)
    cache_o = (None,) * 8 + (0,)
    cache_g = (None,) * 8 + (0,)
    kr, vr = RESIDUAL_RATIO_BY_BITS[k_bits], RESIDUAL_RATIO_BY_BITS[v_bits]
    for step in range(100):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, k_bits, v_bits, kr, vr, group_size=g,
                                                           fixed_window=window)
        out_g, p_g, cache_g = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache_g)
        same_cache(cache_g, cache_o)
        np.testing.assert_allclose(p_g.cpu().numpy().astype(np.float64), p_o.astype(np.float64), rtol=5e-3, atol=2e-5)
        np.testing.assert_allclose(out_g.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3)
    assert cache_o[0] is not None and cache_o[4] is not None


def test_prompt_then_decode(oracle, dev):
    """Prompt branch: dense attention output, cache = oldest tokens quantized by the ratio rule
    (models/modeling_llama_KVmix.py:213-273); the first decode step then flushes several groups."""
    from kvmix_amd.attention import KVmixAttention, flush_length

    rng = np.random.default_rng(3)
    B, nh, nkv, D, T, g = 1, 8, 2, 128, 300, 32
    att = KVmixAttention(3, 2, group_size=g)
    K = kv_like(rng, (B, nkv, T, D), outlier_axis=3)
    V = kv_like(rng, (B, nkv, T, D), outlier_axis=3)
    Q = rng.standard_normal((B, nh, T, D)).astype(np.float16)
    mask = np.triu(np.full((T, T), np.finfo(np.float32).min, np.float32), 1)[None, None]
    out, p, cache = att(to_t(Q, dev), to_t(K, dev), to_t(V, dev), None, attention_mask=to_t(mask, dev))
    nqk = flush_length(T, 0.2, 11)
    nqv = flush_length(T, 0.2, 32)
    assert nqk == 231 and nqv == 224 and cache[-1] == T
    kc, ks, km = oracle.quantize_pack_last_dim(np.ascontiguousarray(K[:, :, :nqk].transpose(0, 1, 3, 2)), 11, 3)
    vc, vs, vm = oracle.quantize_pack_last_dim(np.ascontiguousarray(V[:, :, :nqv]), 32, 2)
    same_cache(cache, (kc, K[:, :, nqk:], ks, km, vc, V[:, :, nqv:], vs, vm, T))
    # dense causal attention in float64
    rep = nh // nkv
    w = np.einsum("bhqd,bhtd->bhqt", Q.astype(np.float64), np.repeat(K.astype(np.float64), rep, 1)) / np.sqrt(D) + mask
    w = np.exp(w - w.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    want = np.einsum("bhqt,bhtd->bhqd", w, np.repeat(V.astype(np.float64), rep, 1))
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want, rtol=1e-2, atol=5e-2)  # fp16 probabilities, |V| up to ~40 in the outlier channels
    # decode continues from the prompt cache on both sides
    cache_o = cache_np(cache)
    for step in range(3):
        k = kv_like(rng, (B, nkv, 1, D))
        v = kv_like(rng, (B, nkv, 1, D))
        q = rng.standard_normal((B, nh, 1, D)).astype(np.float16)
        out_o, p_o, cache_o = oracle.attention_decode_step(q, k, v, cache_o, 3, 2, 0.2, 0.2, group_size=g)
        out_g, p_g, cache = att(to_t(q, dev), to_t(k, dev), to_t(v, dev), cache)
        same_cache(cache, cache_o)
        np.testing.assert_allclose(out_g.cpu().numpy().astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3)


def test_prompt_left_padding_rows_are_uniform_in_both_prompt_forms(dev):
    """A left-padded prompt: the pad query positions see nothing but masked keys.  The reference's fp16
    logits of such a row all end at the lowest finite value (mask added, then clamped;
    models/modeling_llama_KVmix.py:259-262), so the row's output is the plain mean of V over all
    positions.  Both prompt forms (probabilities asked for or not) must give that, and must agree
    on the other rows."""
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(11)
    B, nh, nkv, D, T, pad = 2, 4, 2, 128, 96, 17
    att = KVmixAttention(4, 2, group_size=32)
    K = to_t(kv_like(rng, (B, nkv, T, D)), dev)
    V = to_t(kv_like(rng, (B, nkv, T, D)), dev)
    Q = to_t((4 * rng.standard_normal((B, nh, T, D))).astype(np.float16), dev)
    low = np.finfo(np.float32).min
    mask = np.triu(np.full((T, T), low, np.float32), 1)[None, None].repeat(B, 0)
    mask[1, :, :, :pad] = low  # sequence 1 is left-padded: its first `pad` keys are masked for every query
    mask = to_t(mask, dev)
    out_w, p, _ = att(Q, K, V, None, attention_mask=mask, use_cache=False, need_weights=True)
    out_f, none, _ = att(Q, K, V, None, attention_mask=mask, use_cache=False, need_weights=False)
    assert none is None and p is not None
    mean_v = V[1].float().mean(dim=1).repeat_interleave(nh // nkv, dim=0)  # [nh, D]
    for out in (out_w, out_f):
        got = out[1, :, :pad].float()
        assert torch.allclose(got, mean_v[:, None, :].expand_as(got), rtol=2e-2, atol=2e-2)
    assert torch.allclose(out_w.float(), out_f.float(), rtol=2e-2, atol=3e-2)


def test_mask_shape_error(dev):
    from kvmix_amd.attention import KVmixAttention

    att = KVmixAttention(4, 4)
    q = torch.zeros(1, 2, 1, 128, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError, match="does not match"):
        att(q, q, q, (None,) * 8 + (0,), attention_mask=torch.zeros(1, 1, 1, 7, device=dev))


def _cache_after_steps(att, dev, rng, B, nh, nkv, D, steps):
    cache = att.new_cache(capacity=512)
    for step in range(steps):
        k = to_t(kv_like(rng, (B, nkv, 1, D)), dev)
        v = to_t(kv_like(rng, (B, nkv, 1, D)), dev)
        cache.append(k, v)
    return cache


@pytest.mark.parametrize("k_bits,v_bits,nkv", [(4, 2, 4), (3, 4, 2), (1, 2, 1)])
def test_library_step_equals_the_torch_composition(dev, k_bits, v_bits, nkv):
    """ops.decode_attention against the same step composed from quantized_gemm and torch's matmul /
    cat / softmax (the way the reference composes it), with and without a padding mask."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(70 + k_bits)
    B, nh, D = 2, 4, 128
    att = KVmixAttention(k_bits, v_bits, residual_length=48)
    cache = _cache_after_steps(att, dev, rng, B, nh, nkv, D, 150)
    kc, k_tail, ks, km, vc, v_tail, vs, vm, n = cache.as_tuple()
    assert kc is not None and vc is not None and k_tail.shape[2] > 0
    q = to_t(rng.standard_normal((B, nh, 1, D)).astype(np.float16), dev)
    mask = torch.zeros(B, 1, 1, n, device=dev)
    mask[1, :, :, :40] = torch.finfo(torch.float32).min  # left padding of the second sequence
    for m in (None, mask):
        out_l, p_l = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), k_tail, v_tail, cache.Kgroup_size, k_bits,
                                          cache.Vgroup_size, v_bits, attention_mask=m)
        out_t, p_t = att._decode_with_torch_glue(q, kc, ks, km, k_tail, vc, vs, vm, v_tail, cache.Kgroup_size, 0, 0,
                                                 nh // nkv, m)
        torch.testing.assert_close(p_l, p_t, rtol=5e-3, atol=2e-5)
        torch.testing.assert_close(out_l, out_t, rtol=5e-3, atol=5e-3)
        if m is not None:
            assert float(p_l[1, :, :, :40].abs().max()) == 0.0
        assert abs(float(p_l.float().sum(-1).mean()) - 1.0) < 2e-3


def test_tail_windows_with_device_side_lengths(dev):
    """Fixed-size tail windows whose live lengths are read from device memory give, position by
    position, the bits of the exact-size call; slots past the lengths hold probability zero."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(81)
    B, nh, nkv, D, R = 2, 8, 2, 128, 64
    att = KVmixAttention(3, 2, residual_length=R)   # reference 3-bit keys: the two tails differ in length
    cache = _cache_after_steps(att, dev, rng, B, nh, nkv, D, 200)
    kc, k_tail, ks, km, vc, v_tail, vs, vm, n = cache.as_tuple()
    lk, lv = k_tail.shape[2], v_tail.shape[2]
    assert lk != lv and cache.k_tokens != cache.v_tokens
    q = to_t(rng.standard_normal((B, nh, 1, D)).astype(np.float16), dev)
    args = (cache.Kgroup_size, 3, cache.Vgroup_size, 2)
    out_e, p_e = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), k_tail, v_tail, *args)
    kwin, vwin, nk, nv = cache.tail_windows(R)
    assert (nk, nv) == (lk, lv)
    kwin[:, :, lk:] = 1000.0   # whatever lies in the unused slots must not matter
    vwin[:, :, lv:] = -1000.0
    klen = torch.tensor([lk], dtype=torch.int64, device=dev)
    vlen = torch.tensor([lv], dtype=torch.int64, device=dev)
    out_w, p_w = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), kwin, vwin, *args, k_tail_len=klen, v_tail_len=vlen)
    assert p_w.shape[-1] == max(cache.k_tokens, cache.v_tokens) + R
    assert torch.equal(p_w[..., :n], p_e) and float(p_w[..., n:].abs().max()) == 0.0
    assert torch.equal(out_w, out_e)
    # host-side lengths for the same windows
    out_h, p_h = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), kwin, vwin, *args, k_tail_len=lk, v_tail_len=lv)
    assert torch.equal(out_h, out_e) and torch.equal(p_h[..., :n], p_e)


def test_library_step_without_a_quantized_part_and_argument_errors(dev):
    from kvmix_amd import ops

    rng = np.random.default_rng(5)
    B, nh, nkv, D, L = 1, 4, 2, 128, 9
    q = to_t(rng.standard_normal((B, nh, 1, D)).astype(np.float16), dev)
    k = to_t(rng.standard_normal((B, nkv, L, D)).astype(np.float16), dev)
    v = to_t(rng.standard_normal((B, nkv, L, D)).astype(np.float16), dev)
    out, p = ops.decode_attention(q, None, None, k, v, 32, 4, 32, 4)
    kk = k.float().repeat_interleave(nh // nkv, 1)
    vv = v.float().repeat_interleave(nh // nkv, 1)
    w = torch.softmax((q.float() @ kk.transpose(2, 3)).half().float() / np.float32(np.sqrt(D)), -1)
    torch.testing.assert_close(p.float(), w, rtol=2e-3, atol=2e-5)
    torch.testing.assert_close(out.float(), w.half().float() @ vv, rtol=2e-3, atol=2e-3)
    with pytest.raises(RuntimeError, match="one query position"):
        ops.decode_attention(q.expand(B, nh, 2, D), None, None, k, v, 32, 4, 32, 4)
    with pytest.raises(RuntimeError, match="KV heads"):
        ops.decode_attention(q[:, :3], None, None, k, v, 32, 4, 32, 4)
    with pytest.raises(RuntimeError, match="attention_mask"):
        ops.decode_attention(q, None, None, k, v, 32, 4, 32, 4, attention_mask=torch.zeros(B, 1, 1, L + 1, device=dev))
    with pytest.raises(RuntimeError):  # keys and values must cover the same positions
        ops.decode_attention(q, None, None, k, v[:, :, :5], 32, 4, 32, 4)


def test_full_size_step_properties_b16_t8192(dev):
    """The library step at the size the target is quoted on (B=16, 32 heads, 8064 quantized + 128 fp16
    tokens, 4-bit keys, 2-bit values), through properties that need no CPU pass over 1.3 GB:
    probabilities are non-negative and sum to one, the step equals its composition from the two
    GEMVs and torch's matmul / softmax, and it is linear in V's zero points (adding a constant c
    to every zero point of the quantized values adds c * sum of their probabilities)."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    torch.manual_seed(11)
    B, H, D, Tq, L = 16, 32, 128, 8064, 128
    kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tq // 8), dtype=torch.int64, device=dev).to(torch.int32)
    ks = (torch.rand(B, H, D, Tq // 32, device=dev) * 0.02).half()
    km = (torch.randn(B, H, D, Tq // 32, device=dev) * 0.1).half()
    vc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tq, D // 16), dtype=torch.int64, device=dev).to(torch.int32)
    vs = (torch.rand(B, H, Tq, D // 32, device=dev) * 0.5).half()
    vm = (torch.randn(B, H, Tq, D // 32, device=dev)).half()
    k_tail = torch.randn(B, H, L, D, device=dev).half()
    v_tail = torch.randn(B, H, L, D, device=dev).half()
    q = torch.randn(B, H, 1, D, device=dev).half()
    out, p = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), k_tail, v_tail, 32, 4, 32, 2)
    assert p.shape == (B, H, 1, Tq + L) and float(p.min()) >= 0.0
    assert float((p.float().sum(-1) - 1.0).abs().max()) < 3e-3   # 8192 fp16 roundings of up to 2^-11 relative each
    att = KVmixAttention(4, 2, residual_length=L)
    out_t, p_t = att._decode_with_torch_glue(q, kc, ks, km, k_tail, vc, vs, vm, v_tail, 32, 0, 0, 1, None)
    torch.testing.assert_close(p, p_t, rtol=5e-3, atol=2e-6)
    torch.testing.assert_close(out, out_t, rtol=5e-3, atol=5e-3)
    c = 0.25
    out_c, p_c = ops.decode_attention(q, (kc, ks, km), (vc, vs, (vm.float() + c).half()), k_tail, v_tail, 32, 4, 32, 2)
    assert torch.equal(p_c, p)
    shift = c * p[..., :Tq].float().sum(-1)   # [B,H,1]
    # zero points were rounded to fp16 after the shift: allow their ulp (2^-10 of |zero| <= 4) on top of the output's
    torch.testing.assert_close(out_c.float() - out.float(), shift.unsqueeze(-1).expand(B, H, 1, D), rtol=0, atol=1.2e-2)


def test_library_step_with_a_row_longer_than_the_register_path(dev):
    """More than 16384 positions: the softmax walks the row in three passes instead of holding it in
    registers.  Against the composition from the GEMVs and torch, GQA, with a padding mask."""
    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    torch.manual_seed(12)
    B, H, Hkv, D, Tq, L = 2, 4, 2, 128, 20000 - 32, 37
    kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, D, Tq // 16), dtype=torch.int64, device=dev).to(torch.int32)
    ks = (torch.rand(B, Hkv, D, Tq // 32, device=dev) * 0.05).half()
    km = (torch.randn(B, Hkv, D, Tq // 32, device=dev) * 0.1).half()
    vc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, Tq, D // 8), dtype=torch.int64, device=dev).to(torch.int32)
    vs = (torch.rand(B, Hkv, Tq, D // 32, device=dev) * 0.1).half()
    vm = torch.randn(B, Hkv, Tq, D // 32, device=dev).half()
    k_tail = torch.randn(B, Hkv, L, D, device=dev).half()
    v_tail = torch.randn(B, Hkv, L, D, device=dev).half()
    q = torch.randn(B, H, 1, D, device=dev).half()
    mask = torch.zeros(B, 1, 1, Tq + L, device=dev)
    mask[0, :, :, :5000] = torch.finfo(torch.float32).min
    att = KVmixAttention(2, 4, residual_length=64)
    for m in (None, mask):
        out, p = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), k_tail, v_tail, 32, 2, 32, 4, attention_mask=m)
        out_t, p_t = att._decode_with_torch_glue(q, kc, ks, km, k_tail, vc, vs, vm, v_tail, 32, 0, 0, H // Hkv, m)
        torch.testing.assert_close(p, p_t, rtol=5e-3, atol=2e-6)
        torch.testing.assert_close(out, out_t, rtol=5e-3, atol=5e-3)
    assert float(p[0, :, :, :5000].abs().max()) == 0.0
