"""The fused key+value flush against the two separate operators and the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from helpers import kv_like, same_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k_bits,v_bits", [(4, 4), (2, 4), (3, 2), (4, 3), (1, 1), (3, 3)])
@pytest.mark.parametrize("shape", [(2, 3, 64, 128, 32), (1, 2, 128, 128, 96), (2, 1, 32, 64, 1)])
def test_fused_flush_matches_separate(k_bits, v_bits, shape):
    from kvmix_amd import ops
    from oracle import kvmix_oracle as O

    B, H, n, D, nv = shape
    rng = np.random.default_rng(k_bits * 100 + v_bits * 10 + n)
    k_group = 11 if k_bits == 3 else 32
    nk = (n // k_group) * k_group if k_bits != 3 else 66 if n >= 66 else 33
    k_np = kv_like(rng, (B, H, nk, D)).astype(np.float16)
    v_np = kv_like(rng, (B, H, nv, D)).astype(np.float16)
    k = torch.from_numpy(k_np).cuda()
    v = torch.from_numpy(v_np).cuda()
    v_fmt = ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF
    kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(k, k_group, k_bits, v, 32, v_bits, ops.FMT_REF, v_fmt)
    # separate operators
    kc2, ks2, km2 = ops.quantize_pack_last_dim_cuda(k.transpose(2, 3).contiguous(), k_group, k_bits)
    if v_bits == 3:
        vc2, vs2, vm2 = ops.quantize_pack_dense3(v, 32)
    else:
        vc2, vs2, vm2 = ops.quantize_pack_last_dim_cuda(v, 32, v_bits)
    torch.cuda.synchronize()
    for got, want in ((kc, kc2), (ks, ks2), (km, km2), (vc, vc2), (vs, vs2), (vm, vm2)):
        assert got.shape == want.shape
        assert same_bits(got.cpu().numpy(), want.cpu().numpy())
    # and the oracle for the key half (the transposed call is what the reference runs)
    oc, osc, omn = O.quantize_pack_last_dim(np.ascontiguousarray(k_np.transpose(0, 1, 3, 2)), k_group, k_bits)
    assert same_bits(kc.cpu().numpy(), oc) and same_bits(ks.cpu().numpy(), osc) and same_bits(km.cpu().numpy(), omn)


def test_fused_flush_rejects_bad_halves_before_launching():
    from kvmix_amd import ops

    k = torch.zeros(1, 1, 32, 64, dtype=torch.float16, device="cuda")
    v = torch.zeros(1, 1, 4, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.quantize_kv_flush(k, 32, 4, v, 48, 4)  # 64 not divisible by 48
    with pytest.raises(RuntimeError):
        ops.quantize_kv_flush(k, 11, 3, v, 32, 4)  # 32 tokens not divisible by 11


def test_fused_flush_empty_half():
    from kvmix_amd import ops

    k = torch.randn(1, 2, 0, 64, dtype=torch.float16, device="cuda")
    v = torch.randn(1, 2, 8, 64, dtype=torch.float16, device="cuda")
    kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(k, 32, 4, v, 32, 4)
    vc2, vs2, vm2 = ops.quantize_pack_last_dim_cuda(v, 32, 4)
    assert kc.shape == (1, 2, 64, 0)
    assert torch.equal(vc, vc2) and torch.equal(vs, vs2) and torch.equal(vm, vm2)


def test_flush_at_config1_size_against_the_oracle():
    """One flush of BASELINE configs[1] at full size (batch 8, 32 heads, head_dim 128, 128-token window):
    121 key tokens into the reference's 3-bit words with 128 value tokens into the dense 3-bit stream,
    and 128 / 128 tokens at 4 and 2 bits, written in place at an offset of larger cache buffers;
    codes, scales and zeros bit for bit against the oracle, nothing else in the buffers touched."""
    from kvmix_amd import ops
    from oracle import kvmix_oracle as O

    B, H, D, cap = 8, 32, 128, 8192
    rng = np.random.default_rng(17)
    for k_bits, v_bits, nk in ((3, 3, 121), (4, 2, 128), (2, 4, 128)):
        k_group = 11 if k_bits == 3 else 32
        v_fmt = ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF
        k_np = kv_like(rng, (B, H, nk, D), outlier_axis=3)
        v_np = kv_like(rng, (B, H, 128, D), outlier_axis=3)
        kvpw = 11 if k_bits == 3 else 32 // k_bits
        vwords = D * 3 // 32 if v_bits == 3 else D * v_bits // 32
        k0 = 7936 if k_bits != 3 else 7942          # tokens already in the cache (whole groups)
        kc = torch.full((B, H, D, cap // kvpw), -1, dtype=torch.int32, device="cuda")
        ks = torch.full((B, H, D, cap // k_group), 7.0, dtype=torch.float16, device="cuda")
        km = torch.full_like(ks, 7.0)
        vc = torch.full((B, H, cap, vwords), -1, dtype=torch.int32, device="cuda")
        vs = torch.full((B, H, cap, D // 32), 7.0, dtype=torch.float16, device="cuda")
        vm = torch.full_like(vs, 7.0)
        w0, g0, v0 = k0 // kvpw, k0 // k_group, 7936
        k_out = (kc[..., w0:w0 + nk // kvpw], ks[..., g0:g0 + nk // k_group], km[..., g0:g0 + nk // k_group])
        v_out = (vc[:, :, v0:v0 + 128], vs[:, :, v0:v0 + 128], vm[:, :, v0:v0 + 128])
        ops.quantize_kv_flush_into(torch.from_numpy(k_np).cuda(), k_group, k_bits, k_out, torch.from_numpy(v_np).cuda(), 32,
                                   v_bits, v_out, ops.FMT_REF, v_fmt)
        torch.cuda.synchronize()
        oc, osc, omn = O.quantize_pack_last_dim(np.ascontiguousarray(k_np.transpose(0, 1, 3, 2)), k_group, k_bits)
        if v_bits == 3:
            ovc, ovs, ovm = O.quantize_pack_dense3(v_np, 32)
        else:
            ovc, ovs, ovm = O.quantize_pack_last_dim(v_np, 32, v_bits)
        for got, want in zip(k_out + v_out, (oc, osc, omn, ovc, ovs, ovm)):
            assert same_bits(got.cpu().numpy(), want), (k_bits, v_bits)
        # the rest of the buffers still holds the fill pattern
        for buf, lo, hi, axis, fill in ((kc, w0, w0 + nk // kvpw, 3, -1), (ks, g0, g0 + nk // k_group, 3, 7.0),
                                        (km, g0, g0 + nk // k_group, 3, 7.0), (vc, v0, v0 + 128, 2, -1),
                                        (vs, v0, v0 + 128, 2, 7.0), (vm, v0, v0 + 128, 2, 7.0)):
            before, after = buf.narrow(axis, 0, lo), buf.narrow(axis, hi, buf.shape[axis] - hi)
            assert bool((before == fill).all()) and bool((after == fill).all())


def test_flush_with_group_64_keys_when_both_tails_flush(dev=None):
    """A group size other than 32 (the reference allows any): the key half goes through the generic
    quantizer, the value half through the flush entry point with an empty key half -- which must not
    be refused for the key group it names."""
    from kvmix_amd import ops
    from oracle import kvmix_oracle as O

    rng = np.random.default_rng(23)
    B, H, D, n = 2, 3, 128, 128
    k_np = kv_like(rng, (B, H, n, D), outlier_axis=3)
    v_np = kv_like(rng, (B, H, n, D), outlier_axis=3)
    kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(torch.from_numpy(k_np).cuda(), 64, 4, torch.from_numpy(v_np).cuda(), 64, 2)
    oc, osc, omn = O.quantize_pack_last_dim(np.ascontiguousarray(k_np.transpose(0, 1, 3, 2)), 64, 4)
    ovc, ovs, ovm = O.quantize_pack_last_dim(v_np, 64, 2)
    for got, want in zip((kc, ks, km, vc, vs, vm), (oc, osc, omn, ovc, ovs, ovm)):
        assert same_bits(got.cpu().numpy(), want)


def test_batched_flush_matches_the_flushes_one_by_one():
    """kvmix_quant_pack_kv_flush_batch over 19 caches of mixed formats and sizes (three launches of eight, eight and
    three; two pairs that cannot share a launch -- an empty key half, a value group of 64 -- in between): every
    output bit for bit what quantize_kv_flush_into writes for the same pair."""
    from kvmix_amd import ops

    gen = torch.Generator(device="cuda").manual_seed(19)
    specs = []
    for i in range(19):
        k_bits = (4, 2, 3, 1, 3)[i % 5]
        v_bits = (2, 3, 4, 1)[i % 4]
        kg = 11 if k_bits == 3 else 32
        B, H, D = (2, 4, 128) if i % 3 else (1, 3, 64)
        nk = kg * (1 + i % 4) if i != 5 else 0          # (pair 5: nothing to flush on the key side)
        nv = 32 * (1 + i % 3)
        vg = 64 if i == 11 else 32                      # (pair 11: a value group the fused launch does not take)
        specs.append((k_bits, v_bits, kg, vg, B, H, D, nk, nv))

    def outputs(spec):
        k_bits, v_bits, kg, vg, B, H, D, nk, nv = spec
        kw = nk // 11 if k_bits == 3 else nk * k_bits // 32
        vw = D * 3 // 32 if v_bits == 3 else D * v_bits // 32
        z = lambda *s, dt=torch.float16: torch.zeros(*s, dtype=dt, device="cuda")
        return ((z(B, H, D, kw, dt=torch.int32), z(B, H, D, nk // kg), z(B, H, D, nk // kg)),
                (z(B, H, nv, vw, dt=torch.int32), z(B, H, nv, D // vg), z(B, H, nv, D // vg)))

    args_one, args_batch, outs_one, outs_batch = [], [], [], []
    for spec in specs:
        k_bits, v_bits, kg, vg, B, H, D, nk, nv = spec
        k = torch.randn(B, H, nk, D, device="cuda", generator=gen).half()
        v = torch.randn(B, H, nv, D, device="cuda", generator=gen).half()
        v_fmt = ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF
        for args, outs in ((args_one, outs_one), (args_batch, outs_batch)):
            ko, vo = outputs(spec)
            outs.append(ko + vo)
            args.append((k if nk else None, kg, k_bits, ko if nk else None, v, vg, v_bits, vo, ops.FMT_REF, v_fmt))
    for a in args_one:
        ops.quantize_kv_flush_into(*a)
    ops.quantize_kv_flush_batch(args_batch)
    torch.cuda.synchronize()
    for i, (one, batch) in enumerate(zip(outs_one, outs_batch)):
        for a, b in zip(one, batch):
            assert torch.equal(a, b), (i, specs[i])
        assert i == 5 or one[0].abs().sum() > 0          # (something was written)


@pytest.mark.parametrize("policy", ["window", "ratio"])
def test_flush_ahead_leaves_the_caches_as_flushing_inside_the_appends_does(policy):
    """cache.flush_ahead before every one-token append against caches that flush inside their appends: the
    reference's 9-tuple bit for bit after every one of 200 steps, for five caches of mixed formats under the fixed
    window and under the reference's ratio rule (where the five flush at different steps)."""
    from kvmix_amd import ops
    from kvmix_amd.cache import PackedKVCache, flush_ahead

    gen = torch.Generator(device="cuda").manual_seed(7)
    kinds = [(4, 4, ops.FMT_REF), (2, 3, ops.FMT_DENSE3), (3, 2, ops.FMT_REF), (1, 4, ops.FMT_REF), (3, 3, ops.FMT_DENSE3)]
    kw = dict(residual_length=64) if policy == "window" else {}

    def make():
        return [PackedKVCache(kb, vb, capacity=512, v_fmt=vf, **kw) for kb, vb, vf in kinds]

    plain, ahead = make(), make()
    B, H, D = 2, 4, 128
    prompt = [(torch.randn(B, H, 150, D, device="cuda", generator=gen).half(), torch.randn(B, H, 150, D, device="cuda", generator=gen).half())
              for _ in kinds]
    for group in (plain, ahead):
        for c, (k, v) in zip(group, prompt):
            c.append(k, v, prompt=True)
    flushed = 0
    for step in range(200):
        new = [(torch.randn(B, H, 1, D, device="cuda", generator=gen).half(), torch.randn(B, H, 1, D, device="cuda", generator=gen).half())
               for _ in kinds]
        flushed += flush_ahead(ahead)
        assert not any(c.flushes_on_next_append() for c in ahead)
        for group in (plain, ahead):
            for c, (k, v) in zip(group, new):
                c.append(k, v)
        for i, (a, b) in enumerate(zip(plain, ahead)):
            assert (a.k_tokens, a.v_tokens, a.kv_seq_len) == (b.k_tokens, b.v_tokens, b.kv_seq_len), (step, i)
            for x, y in zip(a.as_tuple()[:8], b.as_tuple()[:8]):
                assert (x is None) == (y is None) and (x is None or torch.equal(x, y)), (step, i)
    assert flushed >= 10


def test_batched_flush_of_large_value_halves_streams_and_matches():
    """Pairs with 16384 value groups or more take the streaming form of the value quantizer inside the batched launch
    (one thread per group): four pairs of the bench step's size, one per value bit width, against the flushes one by
    one."""
    from kvmix_amd import ops

    gen = torch.Generator(device="cuda").manual_seed(23)
    B, H, D, n = 8, 32, 128, 128
    one, batch, outs = [], [], []
    for v_bits, k_bits in ((1, 4), (2, 3), (3, 2), (4, 1)):
        kg = 11 if k_bits == 3 else 32
        nk = n // kg * kg
        k = torch.randn(B, H, nk, D, device="cuda", generator=gen).half()
        v = (torch.randn(B, H, n, D, device="cuda", generator=gen) * 3).half()
        v_fmt = ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF
        for args in (one, batch):
            kw = nk // 11 if k_bits == 3 else nk * k_bits // 32
            vw = D * 3 // 32 if v_bits == 3 else D * v_bits // 32
            ko = (torch.zeros(B, H, D, kw, dtype=torch.int32, device="cuda"), torch.zeros(B, H, D, nk // kg, dtype=torch.float16, device="cuda"),
                  torch.zeros(B, H, D, nk // kg, dtype=torch.float16, device="cuda"))
            vo = (torch.zeros(B, H, n, vw, dtype=torch.int32, device="cuda"), torch.zeros(B, H, n, D // 32, dtype=torch.float16, device="cuda"),
                  torch.zeros(B, H, n, D // 32, dtype=torch.float16, device="cuda"))
            args.append((k, kg, k_bits, ko, v, 32, v_bits, vo, ops.FMT_REF, v_fmt))
            outs.append(ko + vo)
    for a in one:
        ops.quantize_kv_flush_into(*a)
    ops.quantize_kv_flush_batch(batch)
    torch.cuda.synchronize()
    for i in range(0, len(outs), 2):
        for a, b in zip(outs[i], outs[i + 1]):
            assert torch.equal(a, b) and a.abs().sum() > 0, i // 2
