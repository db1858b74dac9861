"""The single-pass attention step (ops.decode_attention(single_pass=True)) against the four-launch
step, which the other tests tie to the oracle.  The two differ by design in the roundings after
the softmax (single pass: fp32 probabilities, one rounding of the output; four launches: the
reference's fp16 probabilities and fp16 halves), i.e. by about 2^-10 of the largest value
magnitude; the tolerance below is 2e-3 of that magnitude plus 2e-3 relative."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n, v_dense3=True, mask_rng=None, window_pad=0, D=128):
    from kvmix_amd import ops

    kg = 11 if k_bits == 3 else 32
    lk, lv = n - tk, n - tv

    def rnd_i32(*shape):
        return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, device=dev, generator=gen).to(torch.int32)

    def rnd_f16(*shape, scale=1.0):
        return (torch.randn(*shape, device=dev, generator=gen) * scale).half()

    kw = tk // 11 if k_bits == 3 else tk * k_bits // 32
    kq = (rnd_i32(B, nkv, D, kw), rnd_f16(B, nkv, D, tk // kg, scale=0.05).abs(), rnd_f16(B, nkv, D, tk // kg, scale=0.3)) if tk else None
    vq = (rnd_i32(B, nkv, tv, D * v_bits // 32), rnd_f16(B, nkv, tv, D // 32, scale=0.2).abs(), rnd_f16(B, nkv, tv, D // 32)) if tv else None
    R = max(lk, lv) + window_pad
    k_tail = rnd_f16(B, nkv, lk + window_pad if window_pad else lk, D)
    v_tail = rnd_f16(B, nkv, lv + window_pad if window_pad else lv, D)
    q = rnd_f16(B, nkv * rep, 1, D)
    mask = None
    if mask_rng is not None:
        width = max(tk + k_tail.shape[2], tv + v_tail.shape[2])
        mask = torch.zeros(B, 1, 1, width, device=dev)
        mask[B - 1, :, :, :int(mask_rng.integers(1, max(n // 2, 2)))] = torch.finfo(torch.float32).min
    fmt = dict(k_fmt=ops.FMT_REF, v_fmt=ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF)
    return q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv


def check(out_s, out_f, v_mag):
    a, b = out_s.float(), out_f.float()
    tol = 2e-3 * v_mag + 2e-3 * b.abs()
    bad = (a - b).abs() > tol
    assert not bool(bad.any()), (float((a - b).abs().max()), v_mag)


def v_magnitude(vq, v_tail, v_bits):
    m = float(v_tail.abs().max()) if v_tail.numel() else 0.0
    if vq is not None:
        m = max(m, float((vq[1].float() * (2 ** v_bits - 1) + vq[2].float().abs()).max()))
    return m


@pytest.mark.parametrize("seed", [5, 6, 7])
def test_single_pass_against_four_launch_step(dev, seed):
    from kvmix_amd import ops

    rng = np.random.default_rng(seed)
    gen = torch.Generator(device=dev).manual_seed(seed)
    for case in range(14):
        B = int(rng.choice([1, 2, 3]))
        nkv = int(rng.choice([1, 2, 4]))
        rep = int(rng.choice([1, 2, 4, 8]))
        k_bits = int(rng.choice([1, 2, 3, 4]))
        v_bits = int(rng.choice([1, 2, 3, 4]))
        kg = 11 if k_bits == 3 else 32
        n = int(rng.integers(40, 2600))
        tk = (int(rng.integers(0, n + 1)) // kg) * kg
        tv = (int(rng.integers(0, n + 1)) // 32) * 32
        if case == 0:
            tk = 0
        if case == 1:
            tv = 0
        print("case", seed, case, dict(B=B, nkv=nkv, rep=rep, k_bits=k_bits, v_bits=v_bits, n=n, tk=tk, tv=tv), flush=True)
        q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n,
                                                                      mask_rng=rng if rng.random() < 0.5 else None)
        assert ops.single_pass_supported(128, rep, k_bits, fmt["k_fmt"], kg, v_bits, fmt["v_fmt"], 32)
        out_f, probs = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, **fmt)
        out_s, none = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask,
                                           single_pass=True, **fmt)
        assert none is None and out_s.shape == out_f.shape
        check(out_s, out_f, v_magnitude(vq, v_tail, v_bits))


def test_single_pass_with_device_side_lengths(dev):
    """Tails held in longer windows whose live lengths are read on the device: same result as with
    exact-size tails, whatever the slots past the live length hold."""
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(9)
    for (k_bits, v_bits, tk, tv, n) in [(4, 2, 1024, 960, 1100), (3, 4, 1408, 1472, 1500), (2, 3, 480, 512, 520), (1, 1, 0, 0, 70)]:
        q, kq, vq, k_tail, v_tail, kg, _, fmt, lk, lv = make_case(dev, gen, 2, 2, 2, k_bits, v_bits, tk, tv, n)
        want, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, single_pass=True, **fmt)
        R = max(lk, lv) + 37
        kwin = torch.full((2, 2, R, 128), 77.0, dtype=torch.float16, device=dev)
        vwin = torch.full((2, 2, R, 128), float("nan"), dtype=torch.float16, device=dev)
        kwin[:, :, :lk], vwin[:, :, :lv] = k_tail, v_tail
        klen = torch.tensor([lk], dtype=torch.int64, device=dev)
        vlen = torch.tensor([lv], dtype=torch.int64, device=dev)
        got, _ = ops.decode_attention(q, kq, vq, kwin, vwin, kg, k_bits, 32, v_bits, k_tail_len=klen, v_tail_len=vlen,
                                      single_pass=True, **fmt)
        assert torch.equal(got, want)


def test_single_pass_against_exact_attention(dev):
    """Against fp64 attention over the dequantized cache, with the one rounding the single-pass step
    keeps from the reference (logits to fp16 before scaling): a few 1e-3 of the value magnitude."""
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(10)
    B, nkv, rep, n, tk, tv = 2, 2, 4, 1700, 1536, 1600
    q, kq, vq, k_tail, v_tail, kg, _, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, 4, 4, tk, tv, n)
    out, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, 4, 32, 4, single_pass=True, **fmt)

    def unpack4(code):  # [..., W] int32 -> [..., W*8] codes, low nibble first
        c = code.to(torch.int64) & 0xffffffff
        return torch.stack([(c >> (4 * i)) & 15 for i in range(8)], -1).flatten(-2).double()

    K = unpack4(kq[0]) * kq[1].double().repeat_interleave(32, -1) + kq[2].double().repeat_interleave(32, -1)  # [B,nkv,D,tk]
    V = unpack4(vq[0]) * vq[1].double().repeat_interleave(32, -1) + vq[2].double().repeat_interleave(32, -1)  # [B,nkv,tv,D]
    K = torch.cat([K.transpose(2, 3), k_tail.double()], 2).repeat_interleave(rep, 1)
    V = torch.cat([V, v_tail.double()], 2).repeat_interleave(rep, 1)
    logits = (q.double() @ K.transpose(2, 3)).half().double() / 128 ** 0.5
    want = torch.softmax(logits, -1) @ V
    err = float((out.double() - want).abs().max())
    assert err <= 4e-3 * float(V.abs().max()), err


def test_single_pass_refuses_what_it_does_not_take(dev):
    from kvmix_amd import ops

    assert not ops.single_pass_supported(64, 1, 4, ops.FMT_REF, 32, 4, ops.FMT_REF, 32)
    assert not ops.single_pass_supported(128, 3, 4, ops.FMT_REF, 32, 4, ops.FMT_REF, 32)
    assert ops.single_pass_supported(128, 1, 3, ops.FMT_DENSE3, 32, 4, ops.FMT_REF, 32)
    assert not ops.single_pass_supported(128, 1, 3, ops.FMT_REF, 32, 4, ops.FMT_REF, 32)   # reference 3-bit words come in groups of 11
    assert not ops.single_pass_supported(128, 1, 4, ops.FMT_REF, 64, 4, ops.FMT_REF, 32)
    q = torch.zeros(1, 2, 1, 64, dtype=torch.float16, device=dev)
    tail = torch.zeros(1, 2, 5, 64, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError, match="single-pass"):
        ops.decode_attention(q, None, None, tail, tail, 32, 4, 32, 4, single_pass=True)


def test_single_pass_with_dense_three_bit_keys(dev):
    """Dense 3-bit keys (32 codes in three words, group 32): the single pass against the four-launch step."""
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(12)
    for (B, nkv, rep, tk, tv, n, v_bits) in [(2, 2, 2, 1504, 1472, 1600, 3), (1, 4, 1, 512, 0, 530, 4), (3, 1, 4, 96, 128, 140, 2)]:
        D = 128
        i32 = lambda *shape: torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, device=dev, generator=gen).to(torch.int32)
        f16 = lambda *shape, scale=1.0: (torch.randn(*shape, device=dev, generator=gen) * scale).half()
        kq = (i32(B, nkv, D, tk * 3 // 32), f16(B, nkv, D, tk // 32, scale=0.05).abs(), f16(B, nkv, D, tk // 32, scale=0.3))
        vq = (i32(B, nkv, tv, D * v_bits // 32), f16(B, nkv, tv, D // 32, scale=0.2).abs(), f16(B, nkv, tv, D // 32)) if tv else None
        k_tail, v_tail, q = f16(B, nkv, n - tk, D), f16(B, nkv, n - tv, D), f16(B, nkv * rep, 1, D)
        fmt = dict(k_fmt=ops.FMT_DENSE3, v_fmt=ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF)
        out_f, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, 32, 3, 32, v_bits, **fmt)
        out_s, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, 32, 3, 32, v_bits, single_pass=True, **fmt)
        check(out_s, out_f, v_magnitude(vq, v_tail, v_bits))
