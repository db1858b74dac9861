"""The single-pass attention step (ops.decode_attention(single_pass=True)): every key and value format
and head grouping against fp64 attention over the cache dequantized with torch integer ops, and
random layouts against the four-launch step, which the other tests tie to the oracle.  The two differ by design in the roundings after
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


KEY_KINDS = {"k1": (1, False), "k2": (2, False), "k4": (4, False), "kref3": (3, False), "kdense3": (3, True)}
VALUE_KINDS = {"v1": (1, False), "v2": (2, False), "v4": (4, False), "vdense3": (3, True)}


@pytest.mark.parametrize("k_kind", list(KEY_KINDS))
@pytest.mark.parametrize("v_kind", list(VALUE_KINDS))
def test_single_pass_against_exact_attention(dev, k_kind, v_kind):
    """Every key and value format, with 1, 4 and 8 query heads per kv head and a padding mask, against
    fp64 attention over the cache dequantized with torch integer ops (no kernel of the library), with the
    one rounding the single-pass step keeps from the reference (logits to fp16 before scaling): a few
    1e-3 of the value magnitude."""
    from helpers import unpack_codes_torch
    from kvmix_amd import ops

    (k_bits, k_dense3), (v_bits, v_dense3) = KEY_KINDS[k_kind], VALUE_KINDS[v_kind]
    gen = torch.Generator(device=dev).manual_seed(10 + 7 * k_bits + v_bits + k_dense3)
    D, B, nkv = 128, 2, 2
    kg = 11 if (k_bits == 3 and not k_dense3) else 32
    i32 = lambda *shape: torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, device=dev, generator=gen).to(torch.int32)
    f16 = lambda *shape, scale=1.0: (torch.randn(*shape, device=dev, generator=gen) * scale).half()
    for rep, n, tk, tv in ((1, 1700, (1536 // kg) * kg, 1600), (4, 900, (700 // kg) * kg, 832), (8, 2300, (2200 // kg) * kg, 2176)):
        kw = tk * 3 // 32 if k_dense3 else (tk // 11 if k_bits == 3 else tk * k_bits // 32)
        vw = D * 3 // 32 if v_dense3 else D * v_bits // 32
        kq = (i32(B, nkv, D, kw), f16(B, nkv, D, tk // kg, scale=0.05).abs(), f16(B, nkv, D, tk // kg, scale=0.3))
        vq = (i32(B, nkv, tv, vw), f16(B, nkv, tv, D // 32, scale=0.2).abs(), f16(B, nkv, tv, D // 32))
        k_tail, v_tail, q = f16(B, nkv, n - tk, D), f16(B, nkv, n - tv, D), f16(B, nkv * rep, 1, D)
        mask = torch.zeros(B, 1, 1, n, device=dev)
        mask[B - 1, :, :, :n // 3] = torch.finfo(torch.float32).min  # the last sequence is left-padded
        fmt = dict(k_fmt=ops.FMT_DENSE3 if k_dense3 else ops.FMT_REF, v_fmt=ops.FMT_DENSE3 if v_dense3 else ops.FMT_REF)
        assert ops.single_pass_supported(D, rep, k_bits, fmt["k_fmt"], kg, v_bits, fmt["v_fmt"], 32)
        out, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask,
                                      single_pass=True, **fmt)
        K = unpack_codes_torch(kq[0], k_bits, k_dense3).double() * kq[1].double().repeat_interleave(kg, -1) \
            + kq[2].double().repeat_interleave(kg, -1)
        V = unpack_codes_torch(vq[0], v_bits, v_dense3).double() * vq[1].double().repeat_interleave(32, -1) \
            + vq[2].double().repeat_interleave(32, -1)                                                # [B,nkv,tv,D]
        K = torch.cat([K.transpose(2, 3), k_tail.double()], 2).repeat_interleave(rep, 1)
        V = torch.cat([V, v_tail.double()], 2).repeat_interleave(rep, 1)
        logits = (q.double() @ K.transpose(2, 3)).half().double() / D ** 0.5 + mask.double()
        want = torch.softmax(logits, -1) @ V
        err = float((out.double() - want).abs().max())
        assert err <= 4e-3 * float(V.abs().max()), (k_kind, v_kind, rep, err)


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


def test_more_rows_than_one_grid_dimension_holds(dev):
    """Batch x kv heads beyond 65535: the single pass launches a one-dimensional grid, the four-launch step
    sends its GEMVs out in parts; both must still agree."""
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(11)
    B, nkv, rep, k_bits, v_bits, n, tk, tv = 32770, 2, 1, 4, 2, 40, 32, 32
    q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n)
    out_f, probs = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, **fmt)
    out_s, none = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, single_pass=True, **fmt)
    check(out_s, out_f, v_magnitude(vq, v_tail, v_bits))
    # the last rows against plain attention over the dequantized cache of those rows
    from helpers import dequantize_torch
    sl = slice(B - 2, B)
    kd = dequantize_torch(kq[0][sl], kq[1][sl], kq[2][sl], k_bits, 32).double()          # [2, nkv, D, tk]
    vd = dequantize_torch(vq[0][sl], vq[1][sl], vq[2][sl], v_bits, 32).double()          # [2, nkv, tv, D]
    keys = torch.cat([kd.transpose(2, 3), k_tail[sl].double()], 2)
    vals = torch.cat([vd, v_tail[sl].double()], 2)
    logits = (q[sl].double() @ keys.transpose(2, 3)) / np.sqrt(128.0)
    want = torch.softmax(logits, -1) @ vals
    check(out_s[sl], want, v_magnitude(vq, v_tail, v_bits))


@pytest.mark.parametrize("k_bits", [1, 2, 4])
@pytest.mark.parametrize("v_bits", [1, 2, 3, 4])
def test_large_steps_on_the_matrix_cores(dev, k_bits, v_bits):
    """Steps with at least 1024 (query head, 1024-position tile) pairs whose keys and values are quantized to
    the same length run their quantized positions through the matrix-core slab kernel: against the four-launch
    step, with a padding mask, query heads sharing kv heads, a last tile that is moved back (8064 = 7.875 tiles)
    and, for one pair, fp64 attention over the dequantized cache of two rows."""
    from kvmix_amd import ops
    from helpers import dequantize_torch

    gen = torch.Generator(device=dev).manual_seed(100 + 10 * k_bits + v_bits)
    rng = np.random.default_rng(k_bits * 7 + v_bits)
    B, nkv, rep, tk, n = 2, 32, 2, 8064, 8064 + 97
    q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tk, n, mask_rng=rng)
    out_f, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, **fmt)
    out_s, none = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask,
                                       single_pass=True, **fmt)
    assert none is None
    vm = v_magnitude(vq, v_tail, v_bits)
    check(out_s, out_f, vm)
    if (k_bits, v_bits) in ((4, 2), (2, 3), (1, 4)):
        sl = slice(B - 1, B)
        kd = dequantize_torch(kq[0][sl, :2], kq[1][sl, :2], kq[2][sl, :2], k_bits, 32).double()      # [1, 2, D, tk]
        vd = dequantize_torch(vq[0][sl, :2], vq[1][sl, :2], vq[2][sl, :2], v_bits, 32, dense3=v_bits == 3).double()
        keys = torch.cat([kd.transpose(2, 3), k_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
        vals = torch.cat([vd, v_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
        qq = q[sl, :2 * rep].double()
        logits = (qq @ keys.transpose(2, 3)).half().double() / np.sqrt(128.0) + mask[sl].double()
        want = torch.softmax(logits, -1) @ vals
        check(out_s[sl, :2 * rep], want, vm)


def test_matrix_core_slabs_with_short_rows_and_device_side_lengths(dev):
    """Two tiles of which the second is moved back almost wholly (1056 positions), tails in longer windows
    with their lengths on the device."""
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(77)
    B, nkv, rep, k_bits, v_bits, tk = 16, 32, 1, 4, 4, 1056
    lk = 41
    q, kq, vq, k_tail, v_tail, kg, _, fmt, _, _ = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tk, tk + lk)
    want, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, **fmt)
    got, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, single_pass=True, **fmt)
    check(got, want, v_magnitude(vq, v_tail, v_bits))
    R = lk + 23
    kwin = torch.full((B, nkv, R, 128), 77.0, dtype=torch.float16, device=dev)
    vwin = torch.full((B, nkv, R, 128), float("nan"), dtype=torch.float16, device=dev)
    kwin[:, :, :lk], vwin[:, :, :lk] = k_tail, v_tail
    klen = torch.tensor([lk], dtype=torch.int64, device=dev)
    got2, _ = ops.decode_attention(q, kq, vq, kwin, vwin, kg, k_bits, 32, v_bits, k_tail_len=klen, v_tail_len=klen.clone(),
                                   single_pass=True, **fmt)
    assert torch.equal(got2, got)


@pytest.mark.parametrize("k_bits,v_bits,tk,tv", [(4, 2, 8064, 7968), (2, 4, 4000 // 32 * 32, 4096), (1, 3, 4096, 4096 + 32),
                                                 (4, 4, 8064, 8064)])
def test_matrix_core_steps_with_keys_and_values_quantized_to_different_lengths(dev, k_bits, v_bits, tk, tv):
    """The matrix-core tiles cover the positions quantized on both sides; what lies between the two quantized lengths
    (codes on one side, the fp16 tail on the other) and the tails run as vector-ALU slabs in the same launch.  Against
    the four-launch step and, for two rows, fp64 attention over the dequantized cache; the library is asked first
    whether these sizes take the matrix-core form, with two launches (tiles + slabs, merge)."""
    from kvmix_amd import ops, _lib
    from helpers import dequantize_torch

    gen = torch.Generator(device=dev).manual_seed(300 + tk % 97 + tv % 89)
    rng = np.random.default_rng(tk + tv)
    B, nkv, rep = 2, 32, 2
    n = max(tk, tv) + 61
    plan = _lib.attn_plan(_lib.attn_step_descriptor(B, nkv * rep, nkv, 128, k_bits, 0, 32, tk, v_bits, 1 if v_bits == 3 else 0, 32, tv,
                                                   n - tk, n - tv))
    assert plan["matrix"] and plan["launches"] == 2 and plan["slab_begin"] == min(tk, tv), plan
    q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n, mask_rng=rng)
    out_f, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, **fmt)
    out_s, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, single_pass=True, **fmt)
    vm = v_magnitude(vq, v_tail, v_bits)
    check(out_s, out_f, vm)
    sl = slice(B - 1, B)
    kd = dequantize_torch(kq[0][sl, :2], kq[1][sl, :2], kq[2][sl, :2], k_bits, 32).double()
    vd = dequantize_torch(vq[0][sl, :2], vq[1][sl, :2], vq[2][sl, :2], v_bits, 32, dense3=v_bits == 3).double()
    keys = torch.cat([kd.transpose(2, 3), k_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    vals = torch.cat([vd, v_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    logits = (q[sl, :2 * rep].double() @ keys.transpose(2, 3)).half().double() / np.sqrt(128.0) + mask[sl].double()
    check(out_s[sl, :2 * rep], torch.softmax(logits, -1) @ vals, vm)


@pytest.mark.parametrize("v_bits,tk,tv", [(2, 8063, 8064), (3, 733 * 11 - 11 * 40, 8064), (4, 1408 + 352, 1408 + 352 + 32), (1, 3 * 1408, 3 * 1408)])
def test_matrix_core_steps_with_the_reference_three_bit_keys(dev, v_bits, tk, tv):
    """Keys in the reference's 3-bit words, the format its profiler assigns to most layers: tiles of 1408 positions
    (128 words a row) over the whole multiples of 352 positions that keys and values both have quantized, a last
    tile that is moved back, vector-ALU slabs over the rest.  Against the four-launch step and, for two rows, fp64
    attention over the dequantized cache."""
    from kvmix_amd import ops, _lib
    from helpers import dequantize_torch

    gen = torch.Generator(device=dev).manual_seed(500 + tk % 97 + v_bits)
    rng = np.random.default_rng(tk + v_bits)
    B, nkv, rep = 4, 32, 2
    n = max(tk, tv) + 77
    plan = _lib.attn_plan(_lib.attn_step_descriptor(B, nkv * rep, nkv, 128, 3, 0, 11, tk, v_bits, 1 if v_bits == 3 else 0, 32, tv,
                                                   n - tk, n - tv))
    assert plan["matrix"] and plan["launches"] == 2 and plan["slab_begin"] == min(tk, tv) // 352 * 352, plan
    q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, 3, v_bits, tk, tv, n, mask_rng=rng)
    out_f, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, 3, 32, v_bits, attention_mask=mask, **fmt)
    out_s, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, 3, 32, v_bits, attention_mask=mask, single_pass=True, **fmt)
    vm = v_magnitude(vq, v_tail, v_bits)
    check(out_s, out_f, vm)
    sl = slice(B - 1, B)
    kd = dequantize_torch(kq[0][sl, :2], kq[1][sl, :2], kq[2][sl, :2], 3, 11).double()
    vd = dequantize_torch(vq[0][sl, :2], vq[1][sl, :2], vq[2][sl, :2], v_bits, 32, dense3=v_bits == 3).double()
    keys = torch.cat([kd.transpose(2, 3), k_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    vals = torch.cat([vd, v_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    logits = (q[sl, :2 * rep].double() @ keys.transpose(2, 3)).half().double() / np.sqrt(128.0) + mask[sl].double()
    check(out_s[sl, :2 * rep], torch.softmax(logits, -1) @ vals, vm)


@pytest.mark.parametrize("k_bits", [1, 2, 3, 4])
@pytest.mark.parametrize("v_bits,tk,dv", [(1, 2176, 0), (2, 1152, 32), (3, 2560, -64), (4, 3072, 0)])
def test_steps_with_few_tiles_share_a_tile_among_four_waves(dev, k_bits, v_bits, tk, dv):
    """Steps with few (query head, tile) pairs -- the sizes of a small-batch decode loop -- run a block per tile: the
    four waves take a quarter of the channel rows each for the logits and then a quarter of the tile's positions
    each as a slab of its own.  Query heads sharing kv heads, a padding mask, last tiles moved back by up to 7/8 of
    their length, values quantized further or less far than the keys; against the four-launch step and, for two rows,
    fp64 attention over the dequantized cache."""
    from kvmix_amd import ops, _lib
    from helpers import dequantize_torch

    kg = 11 if k_bits == 3 else 32
    tk = tk // 352 * 352 + 33 * 11 if k_bits == 3 else tk  # (the reference's words: whole words, not whole tiles)
    tv = tk // 32 * 32 + dv
    gen = torch.Generator(device=dev).manual_seed(700 + 10 * k_bits + v_bits)
    rng = np.random.default_rng(31 * k_bits + v_bits)
    B, nkv, rep = 4, 8, 4
    n = max(tk, tv) + 93
    plan = _lib.attn_plan(_lib.attn_step_descriptor(B, nkv * rep, nkv, 128, k_bits, 0, kg, tk, v_bits, 1 if v_bits == 3 else 0, 32, tv,
                                                   n - tk, n - tv))
    assert plan["matrix"] and plan["matrix_tile_waves"] == 4 and plan["launches"] == 2 and plan["recommended"], plan
    q, kq, vq, k_tail, v_tail, kg, mask, fmt, lk, lv = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n, mask_rng=rng)
    out_f, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, **fmt)
    out_s, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, single_pass=True, **fmt)
    vm = v_magnitude(vq, v_tail, v_bits)
    check(out_s, out_f, vm)
    sl = slice(B - 1, B)
    kd = dequantize_torch(kq[0][sl, :2], kq[1][sl, :2], kq[2][sl, :2], k_bits, kg).double()
    vd = dequantize_torch(vq[0][sl, :2], vq[1][sl, :2], vq[2][sl, :2], v_bits, 32, dense3=v_bits == 3).double()
    keys = torch.cat([kd.transpose(2, 3), k_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    vals = torch.cat([vd, v_tail[sl, :2].double()], 2).repeat_interleave(rep, 1)
    logits = (q[sl, :2 * rep].double() @ keys.transpose(2, 3)).half().double() / np.sqrt(128.0) + mask[sl].double()
    check(out_s[sl, :2 * rep], torch.softmax(logits, -1) @ vals, vm)
    # a second call on other data of the same sizes, then the first again: nothing is carried between calls
    q2 = torch.randn(q.shape, device=dev, generator=gen).half()
    ops.decode_attention(q2, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, single_pass=True, **fmt)
    again, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask, single_pass=True, **fmt)
    assert torch.equal(again, out_s)


@pytest.mark.parametrize("k_bits", [4, 3])
def test_shared_tiles_with_device_side_lengths_and_eight_heads_per_kv_head(dev, k_bits):
    """The four-waves-per-tile form with eight query heads per kv head, tails in longer windows whose lengths live on
    the device, and a second tile that is moved back almost wholly (4-bit keys: 1056 positions; the reference's
    3-bit keys: 1408 + 352)."""
    from kvmix_amd import ops, _lib

    gen = torch.Generator(device=dev).manual_seed(900 + k_bits)
    B, nkv, rep, v_bits = 2, 8, 8, 2
    kg = 11 if k_bits == 3 else 32
    tk = 1408 + 352 + 11 * 5 if k_bits == 3 else 1056
    tv = tk // 32 * 32
    lk = 41 + (tk - tv)
    n = tv + lk
    plan = _lib.attn_plan(_lib.attn_step_descriptor(B, nkv * rep, nkv, 128, k_bits, 0, kg, tk, v_bits, 0, 32, tv, n - tk, n - tv))
    assert plan["matrix"] and plan["matrix_tile_waves"] == 4, plan
    q, kq, vq, k_tail, v_tail, kg, _, fmt, lk_, lv_ = make_case(dev, gen, B, nkv, rep, k_bits, v_bits, tk, tv, n)
    want, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, **fmt)
    got, _ = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, single_pass=True, **fmt)
    check(got, want, v_magnitude(vq, v_tail, v_bits))
    R = max(lk_, lv_) + 23
    kwin = torch.full((B, nkv, R, 128), 77.0, dtype=torch.float16, device=dev)
    vwin = torch.full((B, nkv, R, 128), float("nan"), dtype=torch.float16, device=dev)
    kwin[:, :, :lk_], vwin[:, :, :lv_] = k_tail, v_tail
    klen = torch.tensor([lk_], dtype=torch.int64, device=dev)
    vlen = torch.tensor([lv_], dtype=torch.int64, device=dev)
    got2, _ = ops.decode_attention(q, kq, vq, kwin, vwin, kg, k_bits, 32, v_bits, k_tail_len=klen, v_tail_len=vlen,
                                   single_pass=True, **fmt)
    assert torch.equal(got2, got)
