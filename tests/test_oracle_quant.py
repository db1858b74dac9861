"""Pins the CPU oracle's quantizer / packer with facts that do not come from the oracle:
closed-form grids, hand-packed words, brute-force inverses, rounding ties, and the
quantization error bound.  Reference: quant_cuda/csrc/quantization_cuda.cu:540-721."""
import numpy as np
import pytest

from helpers import kv_like, same_bits

BITS_G = [(1, 32), (2, 32), (4, 32), (3, 11), (4, 8), (2, 16), (1, 64), (4, 64)]


def u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_half_conversions_match_numpy(oracle):
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    assert same_bits(oracle.half_to_float(h), h.astype(np.float32))
    rng = np.random.default_rng(0)
    f = rng.standard_normal(200000).astype(np.float32) * rng.choice(
        np.array([1e-8, 1e-6, 1e-4, 1, 300, 7e4], np.float32), 200000)
    fin = h[np.isfinite(h)].astype(np.float32)
    lo = np.sort(fin)
    mid = ((lo[:-1].astype(np.float64) + lo[1:].astype(np.float64)) / 2).astype(np.float32)
    cases = np.concatenate([f, fin, mid, np.nextafter(mid, np.float32(np.inf)),
                            np.nextafter(mid, np.float32(-np.inf)),
                            np.array([65519.99, 65520, 65504, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -25,
                                      2.0 ** -25 * 1.000001, 2.0 ** -24, 0.0, -0.0], np.float32)])
    with np.errstate(over="ignore"):
        assert same_bits(oracle.float_to_half(cases), cases.astype(np.float16))


def test_hand_packed_words(oracle):
    # words written out by hand, value 0 in the low bits
    assert u32(oracle.pack_np(np.arange(8), 4))[0] == 0x76543210
    assert u32(oracle.pack_np(np.array([0, 1, 2, 3] * 4), 2))[0] == 0xE4E4E4E4
    assert u32(oracle.pack_np(np.array([0, 1] * 16), 1))[0] == 0xAAAAAAAA
    assert u32(oracle.pack_np(np.array([7] * 10 + [3]), 3))[0] == 0xFFFFFFFF
    assert u32(oracle.pack_np(np.array([1] + [0] * 10), 3))[0] == 0x1
    assert u32(oracle.pack_np(np.array([0] * 10 + [1]), 3))[0] == 0x40000000
    assert u32(oracle.pack_np(np.array([0, 0, 5] + [0] * 8), 3))[0] == 5 << 6


@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_pack_unpack_bruteforce(oracle, bits):
    vpw = oracle.values_per_word(bits)
    for pos in range(vpw):
        top = 4 if (bits == 3 and pos == 10) else (1 << bits)
        for c in range(top):
            q = np.zeros(vpw, np.int64)
            q[pos] = c
            w = oracle.pack_np(q, bits)
            shift = 30 if (bits == 3 and pos == 10) else pos * bits
            assert int(u32(w)[0]) == c << shift
            assert np.array_equal(oracle.unpack_np(w, bits), q)
            # the C unpacker agrees
            out = np.zeros(vpw, np.int32)
            oracle.lib().kvo_unpack_row(w.ctypes.data, 1, bits, out.ctypes.data)
            assert np.array_equal(out, q)
    rng = np.random.default_rng(bits)
    q = rng.integers(0, 1 << bits, size=(5, 7, vpw * 6))
    if bits == 3:
        q[..., 10::11] &= 3
    assert np.array_equal(oracle.unpack_np(oracle.pack_np(q, bits), bits), q)


@pytest.mark.parametrize("bits,g", BITS_G)
def test_exact_grid_gives_its_indices(oracle, bits, g):
    """x = mn + k*s on an exactly representable grid -> code k, scale s, zero mn."""
    rng = np.random.default_rng(100 + bits * 10 + g)
    qmax = (1 << bits) - 1
    S = g * 8 * (11 if bits == 3 else 1)
    S = S // g * g
    if bits != 3:
        S = np.lcm(S, 32 // bits)
    k = rng.integers(0, qmax + 1, size=(2, 3, 4, S))
    kg = k.reshape(2, 3, 4, S // g, g)
    kg[..., 0] = 0      # every group contains its min ...
    kg[..., 1] = qmax   # ... and its max
    k = kg.reshape(2, 3, 4, S)
    s, mn = np.float32(0.25), np.float32(-1.5)
    x = (mn + k * s).astype(np.float16)  # exact in fp16
    for fn in (oracle.quantize_pack_last_dim, oracle.quantize_pack_last_dim_np):
        code, scale, zero = fn(x, g, bits)
        want = k.copy()
        if bits == 3:
            want.reshape(2, 3, 4, S // 11, 11)[..., 10] = np.minimum(kg[..., 10], 3)
        assert np.array_equal(oracle.unpack_np(code, bits), want)
        assert scale.dtype == np.float16 and np.all(scale == np.float16(0.25))
        assert np.all(zero == np.float16(-1.5))


@pytest.mark.parametrize("bits,g", BITS_G)
def test_min_max_constant_groups(oracle, bits, g):
    rng = np.random.default_rng(7)
    qmax = (1 << bits) - 1
    S = int(np.lcm(g, 11 if bits == 3 else 32 // bits)) * 3
    x = kv_like(rng, (1, 2, 5, S))
    x[0, 1, 2, :g] = np.float16(3.25)  # a constant group: scale 0, 0/0 -> code 0
    code, scale, zero = oracle.quantize_pack_last_dim(x, g, bits)
    q = oracle.unpack_np(code, bits).reshape(1, 2, 5, S // g, g)
    xg = x.reshape(1, 2, 5, S // g, g).astype(np.float32)
    amin, amax = xg.argmin(-1), xg.argmax(-1)
    qmin = np.take_along_axis(q, amin[..., None], -1)[..., 0]
    qmaxv = np.take_along_axis(q, amax[..., None], -1)[..., 0]
    const = np.zeros(qmin.shape, bool)
    const[0, 1, 2, 0] = True
    assert np.all(qmin == 0)
    top = np.where((amax == 10) & (bits == 3), 3, qmax)
    assert np.all(qmaxv[~const] == top[~const])
    assert np.all(q[0, 1, 2, 0] == 0) and scale[0, 1, 2, 0] == 0 and zero[0, 1, 2, 0] == np.float16(3.25)
    assert np.all(zero.astype(np.float32) == xg.min(-1))


def test_round_half_away_from_zero_ties(oracle):
    """(x-mn)/scale exactly k+0.5 must round up (half-to-even would send 2.5 -> 2)."""
    x = np.zeros((1, 1, 1, 32), np.float32)
    x[..., 1] = 15.0                       # scale = 1, mn = 0
    x[..., 2:10] = [0.5, 1.5, 2.5, 3.5, 6.5, 13.5, 14.5, 0.49999997]
    for fn in (oracle.quantize_pack_last_dim, oracle.quantize_pack_last_dim_np):
        code, scale, zero = fn(x, 32, 4)
        q = oracle.unpack_np(code, 4)[0, 0, 0]
        assert list(q[:10]) == [0, 15, 1, 2, 3, 4, 7, 14, 15, 0]
        assert scale.dtype == np.float32 and scale[0, 0, 0, 0] == 1.0


def test_ref3_eleventh_code_is_rounded_then_clamped_to_3(oracle):
    # group of 11: min 0, max 7 -> scale 1; 11th value v -> min(round(v), 3)
    for v, want in [(0.0, 0), (1.0, 1), (2.0, 2), (2.4, 2), (2.5, 3), (3.0, 3), (6.0, 3), (7.0, 3)]:
        x = np.array([0, 7, 1, 2, 3, 4, 5, 6, 7, 0, v], np.float32).reshape(1, 1, 1, 11)
        code, scale, zero = oracle.quantize_pack_last_dim(x, 11, 3)
        q = oracle.unpack_np(code, 3)[0, 0, 0]
        assert list(q[:10]) == [0, 7, 1, 2, 3, 4, 5, 6, 7, 0] and q[10] == want
        hand = sum(c << (3 * i) for i, c in enumerate([0, 7, 1, 2, 3, 4, 5, 6, 7, 0])) | (want << 30)
        assert int(u32(code)[0, 0, 0, 0]) == hand


@pytest.mark.parametrize("bits,g", BITS_G)
def test_c_and_numpy_twins_agree_and_error_bound(oracle, bits, g):
    rng = np.random.default_rng(bits * 1000 + g)
    S = int(np.lcm(g, 11 if bits == 3 else 32 // bits)) * 5
    for dtype in (np.float16, np.float32):
        x = kv_like(rng, (2, 2, 9, S), outlier_axis=2, n_outliers=2, dtype=dtype)
        a = oracle.quantize_pack_last_dim(x, g, bits)
        b = oracle.quantize_pack_last_dim_np(x, g, bits)
        for u, v in zip(a, b):
            assert same_bits(u, v)
        code, scale, zero = a
        # |dequant - x| <= scale/2 (+ rounding of the stored scale/zero), except ref3's 11th code
        q = oracle.unpack_np(code, bits).astype(np.float64).reshape(2, 2, 9, S // g, g)
        xg = x.astype(np.float64).reshape(q.shape)
        s64 = scale.astype(np.float64)[..., None]
        z64 = zero.astype(np.float64)[..., None]
        err = np.abs(s64 * q + z64 - xg)
        qmax = (1 << bits) - 1
        slack = 2.0 ** -10 * (np.abs(z64) + qmax * s64) if dtype == np.float16 else 1e-6 * (np.abs(z64) + qmax * s64)
        bound = s64 / 2 + slack
        if bits == 3:
            err[..., 10] = 0
        assert np.all(err <= bound)


def test_scale_modes_differ_only_in_rounding(oracle):
    rng = np.random.default_rng(5)
    x = kv_like(rng, (1, 4, 64, 256), dtype=np.float32)
    for bits in (2, 4):
        c0, s0, z0 = oracle.quantize_pack_last_dim(x, 32, bits, oracle.SCALE_RECIPROCAL)
        c1, s1, z1 = oracle.quantize_pack_last_dim(x, 32, bits, oracle.SCALE_DIVIDE)
        assert same_bits(c0, c1) and same_bits(z0, z1)
        qmax = np.float32((1 << bits) - 1)
        rng_ = (x.reshape(1, 4, 64, 8, 32).max(-1) - x.reshape(1, 4, 64, 8, 32).min(-1)).astype(np.float32)
        assert same_bits(s1, (rng_ / qmax).astype(np.float32))
        assert same_bits(s0, (rng_ * (np.float32(1) / qmax)).astype(np.float32))
        assert np.all(np.abs(s0.view(np.int32) - s1.view(np.int32)) <= 1)  # at most one ulp apart


def test_argument_errors(oracle):
    x = np.zeros((1, 1, 2, 64), np.float16)
    with pytest.raises(RuntimeError, match="group_length must be 11"):
        oracle.quantize_pack_last_dim(x, 32, 3)
    with pytest.raises(RuntimeError, match="4D"):
        oracle.quantize_pack_last_dim(x[0], 32, 4)
    with pytest.raises(RuntimeError):
        oracle.quantize_pack_last_dim(x, 48, 4)
    with pytest.raises(RuntimeError):
        oracle.quantize_pack_last_dim(x, 11, 3)  # 64 % 11 != 0
