"""Dense 3-bit stream (extension: the reference has no such format, so there is no reference
parity to claim).  The oracle's C and numpy forms are pinned by hand-packed words, a brute-force
inverse and the same closed-form grid as the reference formats."""
import numpy as np

from helpers import gemv_close, kv_like, same_bits


def u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_hand_packed_stream(oracle):
    q = np.zeros(32, np.int64)
    q[0], q[1], q[10], q[11], q[21], q[31] = 5, 7, 6, 1, 7, 4
    w = u32(oracle.pack_dense3_np(q))
    # code i at stream bit 3i: 10 straddles words 0/1 (bits 30..32), 21 straddles 1/2 (63..65)
    stream = sum(int(c) << (3 * i) for i, c in enumerate(q))
    assert [int(x) for x in w] == [stream & 0xFFFFFFFF, (stream >> 32) & 0xFFFFFFFF, stream >> 64]
    assert int(w[0]) == (5 | 7 << 3 | (6 & 3) << 30) and int(w[1]) & 1 == 6 >> 2


def test_pack_unpack_bruteforce(oracle):
    for pos in range(32):
        for c in range(8):
            q = np.zeros(32, np.int64)
            q[pos] = c
            w = oracle.pack_dense3_np(q)
            assert np.array_equal(oracle.unpack_dense3_np(w), q)
            out = np.zeros(32, np.int32)
            oracle.lib().kvo_unpack_dense3_row(w.ctypes.data, 32, out.ctypes.data)
            assert np.array_equal(out, q)


def test_quantizer_grid_and_twin(oracle):
    rng = np.random.default_rng(0)
    k = rng.integers(0, 8, size=(2, 2, 3, 96))
    kg = k.reshape(2, 2, 3, 3, 32)
    kg[..., 0], kg[..., 1] = 0, 7
    x = (np.float32(-1.5) + k * np.float32(0.25)).astype(np.float16)
    code, scale, zero = oracle.quantize_pack_dense3(x, 32)
    assert np.array_equal(oracle.unpack_dense3_np(code), k)
    assert same_bits(code, oracle.pack_dense3_np(k))
    assert np.all(scale == np.float16(0.25)) and np.all(zero == np.float16(-1.5))
    # random data: same codes as the 4-bit path's arithmetic with qmax 7 (numpy restatement)
    x = kv_like(rng, (1, 2, 9, 128), outlier_axis=2, n_outliers=1)
    code, scale, zero = oracle.quantize_pack_dense3(x, 32)
    g = x.reshape(1, 2, 9, 4, 32).astype(np.float32)
    mn = g.min(-1)
    sc = ((g.max(-1) - mn) / np.float32(7)).astype(np.float32)
    q = np.clip(oracle.round_half_away(((g - mn[..., None]) / sc[..., None]).astype(np.float32)), 0, 7)
    assert np.array_equal(oracle.unpack_dense3_np(code), q.reshape(1, 2, 9, 128).astype(np.int32))
    assert same_bits(zero, mn.astype(np.float16))
    assert same_bits(scale, ((g.max(-1) - mn) * (np.float32(1) / np.float32(7))).astype(np.float32).astype(np.float16))


def test_gemm_equals_float64_matmul(oracle):
    rng = np.random.default_rng(1)
    for K, N in ((64, 256), (200, 128)):
        w = kv_like(rng, (1, 2, K, N), outlier_axis=2, n_outliers=2)
        code, scale, zero = oracle.quantize_pack_dense3(w, 32)
        x = rng.standard_normal((1, 4, 1, K)).astype(np.float16)
        out, o64, a64 = oracle.quantized_gemm_dense3(32, x, code, scale, zero, want_f64=True)
        deq = np.repeat(oracle.dequantize_dense3_np(code, scale, zero).astype(np.float64), 2, axis=1)
        want = np.einsum("bhmk,bhkn->bhmn", x.astype(np.float64), deq)
        np.testing.assert_allclose(o64, want, rtol=1e-12, atol=1e-12)
        ok, worst = gemv_close(out, want, a64)
        assert ok, worst
