"""GPU parity of the fused dequant-GEMV kernels against the CPU oracle
(reference: quant_cuda/csrc/dequantization_gemv_cuda.cu:7-248).  Tolerance: see helpers.gemv_close
(1e-3 relative plus the fp32 accumulation term)."""
import numpy as np
import pytest
import torch

from helpers import gemv_close, kv_like, same_bits

pytestmark = pytest.mark.gpu


def tt(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def run_case(oracle, dev, bits, g, B, nh, nkv, K, N, seed=0, M=1):
    import KVmix

    rng = np.random.default_rng(seed)
    w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=min(2, K))
    code, scale, zero = oracle.quantize_pack_last_dim(w, g, bits)
    x = rng.standard_normal((B, nh, M, K)).astype(np.float16)
    want16, want64, abs64 = oracle.quantized_gemm(g, x, code, scale, zero, bits, want_f64=True)
    got = KVmix.quantized_gemm(g, tt(x, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), bits)
    assert got.shape == (B, nh, M, N) and got.dtype == torch.float16
    got = got.cpu().numpy()
    ok, worst = gemv_close(got, want64, abs64)
    assert ok, ("vs float64", bits, g, K, N, worst)
    ok, worst = gemv_close(got, want16.astype(np.float64), abs64)
    assert ok, ("vs reference-order fp32", bits, g, K, N, worst)
    return got


QK = [(4, 32), (2, 32), (1, 32), (3, 11)]


@pytest.mark.parametrize("bits,g", QK)
def test_qk_shape(oracle, dev, bits, g):
    """q.K^T: K = head_dim 128, N = quantized tokens (ragged counts included)."""
    for tokens in (g, g * 3, g * 65, g * 131):
        run_case(oracle, dev, bits, g, B=2, nh=4, nkv=4, K=128, N=tokens, seed=tokens)


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32)])
def test_pv_shape(oracle, dev, bits, g):
    """p.V: K = quantized tokens, N = head_dim 128 (64 and 256 too); split-K and tails."""
    for tokens in (1, 15, 32, 100, 257, 2048 + 17):
        run_case(oracle, dev, bits, g, B=1, nh=4, nkv=4, K=tokens, N=128, seed=tokens)
    run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=333, N=64, seed=5)
    run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=333, N=256, seed=6)
    run_case(oracle, dev, bits, g, B=40, nh=32, nkv=32, K=96, N=128, seed=7)   # many samples: no split


@pytest.mark.parametrize("bits,g", QK)
def test_gqa_head_mapping(oracle, dev, bits, g):
    run_case(oracle, dev, bits, g, B=2, nh=8, nkv=2, K=128, N=g * 8 * (1 if bits != 3 else 1), seed=21)
    if bits != 3:
        run_case(oracle, dev, bits, g, B=2, nh=8, nkv=2, K=200, N=128, seed=22)


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32)])
def test_matrix_core_kernel_edges(oracle, dev, bits, g):
    """Shapes that exercise the edges of the matrix-core kernels: a last row chunk moved back to
    end at K (K not a multiple of the chunk), a last tile shifted to end at N, several tiles per
    wave, GQA head groups with ragged tiles, GQA split-K, and a query-row count M > 1."""
    # q.K^T: K below / between / above chunk multiples, N ragged against the 512-code tile
    for K, N in ((32, 512), (40, 544), (96, 1024 + 32), (200, 512 * 5 + 96)):
        run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=K, N=N, seed=K + N)
    run_case(oracle, dev, bits, g, B=1, nh=8, nkv=2, K=128, N=32 * 41, seed=41)      # GQA, 4 heads per block
    run_case(oracle, dev, bits, g, B=1, nh=6, nkv=2, K=128, N=32 * 20, seed=42)      # GQA, 3 heads per kv head
    run_case(oracle, dev, bits, g, B=4, nh=16, nkv=16, K=64, N=512 * 9, seed=43)     # many tiles
    # few tiles: several waves share a tile and slice K (9 chunks of 16 rows over 4 waves leave one idle)
    run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=144, N=2048 + 64, seed=46)
    run_case(oracle, dev, bits, g, B=2, nh=4, nkv=4, K=128, N=32 * 75, seed=47)
    # a launch beyond one resident round of waves with short rows (the two-element kernel for every width)
    run_case(oracle, dev, bits, g, B=32, nh=32, nkv=32, K=32, N=32 * 127, seed=48)
    run_case(oracle, dev, bits, g, B=40, nh=32, nkv=32, K=48, N=32 * 127, seed=49)
    if bits != 1:
        # the wide tiles (2048 codes per wave; rows of 6144 codes and more, launches beyond one round of the plain
        # tiles): a last tile moved back (197 groups = 3 tiles + 5 groups), K not a multiple of the chunk
        from kvmix_amd import _lib
        assert _lib.gemv_plan(g, bits, 0, 17 * 32, 1, 1, 24, 32 * 197)["kernel"].endswith(",1>")
        run_case(oracle, dev, bits, g, B=17, nh=32, nkv=32, K=24, N=32 * 197, seed=50)
        run_case(oracle, dev, bits, g, B=9, nh=64, nkv=64, K=16, N=32 * 192, seed=51)
    # p.V: chunks of 128 rows, K ragged; GQA with split-K; M = 2
    for K in (128, 129, 255, 1000):
        run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=K, N=128, seed=K)
    run_case(oracle, dev, bits, g, B=1, nh=8, nkv=2, K=5000, N=128, seed=44)
    run_case(oracle, dev, bits, g, B=1, nh=4, nkv=4, K=777, N=128, seed=45, M=2)


@pytest.mark.parametrize("nkv", [2, 8])
@pytest.mark.parametrize("bits", [4, 2, 1])
def test_pv_with_probability_rows(oracle, dev, bits, nkv):
    """p.V with four query heads per kv head, and one, and probabilities as x -- flat, peaked and one-hot rows --
    against float64, within the library's general tolerance.  With x >= 0 the code term sum p*scale*code and the
    zero term sum p*zero of an output are large and of opposite sign where the values straddle zero, and the kernels
    form the two separately (the reference adds code*scale + zero per element first), so an output in which they
    cancel shows every bit the code term has lost.  Two things keep it whole: x*scale goes to the matrix cores as
    three bf16 parts that hold the product exactly (two parts, measured faster for four heads per pass, are off by
    up to 2^-17 of every product: 1.4 times the tolerance here), and the code fields of the low nibble of a byte are
    moved up before they become operands -- the matrix cores align the four products of a sum by the operands'
    exponent fields, which all byte patterns share, so a pattern with leading zeros leaves that many fewer bits for
    a sum that one product dominates (with the fields in place: 1.7 times the tolerance on a 2-bit output of
    -0.0007 between terms of +-2.28 under a row with one probability of 0.93).  Also checked: the part of the error
    beyond the output's own fp16 rounding stays below 2^-19 of the code term's magnitude."""
    import KVmix

    g, B, nh, N = 32, 2, 8, 128
    for K, seed in ((128, 1), (1000, 2), (4096, 3)):
        rng = np.random.default_rng(100 * bits + seed)
        w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=2)
        code, scale, zero = oracle.quantize_pack_last_dim(w, g, bits)
        logits = rng.standard_normal((B, nh, 1, K)) * np.array([0.1, 1.0, 4.0, 12.0] * 2).reshape(1, nh, 1, 1)
        x = np.exp(logits - logits.max(-1, keepdims=True))
        x = (x / x.sum(-1, keepdims=True)).astype(np.float16)
        x[0, 0, 0, :] = 0
        x[0, 0, 0, K // 3] = 1  # one-hot: the output is one dequantized row
        _, want64, abs64 = oracle.quantized_gemm(g, x, code, scale, zero, bits, want_f64=True)
        _lib_plan_heads(g, bits, B, nh, nkv, K, N)
        got = KVmix.quantized_gemm(g, tt(x, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), bits).cpu().numpy()
        ok, worst = gemv_close(got, want64, abs64)
        assert ok, ("general tolerance", bits, nkv, K, worst)
        # sum over tokens of p * scale * code, per (batch, head, dim)
        codes = unpack_codes_np(code, bits)                                     # [B, nkv, K, N]
        sc = np.repeat(scale.astype(np.float64), g, axis=-1)                    # [B, nkv, K, N]
        terms = np.repeat(sc * codes, nh // nkv, axis=1)                        # [B, nh, K, N]
        mag = np.einsum("bhk,bhkn->bhn", x[:, :, 0, :].astype(np.float64), terms)[:, :, None, :]
        err = np.abs(got.astype(np.float64) - want64)
        beyond = np.maximum(err - 2.0 ** -11 * np.abs(want64), 0.0)
        assert (beyond <= 2.0 ** -19 * mag + 1e-9).all(), (bits, nkv, K, float((beyond / (2.0 ** -24 * mag + 1e-30)).max()))


def test_pv_terms_that_cancel_carry_their_own_rounding_only(oracle, dev):
    """What the separately formed terms leave: the case a seed scan of the test above found outside the relative
    tolerance -- an output of 7.7e-5 between a code term of +2.6003 and a zero term of -2.6002 under a probability of
    0.999 -- is off by the fp32 rounding of those sums and no more: every output of the call stays within 2^-21 of
    its code term (eight units in the last place of an fp32 of that size) beyond its own fp16 rounding.  The
    reference, which adds code*scale + zero per element first, has no such floor; the general tolerance is not
    asserted here (this one output misses its relative part by a factor of three)."""
    import KVmix

    g, B, nh, nkv, N, K, bits = 32, 2, 8, 8, 128, 256, 4
    rng = np.random.default_rng(1033 * 7 + bits)
    w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=2)
    code, scale, zero = oracle.quantize_pack_last_dim(w, g, bits)
    logits = rng.standard_normal((B, nh, 1, K)) * np.array([0.1, 1.0, 4.0, 12.0] * 2).reshape(1, nh, 1, 1)
    x = np.exp(logits - logits.max(-1, keepdims=True))
    x = (x / x.sum(-1, keepdims=True)).astype(np.float16)
    x[0, 0, 0, :] = 0
    x[0, 0, 0, K // 3] = 1
    _, want64, abs64 = oracle.quantized_gemm(g, x, code, scale, zero, bits, want_f64=True)
    got = KVmix.quantized_gemm(g, tt(x, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), bits).cpu().numpy()
    codes = unpack_codes_np(code, bits)
    sc = np.repeat(scale.astype(np.float64), g, axis=-1)
    mag = np.einsum("bhk,bhkn->bhn", x[:, :, 0, :].astype(np.float64), sc * codes)[:, :, None, :]
    err = np.abs(got.astype(np.float64) - want64)
    beyond = np.maximum(err - 2.0 ** -11 * np.abs(want64), 0.0)
    assert (beyond <= 2.0 ** -21 * mag + 1e-9).all(), float((beyond / (2.0 ** -24 * mag + 1e-30)).max())
    # the output the scan found, and how little of the call is like it
    tol = 1e-3 * np.abs(want64) + 2e-5 * abs64
    assert abs(want64[0, 3, 0, 81] - 7.7192e-5) < 1e-8 and err[0, 3, 0, 81] < 4e-7
    assert (err > tol).mean() < 1e-3


def _lib_plan_heads(g, bits, B, nh, nkv, K, N):
    from kvmix_amd import _lib

    plan = _lib.gemv_plan(g, bits, 0, B * nh, nh // nkv, 1, K, N)
    assert plan["kernel"].startswith("gemv_rows_mfma<%d,%d," % (bits, 4 if nh // nkv == 4 else 1)), plan


def unpack_codes_np(code, bits):
    """[..., W] packed int32 words -> [..., W * 32 / bits] codes (code i of a word at bit i * bits)."""
    w = code.astype(np.int64) & 0xFFFFFFFF
    per = 32 // bits
    out = np.stack([(w >> (bits * i)) & ((1 << bits) - 1) for i in range(per)], axis=-1)
    return out.reshape(code.shape[:-1] + (code.shape[-1] * per,)).astype(np.float64)


def test_reference_3bit_kernel_edges(oracle, dev):
    """gemv_cols3: four and two words per lane, GQA head groups (four query heads per pass), K ragged
    against the 8-row rotation, N ragged against the tile, M = 2."""
    run_case(oracle, dev, 3, 11, B=1, nh=8, nkv=2, K=128, N=11 * 150, seed=51)   # GQA, 4 heads per block
    run_case(oracle, dev, 3, 11, B=1, nh=6, nkv=2, K=128, N=11 * 70, seed=52)    # GQA, heads one by one
    run_case(oracle, dev, 3, 11, B=2, nh=2, nkv=2, K=77, N=11 * 300, seed=53)    # K = 77: ragged sections
    run_case(oracle, dev, 3, 11, B=1, nh=8, nkv=2, K=50, N=11 * 64, seed=54)     # smallest fast tile, GQA
    run_case(oracle, dev, 3, 11, B=1, nh=2, nkv=2, K=128, N=11 * 131, seed=55, M=2)
    run_case(oracle, dev, 3, 11, B=8, nh=8, nkv=8, K=128, N=11 * 733, seed=56)   # wide tiles (4 words per lane)
    run_case(oracle, dev, 3, 11, B=32, nh=32, nkv=32, K=64, N=11 * 300, seed=57)  # four waves per tile slicing K, 16 rows each
    run_case(oracle, dev, 3, 11, B=1, nh=2, nkv=2, K=100, N=11 * 260, seed=58, M=2)  # ... K ragged against the slices, M = 2
    run_case(oracle, dev, 3, 11, B=1, nh=3, nkv=3, K=65, N=11 * 128, seed=59)       # ... one tile exactly, a one-row last slice
    run_case(oracle, dev, 3, 11, B=1, nh=1, nkv=1, K=4096, N=11 * 250, seed=60)     # ... the most rows the sliced form takes
    run_case(oracle, dev, 3, 11, B=32, nh=32, nkv=32, K=32, N=11 * 1024, seed=61)   # too few rows to slice: widest tiles, one wave each
    # whole rows: a block per output row, a wave per 256-word tile over all channel rows (one block per CU, or three)
    from kvmix_amd import _lib
    for B, words in ((8, 733), (7, 1012), (8, 2967)):
        assert _lib.gemv_plan(11, 3, 0, B * 32, 1, 1, 128, 11 * words)["kernel"] == "gemv_cols3<1,4,8,1>"
        run_case(oracle, dev, 3, 11, B=B, nh=32, nkv=32, K=128, N=11 * words, seed=62 + B + words)


@pytest.mark.parametrize("bits,g", [(4, 8), (2, 16), (1, 64), (4, 64), (3, 11)])
def test_generic_shapes(oracle, dev, bits, g):
    """Group sizes and shapes outside the fast kernels (including a 3-bit p.V shape)."""
    unit = int(np.lcm(g, oracle.values_per_word(bits)))
    run_case(oracle, dev, bits, g, B=1, nh=2, nkv=1, K=37, N=unit * 5, seed=31)
    run_case(oracle, dev, bits, g, B=1, nh=2, nkv=2, K=260, N=unit * 2, seed=32)


def test_rows_beyond_m1_use_the_same_formula(oracle, dev):
    run_case(oracle, dev, 4, 32, B=1, nh=2, nkv=2, K=128, N=256, seed=41, M=3)
    run_case(oracle, dev, 2, 32, B=1, nh=2, nkv=1, K=300, N=128, seed=42, M=2)


@pytest.mark.parametrize("bits,g", QK)
def test_closed_form_cases(oracle, dev, bits, g):
    import KVmix

    rng = np.random.default_rng(bits)
    B, nh, K = 1, 2, 128
    N = int(np.lcm(g, oracle.values_per_word(bits))) * 6
    qmax = (1 << bits) - 1
    q = rng.integers(0, qmax + 1, size=(B, nh, K, N))
    if bits == 3:
        q[..., 10::11] &= 3
    code = oracle.pack_np(q, bits)
    ones = np.ones((B, nh, K, N // g), np.float16)
    zeros = np.zeros_like(ones)
    x1 = np.ones((B, nh, 1, K), np.float16)
    # all-ones x, scale 1, zero 0 -> exact integer column sums
    out = KVmix.quantized_gemm(g, tt(x1, dev), tt(code, dev), tt(ones, dev), tt(zeros, dev), bits).cpu().numpy()
    assert np.array_equal(out.astype(np.int64)[:, :, 0], q.sum(axis=2))
    # one-hot x -> one dequantized row, bit-exact after fp16 rounding
    scale = (rng.random((B, nh, K, N // g)) + 0.5).astype(np.float16)
    zero = rng.standard_normal((B, nh, K, N // g)).astype(np.float16)
    e = np.zeros((B, nh, 1, K), np.float16)
    e[..., 77] = 1
    out = KVmix.quantized_gemm(g, tt(e, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), bits).cpu().numpy()
    row = np.repeat(scale.astype(np.float64), g, -1)[:, :, 77] * q[:, :, 77] + np.repeat(zero.astype(np.float64), g, -1)[:, :, 77]
    assert same_bits(out[:, :, 0], row.astype(np.float16))
    # scale 0 -> sum_k x[k] zero[k, n/g]
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    out = KVmix.quantized_gemm(g, tt(x, dev), tt(code, dev), tt(zeros, dev), tt(zero, dev), bits).cpu().numpy()
    want = np.repeat(np.einsum("bhmk,bhkg->bhmg", x.astype(np.float64), zero.astype(np.float64)), g, -1)
    ab = np.repeat(np.einsum("bhmk,bhkg->bhmg", np.abs(x.astype(np.float64)), np.abs(zero.astype(np.float64))), g, -1)
    ok, worst = gemv_close(out, want, ab)
    assert ok, worst


def test_strided_views_of_a_larger_cache_and_sliced_probabilities(oracle, dev):
    """Operands passed as views (capacity-padded cache, p[..., :Tq] slice) are read in place."""
    import KVmix

    rng = np.random.default_rng(8)
    B, H, D, Tq, cap = 2, 4, 128, 96, 256
    k = kv_like(rng, (B, H, D, Tq))
    code, scale, zero = oracle.quantize_pack_last_dim(k, 32, 4)
    cbuf = torch.zeros(B, H, D, cap // 8, dtype=torch.int32, device=dev)
    sbuf = torch.zeros(B, H, D, cap // 32, dtype=torch.float16, device=dev)
    zbuf = torch.zeros_like(sbuf)
    cbuf[..., : Tq // 8] = tt(code, dev)
    sbuf[..., : Tq // 32] = tt(scale, dev)
    zbuf[..., : Tq // 32] = tt(zero, dev)
    q = rng.standard_normal((B, H, 1, D)).astype(np.float16)
    got = KVmix.quantized_gemm(32, tt(q, dev), cbuf[..., : Tq // 8], sbuf[..., : Tq // 32], zbuf[..., : Tq // 32], 4)
    _, w64, a64 = oracle.quantized_gemm(32, q, code, scale, zero, 4, want_f64=True)
    ok, worst = gemv_close(got.cpu().numpy(), w64, a64)
    assert ok, worst
    # p.V with p a slice of the probability row (models/modeling_llama_KVmix.py:205-206)
    v = kv_like(rng, (B, H, Tq, D))
    code, scale, zero = oracle.quantize_pack_last_dim(v, 32, 2)
    p = rng.random((B, H, 1, Tq + 40)).astype(np.float16)
    got = KVmix.quantized_gemm(32, tt(p, dev)[..., :Tq], tt(code, dev), tt(scale, dev), tt(zero, dev), 2)
    _, w64, a64 = oracle.quantized_gemm(32, np.ascontiguousarray(p[..., :Tq]), code, scale, zero, 2, want_f64=True)
    ok, worst = gemv_close(got.cpu().numpy(), w64, a64)
    assert ok, worst


def test_empty_k_gives_zeros(dev):
    import KVmix

    q = torch.zeros(1, 2, 1, 0, dtype=torch.float16, device=dev)
    code = torch.zeros(1, 2, 0, 16, dtype=torch.int32, device=dev)
    sz = torch.zeros(1, 2, 0, 4, dtype=torch.float16, device=dev)
    out = KVmix.quantized_gemm(32, q, code, sz, sz, 4)
    assert out.shape == (1, 2, 1, 128) and (out == 0).all()


def test_config0_single_layer(oracle, dev):
    """BASELINE config 0: B=1, 32 heads, head_dim 128, 4096 tokens, 4-bit, group 32, 128-token
    fp16 window; K, V ~N(0,1) with 4 outlier channels per head x10; codes bit-exact, q.K^T and
    softmax.V within tolerance of the oracle."""
    import KVmix

    torch.manual_seed(0)
    B, H, D, T, R, g, bits = 1, 32, 128, 4096, 128, 32, 4
    K = torch.randn(B, H, T, D).half()
    V = torch.randn(B, H, T, D).half()
    for h in range(H):
        ch = torch.randperm(D)[:4]
        K[:, h, :, ch] *= 10
        V[:, h, :, ch] *= 10
    q = torch.randn(B, H, 1, D).half()
    Tq = T - R
    Kq_in = K[:, :, :Tq].transpose(2, 3).contiguous()
    Vq_in = V[:, :, :Tq].contiguous()
    kc, ks, km = KVmix.quantize_pack_last_dim_cuda(Kq_in.to(dev), g, bits)
    vc, vs, vm = KVmix.quantize_pack_last_dim_cuda(Vq_in.to(dev), g, bits)
    okc, oks, okm = oracle.quantize_pack_last_dim(Kq_in.numpy(), g, bits)
    ovc, ovs, ovm = oracle.quantize_pack_last_dim(Vq_in.numpy(), g, bits)
    for a, b in ((kc, okc), (ks, oks), (km, okm), (vc, ovc), (vs, ovs), (vm, ovm)):
        assert same_bits(a.cpu().numpy(), b)
    att_q = KVmix.quantized_gemm(g, q.to(dev), kc, ks, km, bits)
    o16, o64, a64 = oracle.quantized_gemm(g, q.numpy(), okc, oks, okm, bits, want_f64=True)
    ok, worst = gemv_close(att_q.cpu().numpy(), o64, a64)
    assert ok, worst
    # the rest of the decode step exactly as models/modeling_llama_KVmix.py:184-211 does it
    att_f = torch.matmul(q.to(dev), K[:, :, Tq:].to(dev).transpose(2, 3))
    w = torch.cat([att_q.float(), att_f.float()], -1) / (D ** 0.5)
    p = torch.softmax(w, dim=-1, dtype=torch.float32).half()
    out = KVmix.quantized_gemm(g, p[..., :Tq], vc, vs, vm, bits) + torch.matmul(p[..., Tq:], V[:, :, Tq:].to(dev))
    # oracle on the same probabilities (isolates the p.V kernel), then end to end
    pn = p.cpu().numpy()
    _, v64, va64 = oracle.quantized_gemm(g, np.ascontiguousarray(pn[..., :Tq]), ovc, ovs, ovm, bits, want_f64=True)
    got_q = KVmix.quantized_gemm(g, p[..., :Tq], vc, vs, vm, bits).cpu().numpy()
    ok, worst = gemv_close(got_q, v64, va64)
    assert ok, worst
    cache = (okc, K[:, :, Tq:].numpy(), oks, okm, ovc, V[:, :, Tq:].numpy(), ovs, ovm, T)
    k_new = np.zeros((B, H, 0, D), np.float16)
    want_out, want_p, _ = oracle.attention_decode_step(q.numpy(), k_new, k_new, cache, bits, bits, 1.0, 1.0, g)
    np.testing.assert_allclose(pn.astype(np.float64), want_p.astype(np.float64), rtol=4e-3, atol=1e-5)
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want_out.astype(np.float64), rtol=4e-3, atol=4e-3)


def test_full_size_properties_b16_t8192(dev):
    """Target shape (B=16, 32 heads, 8064 quantized tokens, head_dim 128), checked through
    properties that need no CPU oracle: integer column sums (exact), one-hot rows (exact),
    and agreement with torch's own fp32 matmul of the dequantized cache on a slice."""
    import KVmix

    torch.manual_seed(1)
    B, H, D, Tq, g = 16, 32, 128, 8064, 32
    for bits in (4, 2):
        qmax = (1 << bits) - 1
        vpw = 32 // bits
        # keys: [B,H,D,Tq/vpw]
        kcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tq // vpw), dtype=torch.int64, device=dev).to(torch.int32)
        ones = torch.ones(B, H, D, Tq // g, dtype=torch.float16, device=dev)
        shifts = torch.arange(0, 32, bits, device=dev, dtype=torch.int32)
        x1 = torch.ones(B, H, 1, D, dtype=torch.float16, device=dev)
        out = KVmix.quantized_gemm(g, x1, kcode, ones, torch.zeros_like(ones), bits)
        sums = torch.zeros(B, H, Tq, dtype=torch.int32, device=dev)
        for b0 in range(0, B, 4):
            qk = ((kcode[b0:b0 + 4].unsqueeze(-1) >> shifts) & qmax).reshape(4, H, D, Tq)
            sums[b0:b0 + 4] = qk.sum(2)
        assert torch.equal(out[:, :, 0].to(torch.int32), sums)          # sums <= 128*15 are exact in fp16
        # values: [B,H,Tq,D/vpw]; one-hot p picks one dequantized row exactly
        vcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tq, D // vpw), dtype=torch.int64, device=dev).to(torch.int32)
        vs = (torch.rand(B, H, Tq, D // g, device=dev) + 0.5).half()
        vz = torch.randn(B, H, Tq, D // g, device=dev).half()
        p = torch.zeros(B, H, 1, Tq, dtype=torch.float16, device=dev)
        row = 5003
        p[..., row] = 1
        out = KVmix.quantized_gemm(g, p, vcode, vs, vz, bits)
        qv = ((vcode[:, :, row].unsqueeze(-1) >> shifts) & qmax).reshape(B, H, D).float()
        want = (vs[:, :, row].float().repeat_interleave(g, -1) * qv + vz[:, :, row].float().repeat_interleave(g, -1)).half()
        assert torch.equal(out[:, :, 0], want)
        # dense check on two batch entries with torch's fp32 matmul
        pr = torch.softmax(torch.randn(2, H, 1, Tq, device=dev), -1).half()
        out = KVmix.quantized_gemm(g, pr, vcode[:2], vs[:2], vz[:2], bits).float()
        qv = ((vcode[:2].unsqueeze(-1) >> shifts) & qmax).reshape(2, H, Tq, D).float()
        deq = vs[:2].float().repeat_interleave(g, -1) * qv + vz[:2].float().repeat_interleave(g, -1)
        ref = torch.matmul(pr.float(), deq)
        ab = torch.matmul(pr.float().abs(), deq.abs())
        assert ((out - ref).abs() <= 1e-3 * ref.abs() + 2e-5 * ab).all()


def _unpack_torch(code, bits):
    """Reference-layout unpack on the GPU with torch integer ops (test-side checker)."""
    dev = code.device
    if bits == 3:
        shifts = torch.tensor([3 * i for i in range(10)] + [30], device=dev, dtype=torch.int32)
        masks = torch.tensor([7] * 10 + [3], device=dev, dtype=torch.int32)
    else:
        shifts = torch.arange(0, 32, bits, device=dev, dtype=torch.int32)
        masks = torch.full((32 // bits,), (1 << bits) - 1, device=dev, dtype=torch.int32)
    q = (code.unsqueeze(-1) >> shifts) & masks
    return q.reshape(code.shape[:-1] + (code.shape[-1] * shifts.numel(),))


def test_full_size_properties_gqa_32k(dev):
    """BASELINE configs[2] shape: 32 query heads on 8 kv heads, head_dim 128, batch 16, 32768
    tokens, reference 3-bit keys (32637 = 11 * 2967 quantized tokens) and 2-bit values (32640)."""
    import KVmix

    torch.manual_seed(2)
    B, H, Hkv, D = 16, 32, 8, 128
    Tqk, Tqv = 32637, 32640
    kcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, D, Tqk // 11), dtype=torch.int64, device=dev).to(torch.int32)
    ones = torch.ones(B, Hkv, D, Tqk // 11, dtype=torch.float16, device=dev)
    x1 = torch.ones(B, H, 1, D, dtype=torch.float16, device=dev)
    out = KVmix.quantized_gemm(11, x1, kcode, ones, torch.zeros_like(ones), 3)
    assert out.shape == (B, H, 1, Tqk)
    for b0 in range(0, B, 4):
        sums = _unpack_torch(kcode[b0:b0 + 4], 3).sum(2)                       # [4, Hkv, Tqk] <= 128*7
        got = out[b0:b0 + 4, :, 0].to(torch.int32).reshape(4, Hkv, H // Hkv, Tqk)
        assert torch.equal(got, sums.unsqueeze(2).expand_as(got))              # every head of a group
    # values: one-hot probabilities pick one dequantized row, per query head
    vcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, Tqv, D // 16), dtype=torch.int64, device=dev).to(torch.int32)
    vs = (torch.rand(B, Hkv, Tqv, D // 32, device=dev) + 0.5).half()
    vz = torch.randn(B, Hkv, Tqv, D // 32, device=dev).half()
    p = torch.zeros(B, H, 1, Tqv, dtype=torch.float16, device=dev)
    rows = torch.randint(0, Tqv, (H,), device=dev)
    for h in range(H):
        p[:, h, 0, rows[h]] = 1
    out = KVmix.quantized_gemm(32, p, vcode, vs, vz, 2)
    for h in range(H):
        r, kvh = int(rows[h]), h // (H // Hkv)
        qv = _unpack_torch(vcode[:, kvh, r], 2).float()
        want = (vs[:, kvh, r].float().repeat_interleave(32, -1) * qv + vz[:, kvh, r].float().repeat_interleave(32, -1)).half()
        assert torch.equal(out[:, h, 0], want), h
    # dense check of two batch entries against torch's fp32 matmul of the dequantized values
    pr = torch.softmax(torch.randn(2, H, 1, Tqv, device=dev), -1).half()
    out = KVmix.quantized_gemm(32, pr, vcode[:2], vs[:2], vz[:2], 2).float()
    deq = vs[:2].float().repeat_interleave(32, -1) * _unpack_torch(vcode[:2], 2).float() + vz[:2].float().repeat_interleave(32, -1)
    deq = deq.repeat_interleave(H // Hkv, dim=1)
    ref = torch.matmul(pr.float(), deq)
    ab = torch.matmul(pr.float().abs(), deq.abs())
    assert ((out - ref).abs() <= 1e-3 * ref.abs() + 2e-5 * ab).all()


def test_full_size_properties_config1_b8_t8192(oracle, dev):
    """BASELINE configs[1]'s two 3-bit legs at full size (batch 8, 32 heads, head_dim 128, 8192 tokens,
    128-token window): q.K^T over keys in the reference's 3-bit words (8063 = 11 * 733 quantized
    tokens) and p.V over values in the dense 3-bit stream (8064 tokens; no reference counterpart).
    Properties that need no CPU run at this size -- exact integer column sums, exact one-hot rows,
    torch's fp32 matmul of the dequantized operand on a two-batch slice -- and the oracle itself on
    one (batch, head) pair."""
    import KVmix
    from helpers import dequantize_torch, unpack_codes_torch
    from kvmix_amd import ops

    torch.manual_seed(5)
    B, H, D = 8, 32, 128
    Tqk, Tqv = 8063, 8064
    # keys, reference 3-bit words: all-ones query, scale 1, zero 0 -> column sums of the codes (<= 128 * 7)
    kcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tqk // 11), dtype=torch.int64, device=dev).to(torch.int32)
    ones = torch.ones(B, H, D, Tqk // 11, dtype=torch.float16, device=dev)
    x1 = torch.ones(B, H, 1, D, dtype=torch.float16, device=dev)
    out = KVmix.quantized_gemm(11, x1, kcode, ones, torch.zeros_like(ones), 3)
    assert out.shape == (B, H, 1, Tqk)
    assert torch.equal(out[:, :, 0].to(torch.int32), unpack_codes_torch(kcode, 3).sum(2))
    # one-hot query: one dequantized channel row, exact after the fp16 rounding
    ks = (torch.rand(B, H, D, Tqk // 11, device=dev) + 0.5).half()
    kz = torch.randn(B, H, D, Tqk // 11, device=dev).half()
    e = torch.zeros(B, H, 1, D, dtype=torch.float16, device=dev)
    e[..., 101] = 1
    out = KVmix.quantized_gemm(11, e, kcode, ks, kz, 3)
    want = dequantize_torch(kcode[:, :, 101], ks[:, :, 101], kz[:, :, 101], 3, 11).half()
    assert torch.equal(out[:, :, 0], want)
    # random queries against torch's fp32 matmul on two batch entries, and the oracle on one (batch, head)
    q = torch.randn(B, H, 1, D, device=dev).half()
    out = KVmix.quantized_gemm(11, q, kcode, ks, kz, 3)
    deq = dequantize_torch(kcode[:2], ks[:2], kz[:2], 3, 11)                      # [2, H, D, Tqk]
    ref = torch.matmul(q[:2].float(), deq)
    ab = torch.matmul(q[:2].float().abs(), deq.abs())
    assert ((out[:2].float() - ref).abs() <= 1e-3 * ref.abs() + 2e-5 * ab).all()
    b, h = 7, 30
    _, w64, a64 = oracle.quantized_gemm(11, q[b:b + 1, h:h + 1].cpu().numpy(), kcode[b:b + 1, h:h + 1].cpu().numpy(),
                                        ks[b:b + 1, h:h + 1].cpu().numpy(), kz[b:b + 1, h:h + 1].cpu().numpy(), 3,
                                        want_f64=True)
    ok, worst = gemv_close(out[b:b + 1, h:h + 1].cpu().numpy(), w64, a64)
    assert ok, worst
    del kcode, ones, ks, kz, deq, ref, ab

    # values, dense 3-bit stream
    vcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tqv, D * 3 // 32), dtype=torch.int64, device=dev).to(torch.int32)
    vs = (torch.rand(B, H, Tqv, D // 32, device=dev) + 0.5).half()
    vz = torch.randn(B, H, Tqv, D // 32, device=dev).half()
    p = torch.zeros(B, H, 1, Tqv, dtype=torch.float16, device=dev)
    rows = torch.randint(0, Tqv, (H,), device=dev)
    for hh in range(H):
        p[:, hh, 0, rows[hh]] = 1
    out = ops.quantized_gemm(32, p, vcode, vs, vz, 3, fmt=ops.FMT_DENSE3)
    for hh in range(H):
        r = int(rows[hh])
        want = dequantize_torch(vcode[:, hh, r], vs[:, hh, r], vz[:, hh, r], 3, 32, dense3=True).half()
        assert torch.equal(out[:, hh, 0], want), hh
    # all-ones probabilities over the first 256 tokens, scale 1, zero 0: exact sums (<= 256 * 7, exact in fp16)
    one = torch.ones_like(vs[:, :, :256])
    out = ops.quantized_gemm(32, torch.ones(B, H, 1, 256, dtype=torch.float16, device=dev), vcode[:, :, :256], one,
                             torch.zeros_like(one), 3, fmt=ops.FMT_DENSE3)
    assert torch.equal(out[:, :, 0].to(torch.int32), unpack_codes_torch(vcode[:, :, :256], 3, dense3=True).sum(2))
    pr = torch.softmax(torch.randn(B, H, 1, Tqv, device=dev), -1).half()
    out = ops.quantized_gemm(32, pr, vcode, vs, vz, 3, fmt=ops.FMT_DENSE3)
    deq = dequantize_torch(vcode[:2], vs[:2], vz[:2], 3, 32, dense3=True)       # [2, H, Tqv, D]
    ref = torch.matmul(pr[:2].float(), deq)
    ab = torch.matmul(pr[:2].float().abs(), deq.abs())
    assert ((out[:2].float() - ref).abs() <= 1e-3 * ref.abs() + 2e-5 * ab).all()
    _, w64, a64 = oracle.quantized_gemm_dense3(32, pr[b:b + 1, h:h + 1].cpu().numpy(), vcode[b:b + 1, h:h + 1].cpu().numpy(),
                                               vs[b:b + 1, h:h + 1].cpu().numpy(), vz[b:b + 1, h:h + 1].cpu().numpy(),
                                               want_f64=True)
    ok, worst = gemv_close(out[b:b + 1, h:h + 1].cpu().numpy(), w64, a64)
    assert ok, worst


@pytest.mark.parametrize("bits", [1, 2])
def test_full_size_properties_batch128_t4096(dev, bits):
    """BASELINE configs[3] at its largest batch: 128 x 32 heads, 4064 quantized tokens, 1/2 bits."""
    import KVmix

    torch.manual_seed(3)
    B, H, D, Tq, g = 128, 32, 128, 4064, 32
    vpw = 32 // bits
    kcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tq // vpw), dtype=torch.int64, device=dev).to(torch.int32)
    ones = torch.ones(B, H, D, Tq // g, dtype=torch.float16, device=dev)
    x1 = torch.ones(B, H, 1, D, dtype=torch.float16, device=dev)
    out = KVmix.quantized_gemm(g, x1, kcode, ones, torch.zeros_like(ones), bits)
    for b0 in range(0, B, 16):
        assert torch.equal(out[b0:b0 + 16, :, 0].to(torch.int32), _unpack_torch(kcode[b0:b0 + 16], bits).sum(2))
    del kcode, ones
    vcode = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tq, D // vpw), dtype=torch.int64, device=dev).to(torch.int32)
    vs = (torch.rand(B, H, Tq, D // g, device=dev) + 0.5).half()
    vz = torch.randn(B, H, Tq, D // g, device=dev).half()
    p = torch.zeros(B, H, 1, Tq, dtype=torch.float16, device=dev)
    p[..., 4063] = 1
    out = KVmix.quantized_gemm(g, p, vcode, vs, vz, bits)
    qv = _unpack_torch(vcode[:, :, 4063], bits).float()
    want = (vs[:, :, 4063].float().repeat_interleave(g, -1) * qv + vz[:, :, 4063].float().repeat_interleave(g, -1)).half()
    assert torch.equal(out[:, :, 0], want)
    # all-ones probabilities with scale 1, zero 0: exact integer sums over tokens (<= 4064 * 3, exact in fp16 up to 2048)
    if bits == 1:
        one = torch.ones_like(vs)
        out = KVmix.quantized_gemm(g, torch.ones_like(p)[..., :2016], vcode[:, :, :2016], one[:, :, :2016],
                                   torch.zeros_like(one)[:, :, :2016], bits)
        assert torch.equal(out[:, :, 0].to(torch.int32), _unpack_torch(vcode[:, :, :2016], bits).sum(2))


@pytest.mark.parametrize("batch", [1, 16, 64])
@pytest.mark.parametrize("bits", [1, 2])
def test_config3_sizes_against_the_oracle(oracle, dev, bits, batch):
    """BASELINE configs[3] at its smaller batches (T = 4096, residual 32: 4064 quantized tokens, 32 heads, 1 and 2
    bits): whole q.K^T and p.V launches of those sizes against the oracle (the largest batch has its closed-form
    test above)."""
    run_case(oracle, dev, bits, 32, B=batch, nh=32, nkv=32, K=128, N=4064, seed=300 + batch + bits)
    run_case(oracle, dev, bits, 32, B=batch, nh=32, nkv=32, K=4064, N=128, seed=400 + batch + bits)


def test_more_slices_than_one_grid_dimension_holds(oracle, dev):
    """B x heads beyond 65535 (the limit of grid.y): the call goes out in parts over whole kv heads."""
    run_case(oracle, dev, 4, 32, B=16385, nh=4, nkv=4, K=16, N=64, seed=71)      # 65540 slices, two parts
    run_case(oracle, dev, 2, 32, B=8193, nh=8, nkv=2, K=16, N=64, seed=72)       # 65544 query heads on 16386 kv heads
    run_case(oracle, dev, 1, 32, B=1, nh=2, nkv=2, K=8, N=32, seed=73, M=65537)  # rows of the left operand beyond grid.z
