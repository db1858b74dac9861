"""GPU parity of the dense 3-bit extension (quantizer, key-from-tokens quantizer, both GEMV
shapes) against the oracle.  No reference counterpart exists for this format."""
import numpy as np
import pytest
import torch

from helpers import gemv_close, kv_like, same_bits

pytestmark = pytest.mark.gpu


def tt(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def test_quantizer_matches_oracle(oracle, dev):
    from kvmix_amd import ops

    rng = np.random.default_rng(0)
    for shape, g in (((2, 3, 5, 128), 32), ((1, 2, 130, 96), 32), ((1, 1, 7, 256), 64), ((1, 2, 3, 128), 128)):
        for dtype in (np.float16, np.float32):
            x = kv_like(rng, shape, outlier_axis=2, n_outliers=1, dtype=dtype)
            x[0, 0, 0, :g] = dtype(2.5)
            got = ops.quantize_pack_dense3(tt(x, dev), g)
            want = oracle.quantize_pack_dense3(x, g)
            for a, b in zip(got, want):
                assert same_bits(a.cpu().numpy(), b), (shape, g, dtype)


def test_key_tokens_kernel(oracle, dev):
    from kvmix_amd import _lib

    L = _lib.load()
    rng = np.random.default_rng(1)
    B, H, D, n = 2, 2, 128, 96
    tail = kv_like(rng, (B, H, n + 3, D), outlier_axis=3)
    t = tt(tail, dev)
    code = torch.zeros(B, H, D, n * 3 // 32, dtype=torch.int32, device=dev)
    scale = torch.zeros(B, H, D, n // 32, dtype=torch.float16, device=dev)
    zero = torch.zeros_like(scale)
    rc = L.kvmix_quant_pack_key_tokens(t.data_ptr(), B * H, n, D, t.stride(1), t.stride(2), 32, 3, _lib.FMT_DENSE3,
                                       _lib.SCALE_RECIPROCAL, code.data_ptr(), code.stride(1), code.stride(2),
                                       scale.data_ptr(), zero.data_ptr(), scale.stride(1), scale.stride(2),
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.strerror(rc)
    want = oracle.quantize_pack_dense3(np.ascontiguousarray(tail[:, :, :n].transpose(0, 1, 3, 2)), 32)
    for a, b in zip((code, scale, zero), want):
        assert same_bits(a.cpu().numpy(), b)


@pytest.mark.parametrize("K,N,B,nh,nkv", [(128, 32 * 67, 2, 4, 4), (128, 256, 1, 8, 2), (2048 + 40, 128, 1, 4, 4),
                                         (300, 128, 2, 8, 2), (37, 96, 1, 2, 1), (5, 128, 1, 2, 2)])
def test_gemv_matches_oracle(oracle, dev, K, N, B, nh, nkv):
    from kvmix_amd import ops

    rng = np.random.default_rng(K + N)
    w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=min(2, K))
    code, scale, zero = oracle.quantize_pack_dense3(w, 32)
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    want16, want64, abs64 = oracle.quantized_gemm_dense3(32, x, code, scale, zero, want_f64=True)
    got = ops.quantized_gemm(32, tt(x, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), 3, fmt=ops.FMT_DENSE3)
    ok, worst = gemv_close(got.cpu().numpy(), want64, abs64)
    assert ok, worst


@pytest.mark.parametrize("nkv", [2, 8])
def test_pv_with_probability_rows(oracle, dev, nkv):
    """p.V over dense 3-bit values with probabilities as x (flat, peaked and one-hot rows; four query heads per kv
    head, and one): the case of tests/test_gpu_gemv.py::test_pv_with_probability_rows, in which the code term and
    the zero term of an output cancel, within the same general tolerance (the field pairs that sit at bit 0 of
    their byte are moved up by two before they become matrix-core operands)."""
    from kvmix_amd import ops

    B, nh, N = 2, 8, 128
    for K, seed in ((128, 1), (1000, 2), (4096, 3)):
        rng = np.random.default_rng(300 + seed)
        w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=2)
        code, scale, zero = oracle.quantize_pack_dense3(w, 32)
        logits = rng.standard_normal((B, nh, 1, K)) * np.array([0.1, 1.0, 4.0, 12.0] * 2).reshape(1, nh, 1, 1)
        x = np.exp(logits - logits.max(-1, keepdims=True))
        x = (x / x.sum(-1, keepdims=True)).astype(np.float16)
        x[0, 0, 0, :] = 0
        x[0, 0, 0, K // 3] = 1
        _, want64, abs64 = oracle.quantized_gemm_dense3(32, x, code, scale, zero, want_f64=True)
        got = ops.quantized_gemm(32, tt(x, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), 3, fmt=ops.FMT_DENSE3)
        ok, worst = gemv_close(got.cpu().numpy(), want64, abs64)
        assert ok, (nkv, K, worst)


def test_one_hot_row_is_exact(oracle, dev):
    from kvmix_amd import ops

    rng = np.random.default_rng(5)
    B, nh, K, N = 1, 2, 128, 512
    q = rng.integers(0, 8, size=(B, nh, K, N))
    code = oracle.pack_dense3_np(q)
    scale = (rng.random((B, nh, K, N // 32)) + 0.5).astype(np.float16)
    zero = rng.standard_normal((B, nh, K, N // 32)).astype(np.float16)
    e = np.zeros((B, nh, 1, K), np.float16)
    e[..., 90] = 1
    out = ops.quantized_gemm(32, tt(e, dev), tt(code, dev), tt(scale, dev), tt(zero, dev), 3, fmt=ops.FMT_DENSE3)
    row = np.repeat(scale.astype(np.float64), 32, -1)[:, :, 90] * q[:, :, 90] + np.repeat(zero.astype(np.float64), 32, -1)[:, :, 90]
    assert same_bits(out.cpu().numpy()[:, :, 0], row.astype(np.float16))
