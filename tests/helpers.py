"""Shared input generators and comparison helpers for the parity tests."""
import numpy as np


def kv_like(rng, shape, outlier_axis=None, n_outliers=4, scale=10.0, dtype=np.float16):
    """~N(0,1) data with a few channels scaled up (the benchmark's synthetic KV)."""
    x = rng.standard_normal(shape).astype(np.float32)
    if outlier_axis is not None:
        n = shape[outlier_axis]
        idx = rng.permutation(n)[:n_outliers]
        sl = [slice(None)] * len(shape)
        sl[outlier_axis] = idx
        x[tuple(sl)] *= scale
    return x.astype(dtype)


def same_bits(a, b):
    """Bit-for-bit equality of two numpy arrays of equal dtype (NaNs compare by payload)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


# GEMV tolerance (written once, used by every GEMV test):
#   |got - want| <= 1e-3 * |want| + 2e-5 * sum_k |x_k| |w_kn|
# The first term is the stated 1e-3 relative bound (it also covers the two results
# rounding to different neighbouring fp16 values, 2^-10 relative); the second bounds
# the fp32 accumulation-order difference in units of the absolute sum of the terms
# (fp32 eps = 6e-8; a few hundred ulps of head-room for K up to 32k).
GEMV_RTOL = 1e-3
GEMV_ABS_TERM = 2e-5


def gemv_close(got, want, abs_sum):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    tol = GEMV_RTOL * np.abs(want) + GEMV_ABS_TERM * np.asarray(abs_sum, np.float64)
    bad = err > tol
    return not bad.any(), float((err / np.maximum(tol, 1e-30)).max())


def unpack_codes_torch(code, bits, dense3=False):
    """Packed words [..., W] int32 -> integer codes [..., n] on the tensor's device, with torch integer
    ops only (a checker that shares nothing with the HIP kernels or the C oracle).
    Reference layouts: bits 1/2/4, 32/bits codes per word, code i at bit i*bits; bits 3, eleven codes per
    word (ten 3-bit fields, then a 2-bit field at bit 30).  dense3: 32 codes in three words, code i at
    bits [3i, 3i+3) of the 96-bit little-endian stream."""
    import torch

    dev = code.device
    if dense3:
        w = code.reshape(code.shape[:-1] + (code.shape[-1] // 3, 3)).to(torch.int64) & 0xFFFFFFFF
        w0, w1, w2 = w[..., 0], w[..., 1], w[..., 2]
        out = torch.empty(w0.shape + (32,), dtype=torch.int32, device=dev)
        for i in range(32):
            lo = 3 * i
            if lo + 3 <= 32:
                v = w0 >> lo
            elif lo < 32:
                v = (w0 >> lo) | (w1 << (32 - lo))
            elif lo + 3 <= 64:
                v = w1 >> (lo - 32)
            elif lo < 64:
                v = (w1 >> (lo - 32)) | (w2 << (64 - lo))
            else:
                v = w2 >> (lo - 64)
            out[..., i] = (v & 7).to(torch.int32)
        return out.reshape(code.shape[:-1] + (code.shape[-1] // 3 * 32,))
    if bits == 3:
        shifts = torch.tensor([3 * i for i in range(10)] + [30], device=dev, dtype=torch.int32)
        masks = torch.tensor([7] * 10 + [3], device=dev, dtype=torch.int32)
    else:
        shifts = torch.arange(0, 32, bits, device=dev, dtype=torch.int32)
        masks = torch.full((32 // bits,), (1 << bits) - 1, device=dev, dtype=torch.int32)
    q = (code.unsqueeze(-1) >> shifts) & masks
    return q.reshape(code.shape[:-1] + (code.shape[-1] * shifts.numel(),))


def dequantize_torch(code, scale, zero, bits, group, dense3=False):
    """fp32 dequantized tensor [..., n] = scale * code + zero (scale, zero per group along the last dimension)."""
    import torch

    q = unpack_codes_torch(code, bits, dense3).to(torch.float32)
    return scale.float().repeat_interleave(group, -1) * q + zero.float().repeat_interleave(group, -1)
