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
