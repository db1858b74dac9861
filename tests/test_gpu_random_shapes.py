"""Seeded random shapes through quantized_gemm against the CPU oracle: every kernel family is hit
with shapes nobody picked by hand (tile and chunk remainders, head-group counts, M > 1)."""
import numpy as np
import pytest

from test_gpu_gemv import run_case

pytestmark = pytest.mark.gpu


def _cases(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        bits = int(rng.choice([1, 2, 3, 4]))
        g = 11 if bits == 3 else 32
        nkv = int(rng.choice([1, 2, 3]))
        rep = int(rng.choice([1, 1, 2, 4, 8]))
        B = int(rng.choice([1, 2]))
        M = int(rng.choice([1, 1, 1, 2]))
        if rng.random() < 0.5:   # q.K^T-like: few rows, many columns
            K = int(rng.choice([16, 32, 48, 64, 96, 128, 160]))
            N = g * int(rng.integers(1, 120))
        else:                    # p.V-like: many rows, head_dim columns
            K = int(rng.integers(1, 1500))
            N = 128 if bits != 3 else 11 * int(rng.integers(1, 30))
            if bits != 3 and rng.random() < 0.2:
                N = int(rng.choice([64, 256]))
        out.append((bits, g, B, nkv * rep, nkv, K, N, M))
    return out


@pytest.mark.parametrize("seed", [101, 202, 303])
def test_random_shapes(oracle, dev, seed):
    for i, (bits, g, B, nh, nkv, K, N, M) in enumerate(_cases(seed, 24)):
        print("case", seed, i, dict(bits=bits, g=g, B=B, nh=nh, nkv=nkv, K=K, N=N, M=M), flush=True)
        run_case(oracle, dev, bits, g, B=B, nh=nh, nkv=nkv, K=K, N=N, seed=seed * 100 + i, M=M)
