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


@pytest.mark.parametrize("seed", [11, 22])
def test_random_attention_steps(dev, seed):
    """Seeded random configurations of the library's attention step against its composition from
    quantized_gemm and torch's matmul / softmax: bit widths, head grouping, head dimension,
    quantized lengths that differ between keys and values, tail lengths down to zero, padding masks,
    exact-size tails and fixed windows with device-side lengths."""
    import torch

    from kvmix_amd import ops
    from kvmix_amd.attention import KVmixAttention

    rng = np.random.default_rng(seed)
    gen = torch.Generator(device=dev).manual_seed(seed)
    for case in range(16):
        B = int(rng.choice([1, 2, 3]))
        nkv = int(rng.choice([1, 2, 4]))
        rep = int(rng.choice([1, 2, 4]))
        nh = nkv * rep
        D = int(rng.choice([64, 128, 128, 256]))
        k_bits = int(rng.choice([1, 2, 3, 4]))
        v_bits = int(rng.choice([1, 2, 4]))
        kg = 11 if k_bits == 3 else 32
        n = int(rng.integers(40, 1500))                      # positions
        tk = (int(rng.integers(0, n + 1)) // kg) * kg        # quantized key tokens
        tv = (int(rng.integers(0, n + 1)) // 32) * 32        # quantized value tokens
        lk, lv = n - tk, n - tv
        print("case", seed, case, dict(B=B, nh=nh, nkv=nkv, D=D, k_bits=k_bits, v_bits=v_bits, n=n, tk=tk, tv=tv), flush=True)

        def rnd_i32(*shape):
            return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int64, device=dev, generator=gen).to(torch.int32)

        def rnd_f16(*shape, scale=1.0):
            return (torch.randn(*shape, device=dev, generator=gen) * scale).half()

        kw = tk // 11 if k_bits == 3 else tk * k_bits // 32
        kq = (rnd_i32(B, nkv, D, kw), rnd_f16(B, nkv, D, tk // kg, scale=0.05).abs(), rnd_f16(B, nkv, D, tk // kg, scale=0.3)) if tk else None
        vq = (rnd_i32(B, nkv, tv, D * v_bits // 32), rnd_f16(B, nkv, tv, D // 32, scale=0.2).abs(), rnd_f16(B, nkv, tv, D // 32)) if tv else None
        k_tail, v_tail = rnd_f16(B, nkv, lk, D), rnd_f16(B, nkv, lv, D)
        q = rnd_f16(B, nh, 1, D)
        mask = None
        if rng.random() < 0.5:
            mask = torch.zeros(B, 1, 1, n, device=dev)
            mask[B - 1, :, :, :int(rng.integers(1, n // 2))] = torch.finfo(torch.float32).min
        out, p = ops.decode_attention(q, kq, vq, k_tail, v_tail, kg, k_bits, 32, v_bits, attention_mask=mask)
        att = KVmixAttention(k_bits, v_bits)
        kc, ks, km = kq if kq else (None, None, None)
        vc, vs, vm = vq if vq else (None, None, None)
        out_t, p_t = att._decode_with_torch_glue(q, kc, ks, km, k_tail, vc, vs, vm, v_tail, kg, 0, 0, rep, mask)
        torch.testing.assert_close(p, p_t, rtol=5e-3, atol=2e-5)
        torch.testing.assert_close(out, out_t, rtol=5e-3, atol=1e-2)
        # the same step with tails held in longer windows whose lengths come from device memory
        R = max(lk, lv) + int(rng.integers(0, 40))
        kwin = torch.full((B, nkv, R, D), 99.0, dtype=torch.float16, device=dev)
        vwin = torch.full((B, nkv, R, D), -99.0, dtype=torch.float16, device=dev)
        kwin[:, :, :lk], vwin[:, :, :lv] = k_tail, v_tail
        if mask is None:
            klen = torch.tensor([lk], dtype=torch.int64, device=dev)
            vlen = torch.tensor([lv], dtype=torch.int64, device=dev)
            out_w, p_w = ops.decode_attention(q, kq, vq, kwin, vwin, kg, k_bits, 32, v_bits, k_tail_len=klen, v_tail_len=vlen)
            assert torch.equal(out_w, out) and torch.equal(p_w[..., :n], p)
            assert p_w.shape[-1] == max(tk, tv) + R and float(p_w[..., n:].abs().max() if p_w.shape[-1] > n else 0.0) == 0.0
