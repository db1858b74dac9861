"""Writes tests/golden/*.npz: small seeded inputs with the outputs of the CPU oracle, plus
hand-derived known answers (tests/golden/known_answers.json is written by hand, not by this
script).  The reference holds no golden vectors for this path and its CUDA code cannot run
here, so these fixtures pin the ORACLE's behaviour against accidental change and give the GPU
tests fixed vectors; the facts that pin the oracle itself are the closed forms in
tests/test_oracle_*.py.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import kvmix_oracle as O  # noqa: E402


def kv(rng, shape):
    x = rng.standard_normal(shape).astype(np.float32)
    x[..., rng.permutation(shape[-1])[:2]] *= 10
    return x.astype(np.float16)


def main():
    rng = np.random.default_rng(20240601)
    out = {}
    B, Hkv, H, D = 1, 2, 4, 128
    for bits, g in ((4, 32), (2, 32), (1, 32), (3, 11)):
        T = 8 * g if bits != 3 else 11 * 24
        K = kv(rng, (B, Hkv, T, D))
        V = kv(rng, (B, Hkv, T, D))
        kin = np.ascontiguousarray(K.transpose(0, 1, 3, 2))
        kc, ks, km = O.quantize_pack_last_dim(kin, g, bits)
        q = rng.standard_normal((B, H, 1, D)).astype(np.float16)
        att = O.quantized_gemm(g, q, kc, ks, km, bits)
        tag = f"b{bits}"
        out.update({f"{tag}_kin": kin, f"{tag}_kcode": kc, f"{tag}_kscale": ks, f"{tag}_kmin": km,
                    f"{tag}_q": q, f"{tag}_qk": att})
        if bits != 3:
            vc, vs, vm = O.quantize_pack_last_dim(V, g, bits)
            p = rng.random((B, H, 1, T)).astype(np.float16)
            pv = O.quantized_gemm(g, p, vc, vs, vm, bits)
            out.update({f"{tag}_vin": V, f"{tag}_vcode": vc, f"{tag}_vscale": vs, f"{tag}_vmin": vm,
                        f"{tag}_p": p, f"{tag}_pv": pv})
    # dense 3-bit extension
    V = kv(rng, (B, Hkv, 96, D))
    vc, vs, vm = O.quantize_pack_dense3(V, 32)
    p = rng.random((B, H, 1, 96)).astype(np.float16)
    out.update({"d3_vin": V, "d3_vcode": vc, "d3_vscale": vs, "d3_vmin": vm, "d3_p": p,
                "d3_pv": O.quantized_gemm_dense3(32, p, vc, vs, vm)})
    np.savez_compressed(os.path.join(HERE, "hot_path_small.npz"), **out)
    print("wrote", os.path.join(HERE, "hot_path_small.npz"), sum(v.nbytes for v in out.values()), "bytes raw")


if __name__ == "__main__":
    main()
