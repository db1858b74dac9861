"""Golden vectors: hand-derived known answers (tests/golden/known_answers.json) and the seeded
fixture tests/golden/hot_path_small.npz (written by tests/golden/make_golden.py from the oracle).
CPU part: the oracle reproduces both.  GPU part (marked gpu): the HIP path reproduces them."""
import json
import os

import numpy as np
import pytest

from helpers import gemv_close, same_bits

HERE = os.path.dirname(os.path.abspath(__file__))
KA = json.load(open(os.path.join(HERE, "golden", "known_answers.json")))
FIX = np.load(os.path.join(HERE, "golden", "hot_path_small.npz"))


def group_input(case):
    g = case["group"]
    x = np.full(g, case["pad"] if case["pad"] is not None else 0.0, np.float32)
    x[: len(case["x"])] = case["x"]
    return x.reshape(1, 1, 1, g)


def test_known_words(oracle):
    for w in KA["words"]:
        got = int(np.ascontiguousarray(oracle.pack_np(np.array(w["codes"]), w["bits"])).view(np.uint32)[0])
        assert got == int(w["word"], 16), w
        assert list(oracle.unpack_np(np.array([int(w["word"], 16)], np.uint32).view(np.int32), w["bits"])) == w["codes"]


def test_known_quantizations(oracle):
    for c in KA["quantize"]:
        code, scale, mn = oracle.quantize_pack_last_dim(group_input(c), c["group"], c["bits"])
        q = oracle.unpack_np(code, c["bits"])[0, 0, 0]
        assert list(q[: len(c["codes"])]) == c["codes"], c
        assert float(scale[0, 0, 0, 0]) == c["scale"] and float(mn[0, 0, 0, 0]) == c["min"]


def test_oracle_reproduces_fixture(oracle):
    for bits, g in ((4, 32), (2, 32), (1, 32), (3, 11)):
        t = f"b{bits}"
        got = oracle.quantize_pack_last_dim(FIX[f"{t}_kin"], g, bits)
        for a, name in zip(got, ("kcode", "kscale", "kmin")):
            assert same_bits(a, FIX[f"{t}_{name}"]), (t, name)
        assert same_bits(oracle.quantized_gemm(g, FIX[f"{t}_q"], *got, bits), FIX[f"{t}_qk"])
        if bits != 3:
            got = oracle.quantize_pack_last_dim(FIX[f"{t}_vin"], g, bits)
            for a, name in zip(got, ("vcode", "vscale", "vmin")):
                assert same_bits(a, FIX[f"{t}_{name}"]), (t, name)
            assert same_bits(oracle.quantized_gemm(g, FIX[f"{t}_p"], *got, bits), FIX[f"{t}_pv"])
    got = oracle.quantize_pack_dense3(FIX["d3_vin"], 32)
    for a, name in zip(got, ("vcode", "vscale", "vmin")):
        assert same_bits(a, FIX[f"d3_{name}"])


@pytest.mark.gpu
def test_gpu_reproduces_known_answers_and_fixture(oracle, dev):
    import torch

    import KVmix
    from kvmix_amd import ops

    tt = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    for c in KA["quantize"]:
        code, scale, mn = KVmix.quantize_pack_last_dim_cuda(tt(group_input(c)), c["group"], c["bits"])
        q = oracle.unpack_np(code.cpu().numpy(), c["bits"])[0, 0, 0]
        assert list(q[: len(c["codes"])]) == c["codes"], c
        assert float(scale[0, 0, 0, 0]) == c["scale"] and float(mn[0, 0, 0, 0]) == c["min"]
    for w in KA["words"]:  # a word of known codes, scale 1, zero 0, x = e_0 -> the codes come back
        bits = w["bits"]
        g = 11 if bits == 3 else 32
        vpw = len(w["codes"])
        N = vpw if bits == 3 else 32
        words = np.full((1, 1, 1, N // vpw), int(w["word"], 16), np.uint32).view(np.int32)
        one = np.ones((1, 1, 1, N // g), np.float16)
        out = KVmix.quantized_gemm(g, tt(np.ones((1, 1, 1, 1), np.float16)), tt(words), tt(one), tt(one * 0), bits)
        assert list(out.cpu().numpy()[0, 0, 0, :vpw].astype(int)) == w["codes"], w
    for bits, g in ((4, 32), (2, 32), (1, 32), (3, 11)):
        t = f"b{bits}"
        got = KVmix.quantize_pack_last_dim_cuda(tt(FIX[f"{t}_kin"]), g, bits)
        for a, name in zip(got, ("kcode", "kscale", "kmin")):
            assert same_bits(a.cpu().numpy(), FIX[f"{t}_{name}"]), (t, name)
        out = KVmix.quantized_gemm(g, tt(FIX[f"{t}_q"]), *got, bits).cpu().numpy()
        _, w64, a64 = oracle.quantized_gemm(g, FIX[f"{t}_q"], FIX[f"{t}_kcode"], FIX[f"{t}_kscale"], FIX[f"{t}_kmin"],
                                            bits, want_f64=True)
        assert gemv_close(out, w64, a64)[0] and gemv_close(out, FIX[f"{t}_qk"].astype(np.float64), a64)[0]
        if bits != 3:
            got = KVmix.quantize_pack_last_dim_cuda(tt(FIX[f"{t}_vin"]), g, bits)
            for a, name in zip(got, ("vcode", "vscale", "vmin")):
                assert same_bits(a.cpu().numpy(), FIX[f"{t}_{name}"]), (t, name)
            out = KVmix.quantized_gemm(g, tt(FIX[f"{t}_p"]), *got, bits).cpu().numpy()
            _, w64, a64 = oracle.quantized_gemm(g, FIX[f"{t}_p"], FIX[f"{t}_vcode"], FIX[f"{t}_vscale"],
                                                FIX[f"{t}_vmin"], bits, want_f64=True)
            assert gemv_close(out, w64, a64)[0] and gemv_close(out, FIX[f"{t}_pv"].astype(np.float64), a64)[0]
    got = ops.quantize_pack_dense3(tt(FIX["d3_vin"]), 32)
    for a, name in zip(got, ("vcode", "vscale", "vmin")):
        assert same_bits(a.cpu().numpy(), FIX[f"d3_{name}"])
