#!/usr/bin/env python3
"""Benchmark of the KVmix KV-cache hot path on one MI355X.

Workload (BASELINE.json configs[1]): full 32-layer Llama-2-7B KV shape (32 heads x 128, MHA),
batch 8, 8192 tokens of context, mixed per-layer bits from a seeded vector (8 layers 4-bit,
16 layers 3-bit, 8 layers 2-bit; keys and values drawn independently), group 32, 128-token fp16
residual window.  One "step" = for every layer: quantize-and-pack one flush of the residual window
(keys and values) + the fused dequant-GEMV pair q.K^T and p.V over the packed cache.

3-bit keys use the reference's 11-codes-per-word layout (group 11, 8063 quantized tokens, the flush
is 121 tokens); 3-bit values have no working reference form and use the dense 3-bit extension.

Prints one JSON line.  `value` = algorithmic HBM bytes of a step / step time, inputs resident in
HBM.  `roofline` describes the kernel that takes the most time in the step, timed with events on
the launch stream.  `cpu_baseline` times the CPU oracle on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published


def device_kernel(_lib, tag, B, H, D, Tq):
    """the device kernel behind a tag of the step (the name the rocprofv3 summaries list), from the
    library's own dispatch query"""
    fmts = {"b4": (4, _lib.FMT_REF, 32), "b2": (2, _lib.FMT_REF, 32), "b1": (1, _lib.FMT_REF, 32),
            "ref3": (3, _lib.FMT_REF, 11), "dense3": (3, _lib.FMT_DENSE3, 32)}
    try:
        side, f = tag.rstrip("]").split("[")
        bits, fmt, group = fmts[f]
        n = Tq // group * group
        plan = _lib.gemv_plan(group, bits, fmt, B * H, 1, 1, D, n) if side == "gemv_cols" else \
            _lib.gemv_plan(group, bits, fmt, B * H, 1, 1, n, D)
        return "kvmix::" + plan["kernel"]
    except (KeyError, ValueError):
        return ""


def layer_bits(num_layers: int = 32, seed: int = 1):
    rng = np.random.default_rng(seed)
    base = np.array([4] * (num_layers // 4) + [3] * (num_layers // 2) + [2] * (num_layers // 4))
    kb = rng.permutation(base)
    vb = rng.permutation(base)
    return [int(b) for b in kb], [int(b) for b in vb]


def bytes_per_token(bits: int, fmt: str, D: int = 128) -> float:
    """Stored bytes per (batch, kv-head) per quantized token: codes + fp16 scale + fp16 zero."""
    if fmt == "ref3":
        return D * 4 / 11 * 2          # one word and one (scale, zero) pair per 11 tokens, per channel
    if fmt == "dense3":
        return D * 3 / 8 + 4 * (D // 32)
    return D * bits / 8 + 4 * (D // 32)


class Layer:
    pass


def synth_kv(torch, B, H, T, D, dev, gen):
    x = torch.randn(B, H, T, D, device=dev, dtype=torch.float16, generator=gen)
    ch = torch.stack([torch.randperm(D, device=dev, generator=gen)[:4] for _ in range(H)])  # [H,4]
    idx = ch[None, :, None, :].expand(B, H, T, 4)
    x.scatter_(3, idx, x.gather(3, idx) * 10)
    return x


def build_layers(torch, ops, lib, B, H, D, T, R, kbits, vbits, dev):
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    layers = []
    for kb, vb in zip(kbits, vbits):
        L = Layer()
        L.kb, L.vb = kb, vb
        L.kfmt = "ref3" if kb == 3 else f"b{kb}"
        L.vfmt = "dense3" if vb == 3 else f"b{vb}"
        L.kg = 11 if kb == 3 else 32
        L.Tqk = ((T - R) // L.kg) * L.kg  # ref3: 8063 = 11 * 733 for T=8192, R=128 (tail 129)
        L.Tqv = ((T - R) // 32) * 32
        L.nk = (R // L.kg) * L.kg         # tokens per key flush (128, or 121 for ref3)
        L.nv = (R // 32) * 32
        K = synth_kv(torch, B, H, T, D, dev, gen)
        kin = K[:, :, :L.Tqk].transpose(2, 3).contiguous()
        L.kc, L.ks, L.kz = ops.quantize_pack_last_dim_cuda(kin, L.kg, kb)
        L.ktail = K[:, :, L.Tqk:L.Tqk + L.nk].contiguous()  # token-major chunk to flush
        del K, kin
        V = synth_kv(torch, B, H, T, D, dev, gen)
        vin = V[:, :, :L.Tqv].contiguous()
        if vb == 3:
            L.vc, L.vs, L.vz = ops.quantize_pack_dense3(vin, 32)
        else:
            L.vc, L.vs, L.vz = ops.quantize_pack_last_dim_cuda(vin, 32, vb)
        L.vtail = V[:, :, L.Tqv:L.Tqv + L.nv].contiguous()
        del V, vin
        L.q = torch.randn(B, H, 1, D, device=dev, dtype=torch.float16, generator=gen)
        # Scratch of the attention step -- logits out, probabilities in, output -- is one buffer each for all layers,
        # as in a decode loop, whose allocator hands the same blocks to every layer (the logits of a layer are
        # consumed before the next layer runs, the probabilities have just been written by its softmax).  Measured
        # against a buffer set per layer: 2.195 / 2.171 ms (shared outputs / also the probabilities) against 2.229 ms.
        # The packed caches, the flush sources and the flush targets are per layer.
        if not layers:
            shared = Layer()
            shared.p = torch.softmax(torch.randn(B, H, 1, ((T - R) // 32) * 32, device=dev, generator=gen), -1).half()
            shared.logits = torch.empty(B * H * (T - R), device=dev, dtype=torch.float16)
            shared.out = torch.empty(B, H, 1, D, device=dev, dtype=torch.float16)
        L.p = shared.p
        L.logits = shared.logits[:B * H * L.Tqk].view(B, H, 1, L.Tqk)
        L.out = shared.out
        kw = L.nk // 11 if kb == 3 else L.nk * kb // 32
        L.fk_code = torch.empty(B, H, D, kw, device=dev, dtype=torch.int32)
        L.fk_s = torch.empty(B, H, D, L.nk // L.kg, device=dev, dtype=torch.float16)
        L.fk_z = torch.empty_like(L.fk_s)
        vw = D * 3 // 32 if vb == 3 else D * vb // 32
        L.fv_code = torch.empty(B, H, L.nv, vw, device=dev, dtype=torch.int32)
        L.fv_s = torch.empty(B, H, L.nv, D // 32, device=dev, dtype=torch.float16)
        L.fv_z = torch.empty_like(L.fv_s)
        wsb = lib.kvmix_gemv_workspace_bytes(B * H, 1, L.Tqv, D)
        L.ws = torch.empty(max(wsb, 16), device=dev, dtype=torch.uint8)
        L.wsb = wsb
        # algorithmic bytes
        L.bytes_qk = B * H * L.Tqk * bytes_per_token(kb, "ref3" if kb == 3 else "")
        L.bytes_pv = B * H * L.Tqv * bytes_per_token(vb, "dense3" if vb == 3 else "")
        L.bytes_fk = B * H * L.nk * (2 * D + bytes_per_token(kb, "ref3" if kb == 3 else ""))
        L.bytes_fv = B * H * L.nv * (2 * D + bytes_per_token(vb, "dense3" if vb == 3 else ""))
        layers.append(L)
    return layers


def make_calls(torch, _lib, lib, layers, B, H, D, stream):
    """Pre-bound C-ABI calls, one list entry per kernel launch group: (tag, bytes, fn)."""
    calls = []
    for L in layers:
        kfmt = _lib.FMT_REF
        vfmt = _lib.FMT_DENSE3 if L.vb == 3 else _lib.FMT_REF

        # both flushes of the layer in one launch (kvmix_quant_pack_kv_flush)
        L.kflush = _lib.KeyFlush(L.ktail.data_ptr(), B * H, L.nk, D, L.ktail.stride(1), L.ktail.stride(2), L.kg, L.kb,
                                 kfmt, _lib.SCALE_RECIPROCAL, L.fk_code.data_ptr(), L.fk_code.stride(1),
                                 L.fk_code.stride(2), L.fk_s.data_ptr(), L.fk_z.data_ptr(), L.fk_s.stride(1),
                                 L.fk_s.stride(2))
        L.vflush = _lib.ValueFlush(L.vtail.data_ptr(), B * H, L.nv, D, L.vtail.stride(1), L.vtail.stride(2), 32, L.vb,
                                   vfmt, _lib.SCALE_RECIPROCAL, L.fv_code.data_ptr(), L.fv_code.stride(1),
                                   L.fv_code.stride(2), L.fv_s.data_ptr(), L.fv_z.data_ptr(), L.fv_s.stride(1),
                                   L.fv_s.stride(2))

        def qk(L=L):
            return lib.kvmix_quantized_gemv(
                L.kg, L.q.data_ptr(), D, D, L.kc.data_ptr(), L.kc.stride(1), L.kc.stride(2), L.ks.data_ptr(),
                L.kz.data_ptr(), L.ks.stride(1), L.ks.stride(2), L.kb, kfmt, B * H, 1, 1, D, L.Tqk,
                L.logits.data_ptr(), L.Tqk, L.Tqk, None, 0, stream)

        def pv(L=L, vfmt=vfmt):
            return lib.kvmix_quantized_gemv(
                32, L.p.data_ptr(), L.Tqv, L.Tqv, L.vc.data_ptr(), L.vc.stride(1), L.vc.stride(2), L.vs.data_ptr(),
                L.vz.data_ptr(), L.vs.stride(1), L.vs.stride(2), L.vb, vfmt, B * H, 1, 1, L.Tqv, D,
                L.out.data_ptr(), D, D, L.ws.data_ptr(), L.wsb, stream)

        calls += [(f"gemv_cols[{L.kfmt}]", L.bytes_qk, qk), (f"gemv_rows[{L.vfmt}]", L.bytes_pv, pv)]
    # The flushes of the step, batched: what a layer flushes in a decode step are the oldest tokens of its fp16
    # tails (models/modeling_llama_KVmix.py:122-127,152-156), tokens of earlier steps, so the flushes of all layers
    # go out before the first layer runs -- kvmix_quant_pack_kv_flush_batch, eight layers to a launch.
    flushes = []
    for i in range(0, len(layers), 8):
        part = layers[i:i + 8]
        ka = (ctypes.POINTER(_lib.KeyFlush) * len(part))(*[ctypes.pointer(L.kflush) for L in part])
        va = (ctypes.POINTER(_lib.ValueFlush) * len(part))(*[ctypes.pointer(L.vflush) for L in part])

        def fl(ka=ka, va=va, n=len(part)):
            return lib.kvmix_quant_pack_kv_flush_batch(ka, va, n, stream)

        flushes.append((f"quant_kv_flush_batch[{len(part)} layers]", sum(L.bytes_fk + L.bytes_fv for L in part), fl))
    return flushes + calls


def run_step(calls):
    for _, _, fn in calls:
        rc = fn()
        if rc != 0:
            raise RuntimeError(f"kvmix call failed: {rc}")


def time_kernels(torch, calls, reps=10):
    """Per kernel kind: average duration of one launch (events on the launch stream), over the
    step's own launches (each on its own layer's buffers, so nothing is served from cache)."""
    kinds = {}
    for tag, nbytes, fn in calls:
        kinds.setdefault(tag, []).append((nbytes, fn))
    out = {}
    for tag, lst in kinds.items():
        for _, fn in lst:
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            for _, fn in lst:
                fn()
        e.record()
        torch.cuda.synchronize()
        n = reps * len(lst)
        out[tag] = {"launches_per_step": len(lst), "avg_us": s.elapsed_time(e) * 1e3 / n,
                    "bytes_per_launch": float(np.mean([b for b, _ in lst]))}
    return out


def cpu_baseline(layers, kbits, vbits, B, H, D, T, R, sample_layers=None, budget_s=20.0):
    """The CPU oracle (scalar C restatement of the reference kernels, OpenMP over rows) on the
    step's own data, layer by layer at full batch (one flush + the GEMV pair each), until about
    `budget_s` seconds of CPU time are spent or the layers run out."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import kvmix_oracle as O

    O.lib()
    rng = np.random.default_rng(0)
    total_bytes, total_t = 0.0, 0.0
    done = 0
    for li in range(len(layers) if sample_layers is None else sample_layers):
        if total_t > budget_s:
            break
        done += 1
        L = layers[li]
        kc = L.kc.cpu().numpy()
        ks, kz = L.ks.cpu().numpy(), L.kz.cpu().numpy()
        vc = L.vc.cpu().numpy()
        vs, vz = L.vs.cpu().numpy(), L.vz.cpu().numpy()
        q = L.q.cpu().numpy()
        p = L.p.cpu().numpy()
        ktail = np.ascontiguousarray(L.ktail.cpu().numpy().transpose(0, 1, 3, 2))
        vtail = L.vtail.cpu().numpy()
        t0 = time.perf_counter()
        O.quantize_pack_last_dim(ktail, L.kg, L.kb)
        if L.vb == 3:
            O.quantize_pack_dense3(vtail, 32)
        else:
            O.quantize_pack_last_dim(vtail, 32, L.vb)
        O.quantized_gemm(L.kg, q, kc, ks, kz, L.kb, mode=O.GEMM_SEQUENTIAL)
        if L.vb == 3:
            O.quantized_gemm_dense3(32, p, vc, vs, vz)
        else:
            O.quantized_gemm(32, p, vc, vs, vz, L.vb, mode=O.GEMM_SEQUENTIAL)
        total_t += time.perf_counter() - t0
        total_bytes += L.bytes_qk + L.bytes_pv + L.bytes_fk + L.bytes_fv
    res = {"value": round(total_bytes / total_t / 1e9, 3), "unit": "GB/s", "cores": int(O.num_threads()),
           "kind": "port",
           "sample": f"layers 0..{done - 1} of the step at full batch (one flush + q.K^T + p.V each, "
                     f"{total_bytes / 1e9:.2f} GB algorithmic), {total_t:.1f} s of CPU time, "
                     f"C oracle with OpenMP on {int(O.num_threads())} threads"}
    try:
        res["torch_cpu"] = torch_cpu_baseline(layers, int(O.num_threads()))
    except Exception as ex:  # (the C port above is the figure of record; this leg must not take it down)
        res["torch_cpu"] = {"error": f"{type(ex).__name__}: {ex}"}
    return res


def torch_cpu_baseline(layers, threads, batch_slice=2, reps=5, warm=2):
    """The same work as vectorised PyTorch on the CPU: quantize = fp32 min / max / scale / round-half-away / pack
    with tensor ops, GEMV = unpack with shifts and masks, dequantize to fp32, torch.matmul
    (quant_cuda/csrc/quantization_cuda.cu:540-721, dequantization_gemv_cuda.cu:7-124 restated on tensors).  One layer
    of each reference-layout bit width present in the step (2/2 and 4/4 bits), the first `batch_slice` batch entries
    of it, `reps` repetitions after `warm` warm-ups, all host threads."""
    import torch

    torch.set_num_threads(threads)

    def unpack(code, bits):
        shifts = torch.arange(0, 32, bits, dtype=torch.int32)
        return ((code.unsqueeze(-1) >> shifts) & ((1 << bits) - 1)).flatten(-2)

    def dequant(code, scale, zero, bits, g=32):
        return unpack(code, bits).float() * scale.float().repeat_interleave(g, -1) + zero.float().repeat_interleave(g, -1)

    def quantize(x, bits, g=32):
        qmax = (1 << bits) - 1
        xf = x.float().unflatten(-1, (-1, g))
        mn, mx = xf.amin(-1, keepdim=True), xf.amax(-1, keepdim=True)
        scale = (mx - mn) / qmax
        q = torch.nan_to_num(torch.floor((xf - mn) / scale + 0.5), nan=0.0).clamp_(0, qmax).to(torch.int32).flatten(-2)
        shifts = torch.arange(0, 32, bits, dtype=torch.int32)
        words = (q.unflatten(-1, (-1, 32 // bits)) << shifts).sum(-1, dtype=torch.int32)
        return words, ((mx - mn) * (1.0 / qmax)).half().squeeze(-1), mn.half().squeeze(-1)

    out = {}
    total_bytes = total_t = 0.0
    for L in layers:
        if (L.kb, L.vb) not in ((2, 2), (4, 4)) or f"k{L.kb}v{L.vb}" in out:
            continue
        n = min(batch_slice, L.q.shape[0])
        frac = n / L.q.shape[0]
        kc, ks, kz = (t[:n].cpu() for t in (L.kc, L.ks, L.kz))
        vc, vs, vz = (t[:n].cpu() for t in (L.vc, L.vs, L.vz))
        q, p = L.q[:n].cpu().float(), L.p[:n].cpu().float()
        ktail, vtail = L.ktail[:n].cpu().transpose(2, 3).contiguous(), L.vtail[:n].cpu()

        def step():
            quantize(ktail, L.kb)
            quantize(vtail, L.vb)
            a = torch.matmul(q, dequant(kc, ks, kz, L.kb)).half()
            b = torch.matmul(p, dequant(vc, vs, vz, L.vb)).half()
            return a, b

        for _ in range(warm):
            step()
        t0 = time.perf_counter()
        for _ in range(reps):
            step()
        dt = (time.perf_counter() - t0) / reps
        nbytes = (L.bytes_qk + L.bytes_pv + L.bytes_fk + L.bytes_fv) * frac
        out[f"k{L.kb}v{L.vb}"] = {"ms": round(dt * 1e3, 1), "GBps": round(nbytes / dt / 1e9, 3)}
        total_bytes += nbytes
        total_t += dt
    out["value"] = round(total_bytes / total_t / 1e9, 3) if total_t else None
    out["unit"], out["cores"] = "GB/s", threads
    out["sample"] = (f"one 2/2-bit and one 4/4-bit layer of the step, first {batch_slice} of its batch entries (flush + q.K^T + p.V), "
                     f"{reps} repetitions after {warm} warm-ups, torch {torch.__version__} on {threads} threads")
    return out


def mha_pair_times(torch, lib, dev, stream, B, Tq, bits, nsets=3, warm=30, iters=100, H=32, D=128):
    """q.K^T and p.V of one MHA shape (B x H slices, Tq quantized tokens, `bits`-bit codes in groups of 32):
    event-timed eager launches over `nsets` buffer sets taken in turn, so that the Infinity Cache cannot
    serve them."""
    sets = []
    for _ in range(nsets):
        kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tq * bits // 32), dtype=torch.int64, device=dev).to(torch.int32)
        ks = torch.rand(B, H, D, Tq // 32, device=dev).half()
        kz = torch.randn(B, H, D, Tq // 32, device=dev).half()
        vc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tq, D * bits // 32), dtype=torch.int64, device=dev).to(torch.int32)
        vs = torch.rand(B, H, Tq, D // 32, device=dev).half()
        vz = torch.randn(B, H, Tq, D // 32, device=dev).half()
        sets.append((kc, ks, kz, vc, vs, vz))
    q = torch.randn(B, H, 1, D, device=dev).half()
    p = torch.softmax(torch.randn(B, H, 1, Tq, device=dev), -1).half()
    lo = torch.empty(B, H, 1, Tq, device=dev, dtype=torch.float16)
    o = torch.empty(B, H, 1, D, device=dev, dtype=torch.float16)
    wsb = lib.kvmix_gemv_workspace_bytes(B * H, 1, Tq, D)
    ws = torch.empty(max(wsb, 16), device=dev, dtype=torch.uint8)

    def qk(i):
        kc, ks, kz = sets[i % nsets][:3]
        return lib.kvmix_quantized_gemv(32, q.data_ptr(), D, D, kc.data_ptr(), kc.stride(1), kc.stride(2), ks.data_ptr(),
                                        kz.data_ptr(), ks.stride(1), ks.stride(2), bits, 0, B * H, 1, 1, D, Tq,
                                        lo.data_ptr(), Tq, Tq, None, 0, stream)

    def pv(i):
        vc, vs, vz = sets[i % nsets][3:]
        return lib.kvmix_quantized_gemv(32, p.data_ptr(), Tq, Tq, vc.data_ptr(), vc.stride(1), vc.stride(2), vs.data_ptr(),
                                        vz.data_ptr(), vs.stride(1), vs.stride(2), bits, 0, B * H, 1, 1, Tq, D,
                                        o.data_ptr(), D, D, ws.data_ptr(), wsb, stream)

    nbytes = B * H * Tq * bytes_per_token(bits, "")
    res = {}
    for name, fn in (("qk", qk), ("pv", pv)):
        for i in range(warm):
            assert fn(i) == 0
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for i in range(iters):
            fn(i)
        e.record()
        torch.cuda.synchronize()
        us = s.elapsed_time(e) * 1e3 / iters
        res[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del sets
    return res


def target_shape_extra(torch, _lib, lib, dev, stream):
    """The shape the target is quoted on: B=16, 32 heads, T=8192 (8064 quantized), 4- and 2-bit."""
    res = {}
    for bits in (4, 2):
        r = mha_pair_times(torch, lib, dev, stream, 16, 8064, bits)  # three buffer sets: ~1 GB at 4 bits
        res[f"qk_{bits}bit"], res[f"pv_{bits}bit"] = r["qk"], r["pv"]
    return res


def length_scan_extra(torch, _lib, lib, dev, stream):
    """The same pair against the number of quantized tokens at B = 8 and 16 (--length-scan): the time that does
    not scale with the bytes (the intercept) and the rate the kernels approach for long rows; with the kernel
    each launch was dispatched to."""
    res = {}
    for B in (8, 16):
        for bits in (4, 2):
            for Tq in (1024, 2048, 4096, 8064, 16128, 32256):
                nbytes = B * 32 * Tq * bytes_per_token(bits, "")
                nsets = int(min(12, max(3, 600e6 // nbytes + 1)))
                r = mha_pair_times(torch, lib, dev, stream, B, Tq, bits, nsets=nsets, warm=2 * nsets, iters=5 * nsets)
                r["qk"]["kernel"] = _lib.gemv_plan(32, bits, 0, B * 32, 1, 1, 128, Tq)["kernel"]
                r["pv"]["kernel"] = _lib.gemv_plan(32, bits, 0, B * 32, 1, 1, Tq, 128)["kernel"]
                res[f"B{B}_{bits}bit_T{Tq}"] = r
                torch.cuda.empty_cache()
    return res


def gqa_shape_extra(torch, _lib, lib, dev, stream):
    """BASELINE configs[2]: GQA 32 query / 8 kv heads, B=16, T=32768, reference 3-bit keys (group 11,
    32637 quantized tokens), 2-bit values (32640).  The bytes are the packed cache's, counted once:
    the four query heads of a kv head are served from one pass (p.V) or from one L2 (q.K^T)."""
    B, H, Hkv, D = 16, 32, 8, 128
    Tk, Tv = 32637, 32640
    sets = []
    for _ in range(2):
        kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, D, Tk // 11), dtype=torch.int64, device=dev).to(torch.int32)
        ks = torch.rand(B, Hkv, D, Tk // 11, device=dev).half()
        kz = torch.randn(B, Hkv, D, Tk // 11, device=dev).half()
        vc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, Hkv, Tv, D * 2 // 32), dtype=torch.int64, device=dev).to(torch.int32)
        vs = torch.rand(B, Hkv, Tv, D // 32, device=dev).half()
        vz = torch.randn(B, Hkv, Tv, D // 32, device=dev).half()
        sets.append((kc, ks, kz, vc, vs, vz))
    q = torch.randn(B, H, 1, D, device=dev).half()
    p = torch.softmax(torch.randn(B, H, 1, Tv, device=dev), -1).half()
    lo = torch.empty(B, H, 1, Tk, device=dev, dtype=torch.float16)
    o = torch.empty(B, H, 1, D, device=dev, dtype=torch.float16)
    wsb = lib.kvmix_gemv_workspace_bytes(B * H, 1, Tv, D)
    ws = torch.empty(max(wsb, 16), device=dev, dtype=torch.uint8)

    def qk(i):
        kc, ks, kz = sets[i % 2][:3]
        return lib.kvmix_quantized_gemv(11, q.data_ptr(), D, D, kc.data_ptr(), kc.stride(1), kc.stride(2), ks.data_ptr(),
                                        kz.data_ptr(), ks.stride(1), ks.stride(2), 3, _lib.FMT_REF, B * H, H // Hkv, 1, D, Tk,
                                        lo.data_ptr(), Tk, Tk, None, 0, stream)

    def pv(i):
        vc, vs, vz = sets[i % 2][3:]
        return lib.kvmix_quantized_gemv(32, p.data_ptr(), Tv, Tv, vc.data_ptr(), vc.stride(1), vc.stride(2), vs.data_ptr(),
                                        vz.data_ptr(), vs.stride(1), vs.stride(2), 2, _lib.FMT_REF, B * H, H // Hkv, 1, Tv, D,
                                        o.data_ptr(), D, D, ws.data_ptr(), wsb, stream)

    res = {}
    for name, fn, nbytes in (("qk_ref3", qk, B * Hkv * Tk * bytes_per_token(3, "ref3")),
                             ("pv_2bit", pv, B * Hkv * Tv * bytes_per_token(2, ""))):
        for i in range(20):  # warm-up: 20 launches, then 100 timed ones
            assert fn(i) == 0
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for i in range(100):
            fn(i)
        e.record()
        torch.cuda.synchronize()
        us = s.elapsed_time(e) * 1e3 / 100
        res[name] = {"us": round(us, 2), "packed_MB": round(nbytes / 1e6, 1), "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    return res


def sweep_extra(torch, _lib, lib, dev, stream):
    """BASELINE configs[3]: MHA 32 x 128, T=4096 with a 32-token fp16 window (4064 quantized tokens),
    1- and 2-bit keys and values, batch 1 / 16 / 64 / 128.  Each entry is one q.K^T or p.V launch;
    enough buffer sets are rotated that no set is still in the 256 MB Infinity Cache when reused."""
    H, D, Tq = 32, 128, 4064
    res = {}
    side = torch.cuda.Stream()
    stream = side.cuda_stream
    for bits in (1, 2):
        for B in (1, 16, 64, 128):
            nbytes = B * H * Tq * bytes_per_token(bits, "")
            nsets = int(min(64, max(2, -(-(600 << 20) // int(nbytes)))))
            sets = []
            for _ in range(nsets):
                kc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, Tq * bits // 32), dtype=torch.int64, device=dev).to(torch.int32)
                ks = torch.rand(B, H, D, Tq // 32, device=dev).half()
                kz = torch.randn(B, H, D, Tq // 32, device=dev).half()
                vc = torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, Tq, D * bits // 32), dtype=torch.int64, device=dev).to(torch.int32)
                vs = torch.rand(B, H, Tq, D // 32, device=dev).half()
                vz = torch.randn(B, H, Tq, D // 32, device=dev).half()
                sets.append((kc, ks, kz, vc, vs, vz))
            q = torch.randn(B, H, 1, D, device=dev).half()
            p = torch.softmax(torch.randn(B, H, 1, Tq, device=dev), -1).half()
            lo = torch.empty(B, H, 1, Tq, device=dev, dtype=torch.float16)
            o = torch.empty(B, H, 1, D, device=dev, dtype=torch.float16)
            wsb = lib.kvmix_gemv_workspace_bytes(B * H, 1, Tq, D)
            ws = torch.empty(max(wsb, 16), device=dev, dtype=torch.uint8)

            def qk(i):
                kc, ks, kz = sets[i % nsets][:3]
                return lib.kvmix_quantized_gemv(32, q.data_ptr(), D, D, kc.data_ptr(), kc.stride(1), kc.stride(2),
                                                ks.data_ptr(), kz.data_ptr(), ks.stride(1), ks.stride(2), bits, 0, B * H, 1,
                                                1, D, Tq, lo.data_ptr(), Tq, Tq, None, 0, stream)

            def pv(i):
                vc, vs, vz = sets[i % nsets][3:]
                return lib.kvmix_quantized_gemv(32, p.data_ptr(), Tq, Tq, vc.data_ptr(), vc.stride(1), vc.stride(2),
                                                vs.data_ptr(), vz.data_ptr(), vs.stride(1), vs.stride(2), bits, 0, B * H, 1,
                                                1, Tq, D, o.data_ptr(), D, D, ws.data_ptr(), wsb, stream)

            iters = max(30, 2 * nsets)
            for name, fn in (("qk", qk), ("pv", pv)):
                torch.cuda.synchronize()  # (the buffers were filled on the default stream)
                for i in range(nsets):
                    assert fn(i) == 0
                torch.cuda.synchronize()
                # the launches are replayed from a HIP graph: at batch 1 a kernel is shorter than the
                # host needs to issue the next call, and the loop would time the host
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(iters):
                        fn(i)
                graph.replay()
                torch.cuda.synchronize()
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                graph.replay()
                e.record()
                torch.cuda.synchronize()
                us = s.elapsed_time(e) * 1e3 / iters
                del graph
                res[f"{name}_{bits}bit_B{B}"] = {"us": round(us, 2), "packed_MB": round(nbytes / 1e6, 1),
                                                 "GBps": round(nbytes / us / 1e3, 1),
                                                 "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            del sets
            torch.cuda.empty_cache()
    return res


def stream_ceiling_extra(torch, _lib, lib, dev):
    """What a kernel that only reads reaches on this GPU (kvmix_probe_stream_read: no arithmetic), in the
    access patterns of the GEMV kernels, over 1 GiB regions of a 4 GiB buffer taken in turn (nothing is
    served from the Infinity Cache).  The GEMV figures are to be read against these, not against 8 TB/s alone:
      slab       contiguous slab per block (the p.V pattern), 1024 blocks of 8 waves, 16 bytes per lane
      rows       512-byte row pieces down 128 rows of a [512][128][4032 B] array (the q.K^T 4-bit pattern)
      rows_side  the same plus the two side arrays read as the scales and zeros are (what a 4-bit q.K^T
                 launch at B=16, T=8192 reads), blocks in XCD-aware order
    each with plain and with non-temporal loads; rows_side also in the kernels' order of issue for three row
    lengths."""
    GiB = 1 << 30
    buf = torch.empty(4 * GiB, dtype=torch.uint8, device=dev)
    buf.view(torch.int64).random_()
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    NT, SIDE_NT, XCD = 1, 2, 4

    def run(pattern, a0, a1, count, waves, bpl, u, flags, nbytes, reps=20):
        regions = (4 * GiB) // nbytes

        def go(i):
            rc = lib.kvmix_probe_stream_read(buf.data_ptr() + (i % regions) * nbytes, pattern, a0, a1, count, waves, bpl, u,
                                             flags, sink.data_ptr(), st)
            if rc != 0:
                raise RuntimeError(_lib.strerror(rc))
        for i in range(5):
            go(i)
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for i in range(reps):
            go(i)
        e.record()
        torch.cuda.synchronize()
        us = s.elapsed_time(e) * 1e3 / reps
        return {"us": round(us, 1), "MB": round(nbytes / 1e6, 1), "GBps": round(nbytes / us / 1e3, 1)}

    res = {}
    slab = (GiB // 1024) // (64 * 16 * 8) * (64 * 16 * 8)
    for name, flags in (("plain", 0), ("nontemporal", NT)):
        res[f"slab_{name}"] = run(0, slab, 0, 1024, 8, 16, 8, flags, slab * 1024)
        res[f"rows_{name}"] = run(1, 128, 4032, 512, 4, 8, 16, flags, 512 * 128 * 4032)
        res[f"rows_side_{name}"] = run(2, 128, 4032, 512, 4, 8, 16, flags | XCD, 512 * 128 * (4032 + 2 * 504))
    # the same bytes with the loads issued in the kernels' rotating order (four rows consumed, four refilled)
    # instead of in bursts, for three row lengths: 4032 bytes is a 4-bit key row at T = 8192, 2016 a 2-bit one,
    # 8064 a 4-bit one at T = 16384 -- the shorter the rows, the lower the ceiling of this pattern
    ROT = 8
    for row, count in ((2016, 1024), (4032, 512), (8064, 256)):
        res[f"rows_side_nontemporal_kernel_order_row{row}"] = run(2, 128, row, count, 4, 8, 16, NT | XCD | ROT,
                                                                 count * 128 * (row + 2 * (row // 8)))
    del buf
    torch.cuda.empty_cache()
    return res


def attention_step_extra(torch, dev, shapes=None):
    """The whole attention step of one layer (logits over packed keys + fp16 tail, softmax, output
    over packed values + fp16 tail) in its two forms: four launches with the reference's roundings,
    and one pass over the positions (two launches).  MHA 32 x 128, 128-token fp16 tails; buffer sets
    are rotated so that they come from HBM; launches replayed from a HIP graph."""
    from kvmix_amd import ops

    H, D, R = 32, 128, 128
    res = {}
    side = torch.cuda.Stream()
    # (3-bit keys: the reference's words of 11 codes; 3-bit values: the dense stream)
    for (B, T, kb, vb) in shapes or [(1, 4096, 4, 4), (4, 2304, 4, 4), (4, 2304, 3, 2), (4, 2304, 2, 2), (8, 8192, 4, 4),
                                     (16, 8192, 4, 4), (8, 8192, 2, 2), (16, 8192, 2, 2), (8, 8192, 3, 2), (16, 8192, 3, 2),
                                     (8, 8192, 2, 4), (16, 8192, 2, 4), (8, 8192, 3, 3), (16, 8192, 3, 3)]:
        kg = 11 if kb == 3 else 32
        vfmt = ops.FMT_DENSE3 if vb == 3 else ops.FMT_REF
        tk, tv = ((T - R) // kg) * kg, ((T - R) // 32) * 32
        kbytes = (1024 / 11 if kb == 3 else 16 * kb + 16) * tk
        nbytes = B * H * (kbytes + (16 * vb + 16) * tv + (2 * T - tk - tv) * 2 * D)
        nsets = int(min(48, max(2, -(-(600 << 20) // int(nbytes)))))
        sets = []
        for _ in range(nsets):
            kw = tk // 11 if kb == 3 else tk * kb // 32
            kq = (torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, D, kw), dtype=torch.int64, device=dev).to(torch.int32),
                  (torch.rand(B, H, D, tk // kg, device=dev) * 0.05).half(), (torch.randn(B, H, D, tk // kg, device=dev) * 0.3).half())
            vq = (torch.randint(-2 ** 31, 2 ** 31 - 1, (B, H, tv, D * vb // 32), dtype=torch.int64, device=dev).to(torch.int32),
                  (torch.rand(B, H, tv, D // 32, device=dev) * 0.2).half(), torch.randn(B, H, tv, D // 32, device=dev).half())
            sets.append((kq, vq, torch.randn(B, H, T - tk, D, device=dev).half(), torch.randn(B, H, T - tv, D, device=dev).half()))
        q = torch.randn(B, H, 1, D, device=dev).half()
        entry = {"packed_plus_tail_MB": round(nbytes / 1e6, 1)}
        for name, single in (("four_launch", False), ("single_pass", True)):
            def fn(i):
                kq, vq, kt, vt = sets[i % nsets]
                return ops.decode_attention(q, kq, vq, kt, vt, kg, kb, 32, vb, v_fmt=vfmt, single_pass=single)
            iters = max(100, 2 * nsets)
            with torch.cuda.stream(side):
                for i in range(max(nsets, 20)):
                    fn(i)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(iters):
                        fn(i)
                graph.replay()
                torch.cuda.synchronize()
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                graph.replay()
                e.record()
                torch.cuda.synchronize()
            us = s.elapsed_time(e) * 1e3 / iters
            del graph
            entry[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1)}
        entry["chosen"] = "single_pass" if ops.prefer_single_pass(B, H, H, D, T, kb, 0, kg, vb, vfmt, 32, k_tokens=tk,
                                                                   v_tokens=tv) else "four_launch"
        res[f"B{B}_T{T}_k{'ref3' if kb == 3 else kb}v{'dense3' if vb == 3 else vb}"] = entry
        del sets
        torch.cuda.empty_cache()
    return res


def e2e_extra(torch, dev, batch=4, prompt_len=2048, new_tokens=512):
    """BASELINE configs[4]: greedy decoding on a random-init Llama-2-7B (fp16 weights ~N(0, 0.02), seed 4),
    prompt of random token ids, mixed per-layer bits as in configs[1], 128-token fp16 window, in-place
    caches.  The host loop is eager PyTorch (projections, RoPE, norms, MLP through torch / hipBLASLt);
    the KV path is the library's.  Tokens/s as the reference's driver counts them
    (Inference-comparision.py:147-151): new tokens and all tokens over the whole wall time; the
    decode-only rate is given beside them."""
    from kvmix_amd.decoder import Decoder, DecoderConfig, GraphDecoder, init_weights, kvmix_layers

    cfg = DecoderConfig()
    kbits, vbits = layer_bits(cfg.num_layers)
    weights = init_weights(cfg, dev)
    gen = torch.Generator(device="cpu").manual_seed(4)

    def run(B, T, new, graph=True):
        atts, caches = kvmix_layers(cfg, kbits, vbits, residual_length=128, capacity=T + new)
        dec = (GraphDecoder if graph else Decoder)(cfg, weights, atts, caches)
        prompt = torch.randint(0, cfg.vocab_size, (B, T), generator=gen).to(dev)
        marks = {}

        def on_step(step, logits):
            if step == 0:
                torch.cuda.synchronize()
                marks["prefill_end"] = time.perf_counter()

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tokens = dec.generate(prompt, new, on_step)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        steps = (dec.graph_steps, dec.eager_steps, dec.captures) if graph else (0, new, 0)
        return tokens, marks["prefill_end"] - t0, t1 - marks["prefill_end"], [c.k_tokens for c in caches], steps

    run(batch, 256, 8)  # warm-up: library heuristics, kernel loading
    _, _, eager_decode_s, _, _ = run(batch, prompt_len, new_tokens, graph=False)
    tokens, prefill_s, decode_s, k_tokens, steps = run(batch, prompt_len, new_tokens)
    total = prefill_s + decode_s
    return {
        "model": "Llama-2-7B shape (32 layers, hidden 4096, 32 heads, ffn 11008, vocab 32000), random init, fp16",
        "batch": batch, "prompt_tokens": prompt_len, "new_tokens": new_tokens, "residual": 128,
        "k_bits": kbits, "v_bits": vbits,
        "prefill_s": round(prefill_s, 3), "decode_s": round(decode_s, 3),
        "decode_ms_per_step": round(decode_s * 1e3 / (new_tokens - 1), 3),
        "new_tokens_per_s": round(batch * new_tokens / total, 1),
        "all_tokens_per_s": round(batch * (prompt_len + new_tokens) / total, 1),
        "decode_only_tokens_per_s": round(batch * (new_tokens - 1) / decode_s, 1),
        "quantized_key_tokens_at_end": [int(min(k_tokens)), int(max(k_tokens))],
        "host_loop": "decode steps replayed from a HIP graph, re-captured after every step that flushes "
                     "(those steps run eagerly); prompt eager",
        "graph_steps": steps[0], "eager_steps": steps[1], "graph_captures": steps[2],
        "eager_host_loop": {"decode_ms_per_step": round(eager_decode_s * 1e3 / (new_tokens - 1), 3),
                            "decode_only_tokens_per_s": round(batch * (new_tokens - 1) / eager_decode_s, 1)},
    }


def hf_generate_extra(torch, dev, batch=4, prompt_len=2048, new_tokens=512):
    """The reference's own harness in small (Inference-comparision.py:89-201): `generate()` of the
    stock model with its fp16 cache against `LlamaForCausalLM_KVmix.generate()` with the packed
    cache, same random-init Llama-2-7B-shaped weights, same prompt; throughput counted over all
    tokens as the reference prints it (:147-151), plus the memory both caches add to the weights."""
    import gc

    from transformers import LlamaConfig, LlamaForCausalLM

    from kvmix_amd.hf import LlamaForCausalLM_KVmix

    cfg = LlamaConfig(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=32, vocab_size=32000, max_position_embeddings=4096)
    cfg._attn_implementation = "eager"
    kbits, vbits = layer_bits(32)
    quant_bits = {i: {"k_bits": kbits[i], "v_bits": vbits[i]} for i in range(32)}
    cfg.residual_length = 128  # the fixed window of BASELINE configs[4] instead of the ratio rule

    def build(cls, **kw):
        with torch.device("meta"):
            m = cls(cfg, **kw)
        m = m.to(torch.float16).to_empty(device=dev)
        g = torch.Generator(device=dev).manual_seed(4)
        with torch.no_grad():
            for name, w in m.named_parameters():
                if w.dim() == 1:
                    w.fill_(1.0)
                else:
                    w.normal_(0.0, 0.02, generator=g)
        m.model.rotary_emb.__init__(config=cfg, device=dev)  # (the inverse frequencies are a buffer, not a parameter)
        return m.eval()

    gen = torch.Generator(device="cpu").manual_seed(4)
    prompt = torch.randint(0, cfg.vocab_size, (batch, prompt_len), generator=gen).to(dev)
    mask = torch.ones_like(prompt)
    res = {"model": "Llama-2-7B shape, random init, fp16, transformers generate(), eager attention",
           "batch": batch, "prompt_tokens": prompt_len, "new_tokens": new_tokens}
    for name, cls, kw in (("stock_fp16_cache", LlamaForCausalLM, {}), ("kvmix_packed_cache", LlamaForCausalLM_KVmix, {"quant_bits": quant_bits})):
        model = build(cls, **kw)
        model.generate(prompt[:1, :64], attention_mask=mask[:1, :64], max_new_tokens=8, do_sample=False, pad_token_id=0)  # warm-up
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats(dev)
        before = torch.cuda.memory_allocated(dev)
        t0 = time.perf_counter()
        out = model.generate(prompt, attention_mask=mask, max_new_tokens=new_tokens, min_new_tokens=new_tokens, do_sample=False,
                             pad_token_id=0)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        res[name] = {"wall_s": round(wall, 3), "all_tokens_per_s": round(out.numel() / wall, 1),
                     "new_tokens_per_s": round(batch * new_tokens / wall, 1),
                     "peak_memory_above_weights_MB": round((torch.cuda.max_memory_allocated(dev) - before) / 2 ** 20, 1)}
        # what the cache itself holds for this context: one more prompt forward, cache kept alive
        cache = model.new_cache(prompt_len + 1) if hasattr(model, "new_cache") else None
        torch.cuda.empty_cache()
        base = torch.cuda.memory_allocated(dev)
        with torch.no_grad():
            o = model(prompt, attention_mask=mask, past_key_values=cache, use_cache=True, logits_to_keep=1)
        cache = o.past_key_values
        del o
        torch.cuda.synchronize()
        res[name]["cache_MB_after_prompt"] = round((torch.cuda.memory_allocated(dev) - base) / 2 ** 20, 1)
        del model, out, cache
        gc.collect()
        torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-target-shape", action="store_true")
    ap.add_argument("--no-sweep", action="store_true", help="skip the batch sweep of BASELINE configs[3]")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end Llama-2-7B-shape decode loop")
    ap.add_argument("--e2e-only", action="store_true", help="run only the end-to-end decode loop")
    ap.add_argument("--hf-batch", type=int, default=4)
    ap.add_argument("--hf-new-tokens", type=int, default=512)
    ap.add_argument("--hf-prompt", type=int, default=2048)
    ap.add_argument("--hf-only", action="store_true",
                    help="run only the transformers generate() comparison (stock fp16 cache against the KVmix wrappers)")
    ap.add_argument("--no-attention-step", action="store_true", help="skip the attention-step comparison")
    ap.add_argument("--attention-step-only", action="store_true", help="run only the attention-step comparison")
    ap.add_argument("--shapes-only", action="store_true",
                    help="skip the step: only the B=16/T=8192 target shape and the GQA configuration (for profiling)")
    ap.add_argument("--stream-ceiling", action="store_true",
                    help="run only the streaming-read probe (what a kernel without arithmetic reaches)")
    ap.add_argument("--no-stream-ceiling", action="store_true", help="skip the streaming-read probe")
    ap.add_argument("--length-scan", action="store_true",
                    help="only q.K^T / p.V at B = 8 and 16 against the number of quantized tokens (1k .. 32k)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run plain 1 GiB device copies (a known-size kernel to scale HBM counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only. Every (batch, kv-head) slice is independent, so the path "
              "shards over batch or kv heads without any exchange; no multi-GPU figure is produced. "
              "Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from kvmix_amd import _lib, ops

    lib = _lib.load()  # fails loudly if the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, H, D, T, R = args.batch, 32, 128, args.context, 128
    if args.length_scan:
        print(json.dumps({"length_scan": length_scan_extra(torch, _lib, lib, dev, torch.cuda.current_stream().cuda_stream)}))
        return
    if args.stream_ceiling:
        res = stream_ceiling_extra(torch, _lib, lib, dev)
        print(json.dumps({"hbm_read_ceiling_GBps": max(v["GBps"] for v in res.values()), "stream_ceiling": res}))
        return
    if args.e2e_only:
        print(json.dumps({"e2e_config4_llama2_7b": e2e_extra(torch, dev)}))
        return
    if args.hf_only:
        print(json.dumps({"hf_generate_config4": hf_generate_extra(torch, dev, batch=args.hf_batch, prompt_len=args.hf_prompt, new_tokens=args.hf_new_tokens)}))
        return
    if args.attention_step_only:
        if args.copy_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            for _ in range(5):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst
        print(json.dumps({"attention_step": attention_step_extra(torch, dev)}))
        return
    if args.shapes_only:
        if args.copy_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            for _ in range(5):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst
        st = torch.cuda.current_stream().cuda_stream
        res = {"target_shape_B16_T8192": target_shape_extra(torch, _lib, lib, dev, st),
               "gqa_config2_B16_T32768": gqa_shape_extra(torch, _lib, lib, dev, st)}
        if not args.no_sweep:
            res["sweep_config3_T4096"] = sweep_extra(torch, _lib, lib, dev, st)
        if not args.no_attention_step:
            torch.cuda.empty_cache()
            res["attention_step"] = attention_step_extra(torch, dev)
        print(json.dumps(res))
        return
    kbits, vbits = layer_bits(args.layers)
    layers = build_layers(torch, ops, lib, B, H, D, T, R, kbits, vbits, dev)
    torch.cuda.synchronize()

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    side = torch.cuda.Stream()
    mode = "eager"
    graph = None
    with torch.cuda.stream(side):
        calls = make_calls(torch, _lib, lib, layers, B, H, D, side.cuda_stream)
        run_step(calls)
        side.synchronize()
        per_kernel = time_kernels(torch, calls)
        if not args.no_graph:
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    run_step(calls)
                mode = "hipgraph"
            except Exception as ex:  # capture unsupported: stay eager
                graph = None
                mode = f"eager (graph capture failed: {type(ex).__name__})"

        def step():
            if graph is not None:
                graph.replay()
            else:
                run_step(calls)

        for _ in range(args.warmup):
            step()
        side.synchronize()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        s.record(side)
        for _ in range(args.steps):
            step()
        e.record(side)
        side.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ev_ms = s.elapsed_time(e)

    ms_per_step = wall * 1e3 / args.steps
    step_bytes = sum(b for _, b, _ in calls)
    gemv_bytes = sum(b for t, b, _ in calls if t.startswith("gemv"))
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # dominant kernel of the step
    dom = max(per_kernel.items(), key=lambda kv: kv[1]["launches_per_step"] * kv[1]["avg_us"])
    dname, d = dom
    achieved = d["bytes_per_launch"] / d["avg_us"] / 1e3
    # HBM traffic of the dominant kernel: NOT measured in this run -- read from the committed counter summary
    # (two rocprofv3 --pmc passes, FETCH_SIZE and WRITE_SIZE scaled by a plain copy; profiles/bench_step_kernels_config1.md)
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        try:
            tj = json.load(open(tpath))
            traffic = tj.get(dname)
            traffic_source = ("profiles/hbm_traffic.json (static: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                              + str(tj.get("_measured", "date not recorded")) + "; not re-measured in this run)")
            # the figure belongs to the device kernel that ran when the counters were taken: if the dispatch has
            # moved on since, it is not this kernel's traffic
            then, now = tj.get("_kernels", {}).get(dname), device_kernel(_lib, dname, B, H, D, T - R)
            if then is not None and then != now:
                traffic = None
                traffic_source += f" -- stale: measured on {then}, the step now runs {now}"
        except Exception:
            traffic = None
    gemv_us = sum(v["launches_per_step"] * v["avg_us"] for k, v in per_kernel.items() if k.startswith("gemv"))
    quant_us = sum(v["launches_per_step"] * v["avg_us"] for k, v in per_kernel.items() if k.startswith("quant"))
    quant_bytes = step_bytes - gemv_bytes

    result = {
        "metric": "fused dequant-GEMV HBM GB/s (% peak) + decode tok/s, Llama-2-7B mixed-bit KV",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32 codes / fp16 scale,zero / fp32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: 32-layer Llama-2-7B KV shape, mixed per-layer bits, one flush + q.K^T + p.V per layer "
                        "(the layers' flushes batched eight to a launch at the head of the step: they take tokens of earlier steps only)",
            "batch": B, "context": T, "heads": H, "head_dim": D, "group": 32, "residual": R, "layers": args.layers,
            "k_bits": kbits, "v_bits": vbits, "k3_format": "reference 11-per-word (group 11)",
            "v3_format": "dense 3-bit stream (extension)", "launch": mode,
            "scratch": "logits, probabilities and attention output: one buffer each shared by the layers, as a decode "
                       "loop reuses them; packed caches, flush sources and flush targets per layer",
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "kv_path_only_decode_tokens_per_s": round(B / (ms_per_step * 1e-3), 1),
        "step_bytes": int(step_bytes),
        "event_ms_per_step": round(ev_ms / args.steps, 4),
        "gemv_only": {"bytes": int(gemv_bytes), "us": round(gemv_us, 1), "GBps": round(gemv_bytes / gemv_us / 1e3, 1),
                      "frac_of_peak": round(gemv_bytes / gemv_us / 1e3 / HBM_PEAK_GBPS, 4)},
        "quantizer_only": {"bytes": int(quant_bytes), "us": round(quant_us, 1),
                           "GBps": round(quant_bytes / quant_us / 1e3, 1)},
        "kernels": {k: {"launches_per_step": v["launches_per_step"], "avg_us": round(v["avg_us"], 2),
                        "GBps": round(v["bytes_per_launch"] / v["avg_us"] / 1e3, 1)} for k, v in per_kernel.items()},
        "roofline": {"kernel": dname, "device_kernel": device_kernel(_lib, dname, B, H, D, T - R),
                     "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "traffic_source": traffic_source,
                     "bytes_per_launch": int(d["bytes_per_launch"]), "avg_launch_us": round(d["avg_us"], 2)},
    }
    print_result(result, args, torch, _lib, lib, dev, layers, kbits, vbits, B, H, D, T, R)


def print_result(result, args, torch, _lib, lib, dev, layers, kbits, vbits, B, H, D, T, R):
    def extra(key, fn):
        """One more object on the line; whatever goes wrong in it, the headline is still printed."""
        try:
            result[key] = fn()
        except Exception as ex:
            result[key] = {"error": f"{type(ex).__name__}: {ex}"}
            result.setdefault("extras_failed", []).append(key)  # (the headline stands; what broke is named on the line)
        torch.cuda.empty_cache()

    st = torch.cuda.current_stream().cuda_stream
    if not args.no_cpu_baseline:
        extra("cpu_baseline", lambda: cpu_baseline(layers, kbits, vbits, B, H, D, T, R))
    if not args.no_target_shape:
        # free the 32-layer cache first: the target-shape buffers need ~3 GB of their own
        for L in layers:
            L.__dict__.clear()
        torch.cuda.empty_cache()
        if not args.no_stream_ceiling:
            extra("stream_ceiling", lambda: stream_ceiling_extra(torch, _lib, lib, dev))
            if "error" not in result["stream_ceiling"]:
                result["hbm_read_ceiling_GBps"] = max(v["GBps"] for v in result["stream_ceiling"].values())
        extra("target_shape_B16_T8192", lambda: target_shape_extra(torch, _lib, lib, dev, st))
        extra("gqa_config2_B16_T32768", lambda: gqa_shape_extra(torch, _lib, lib, dev, st))
        if not args.no_sweep:
            extra("sweep_config3_T4096", lambda: sweep_extra(torch, _lib, lib, dev, st))
        if not args.no_attention_step:
            extra("attention_step", lambda: attention_step_extra(torch, dev))
    if not args.no_e2e:
        extra("e2e_config4_llama2_7b", lambda: e2e_extra(torch, dev))
        extra("hf_generate_config4", lambda: hf_generate_extra(torch, dev))
        # the same at batch 16, where the transformers host loop no longer hides the cache
        extra("hf_generate_config4_batch16", lambda: hf_generate_extra(torch, dev, batch=16))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
