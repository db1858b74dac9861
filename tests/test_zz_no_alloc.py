"""kvmix_quantized_gemv_static (the entry point that allocates nothing) through the C ABI against
kvmix_quantized_gemv with a caller-owned workspace: same kernels, so the outputs must be equal bit
for bit.  Two calls in a row share the library's built-in scratch buffer; the second is smaller, so
stale partial sums of the first lie beyond (and partly under) what it writes.  Shapes are p.V
products small enough in batch to be split over K (the only user of the scratch), plus one q.K^T
product and one unsplit batch that must not touch it."""

import numpy as np
import pytest
import torch

from helpers import gemv_close, kv_like

pytestmark = pytest.mark.gpu


def _operands(oracle, dev, bits, g, B, nh, nkv, K, N, seed):
    rng = np.random.default_rng(seed)
    w = kv_like(rng, (B, nkv, K, N), outlier_axis=2, n_outliers=min(2, K))
    code, scale, zero = oracle.quantize_pack_last_dim(w, g, bits)
    x = rng.standard_normal((B, nh, 1, K)).astype(np.float16)
    _, want64, abs64 = oracle.quantized_gemm(g, x, code, scale, zero, bits, want_f64=True)
    dv = [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in (x, code, scale, zero)]
    return dv, want64, abs64


def _call(L, static, g, bits, dv, B, nh, nkv, K, N, ws=None):
    x, code, scale, zero = dv
    out = torch.full((B, nh, 1, N), float("nan"), dtype=torch.float16, device=x.device)
    head = (g, x.data_ptr(), K, K, code.data_ptr(), code.stride(1), code.stride(2), scale.data_ptr(), zero.data_ptr(),
            scale.stride(1), scale.stride(2), bits, 0, B * nh, nh // nkv, 1, K, N, out.data_ptr(), N, N)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    if static:
        rc = L.kvmix_quantized_gemv_static(*head, stream)
    else:
        rc = L.kvmix_quantized_gemv(*head, ws.data_ptr() if ws is not None else None,
                                    ws.numel() if ws is not None else 0, stream)
    torch.cuda.synchronize()
    return rc, out.cpu().numpy()


CASES = [
    # (bits, g, B, nh, nkv, K, N): first call, then a smaller one
    ((4, 32, 1, 32, 32, 8064, 128), (4, 32, 1, 8, 8, 2048 + 17, 128)),
    ((2, 32, 2, 8, 2, 4000, 128), (1, 32, 1, 4, 4, 1500, 128)),      # GQA (four heads per block), then 1-bit
    ((4, 32, 1, 4, 4, 3000, 256), (2, 32, 1, 2, 2, 700, 64)),        # vector-ALU p.V kernel (N != 128)
    ((4, 32, 1, 4, 4, 128, 4096), (4, 32, 16, 32, 32, 256, 128)),    # q.K^T, then an unsplit batch: no scratch used
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_gemv_equals_workspace_gemv(oracle, dev, first, second):
    from kvmix_amd import _lib

    L = _lib.load()
    with torch.cuda.device(dev):
        prepared = []
        for i, (bits, g, B, nh, nkv, K, N) in enumerate((first, second)):
            dv, want64, abs64 = _operands(oracle, dev, bits, g, B, nh, nkv, K, N, seed=100 + i)
            need = L.kvmix_gemv_workspace_bytes(B * nh, 1, K, N)
            assert need <= _lib.GEMV_STATIC_SCRATCH_BYTES
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
            rc, ref = _call(L, False, g, bits, dv, B, nh, nkv, K, N, ws)
            assert rc == 0, _lib.strerror(rc)
            ok, worst = gemv_close(ref, want64, abs64)
            assert ok, ("workspace entry point vs oracle", first, second, worst)
            prepared.append((bits, g, B, nh, nkv, K, N, dv, ref, want64, abs64))
        # the two static calls back to back, nothing else touching the scratch in between
        for bits, g, B, nh, nkv, K, N, dv, ref, want64, abs64 in prepared:
            rc, got = _call(L, True, g, bits, dv, B, nh, nkv, K, N)
            assert rc == 0, _lib.strerror(rc)
            assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), ("static vs workspace", bits, B, nh, K, N)
            ok, worst = gemv_close(got, want64, abs64)
            assert ok, ("static entry point vs oracle", bits, B, nh, K, N, worst)


def test_static_scratch_rejects_oversized_problem(dev):
    """A split-K problem beyond the built-in buffer is refused before anything is launched."""
    from kvmix_amd import _lib

    L = _lib.load()
    with torch.cuda.device(dev):
        # 120 output rows of 64k tokens, 256 columns: 2.11 MiB of partial sums
        B, nh, K, N, g, bits = 1, 120, 1 << 16, 256, 32, 4
        need = L.kvmix_gemv_workspace_bytes(B * nh, 1, K, N)
        assert need > _lib.GEMV_STATIC_SCRATCH_BYTES, need
        one = torch.zeros(16, dtype=torch.uint8, device=dev)  # never dereferenced: the call fails on the host
        p = one.data_ptr()
        rc = L.kvmix_quantized_gemv_static(g, p, K, K, p, K * (N // 8), N // 8, p, p, K * (N // 32), N // 32, bits, 0,
                                           B * nh, 1, 1, K, N, p, N, N, torch.cuda.current_stream(dev).cuda_stream)
        assert rc == -13
        assert "built-in buffer" in _lib.strerror(rc)
        torch.cuda.synchronize()


def test_static_scratch_gemv_allocates_nothing_and_replays_from_a_graph(oracle, dev):
    """What the entry point promises: after one warm call (the buffer's address is looked up then) further calls
    leave the device's free memory and torch's allocator untouched; and a call recorded into a HIP graph -- where an
    allocation would fail the capture -- replays to the eager result, every time."""
    from kvmix_amd import _lib

    L = _lib.load()
    bits, g, B, nh, nkv, K, N = 4, 32, 1, 16, 16, 4096 + 32, 128    # a p.V product that is split over K
    assert L.kvmix_gemv_workspace_bytes(B * nh, 1, K, N) > 0
    with torch.cuda.device(dev):
        dv, want64, abs64 = _operands(oracle, dev, bits, g, B, nh, nkv, K, N, seed=7)
        x, code, scale, zero = dv
        out = torch.full((B, nh, 1, N), float("nan"), dtype=torch.float16, device=dev)
        head = (g, x.data_ptr(), K, K, code.data_ptr(), code.stride(1), code.stride(2), scale.data_ptr(), zero.data_ptr(),
                scale.stride(1), scale.stride(2), bits, 0, B * nh, nh // nkv, 1, K, N, out.data_ptr(), N, N)
        stream = torch.cuda.current_stream(dev).cuda_stream
        assert L.kvmix_quantized_gemv_static(*head, stream) == 0     # warm: symbol lookup, kernel attributes
        torch.cuda.synchronize()
        eager = out.clone()
        ok, worst = gemv_close(eager.cpu().numpy(), want64, abs64)
        assert ok, worst
        free0, alloc0, reserved0 = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)
        for _ in range(3):
            assert L.kvmix_quantized_gemv_static(*head, stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free0
        assert (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)) == (alloc0, reserved0)
        assert torch.equal(out, eager)
        # under capture: the launches are recorded on the capturing stream, nothing else happens
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(dev)
        with torch.cuda.graph(graph, stream=side):
            rc = L.kvmix_quantized_gemv_static(*head, side.cuda_stream)
        assert rc == 0, _lib.strerror(rc)
        for _ in range(3):
            out.fill_(float("nan"))        # the program's own eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
