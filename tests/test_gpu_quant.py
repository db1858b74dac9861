"""GPU parity of the HIP quantize + bit-pack kernels against the CPU oracle, through the
reference's operator surface (module KVmix) and the C ABI.  Codes, scale and zero must be
bit-exact.  Reference: quant_cuda/csrc/quantization_cuda.cu:298-721."""
import numpy as np
import pytest
import torch

from helpers import kv_like, same_bits

pytestmark = pytest.mark.gpu

BITS_G = [(1, 32), (2, 32), (4, 32), (3, 11), (4, 8), (2, 16), (1, 64), (4, 64), (4, 128)]


def to_np(t):
    return t.detach().cpu().numpy()


def check_triplet(got, want, what=""):
    for name, g, w in zip(("code", "scale", "min"), got, want):
        g = to_np(g)
        assert g.dtype == w.dtype, (what, name, g.dtype, w.dtype)
        assert same_bits(g, w), (what, name, int((g.view(np.uint8) != w.view(np.uint8)).sum()))


@pytest.mark.parametrize("bits,g", BITS_G)
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_one_shot_matches_oracle(oracle, dev, bits, g, dtype):
    import KVmix

    rng = np.random.default_rng(bits * 100 + g)
    unit = int(np.lcm(g, oracle.values_per_word(bits)))
    for shape in [(2, 3, 5, unit * 4), (1, 1, 1, unit), (1, 2, 130, unit * 3)]:
        x = kv_like(rng, shape, outlier_axis=2, n_outliers=1, dtype=dtype)
        x[0, 0, 0, :g] = dtype(1.5)                      # constant group -> scale 0, codes 0
        got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(x).to(dev), g, bits)
        check_triplet(got, oracle.quantize_pack_last_dim(x, g, bits), f"{bits}b g{g} {shape}")


def test_key_and_value_call_shapes_of_the_model(oracle, dev):
    """The two call sites of models/modeling_llama_KVmix.py:131-133,159-161 at head_dim 128."""
    import KVmix

    rng = np.random.default_rng(1)
    B, H, n, D = 2, 8, 128, 128
    tail_k = kv_like(rng, (B, H, n, D), outlier_axis=3)
    tail_v = kv_like(rng, (B, H, n, D), outlier_axis=3)
    for bits in (1, 2, 4):
        kt = torch.from_numpy(tail_k).to(dev).transpose(2, 3).contiguous()
        got = KVmix.quantize_pack_last_dim_cuda(kt, 32, bits)
        check_triplet(got, oracle.quantize_pack_last_dim(np.ascontiguousarray(tail_k.transpose(0, 1, 3, 2)), 32, bits))
        got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(tail_v).to(dev), 32, bits)
        check_triplet(got, oracle.quantize_pack_last_dim(tail_v, 32, bits))
    k3 = tail_k[:, :, :121]
    got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(k3).to(dev).transpose(2, 3).contiguous(), 11, 3)
    check_triplet(got, oracle.quantize_pack_last_dim(np.ascontiguousarray(k3.transpose(0, 1, 3, 2)), 11, 3))


def test_special_values(oracle, dev):
    """NaN elements are ignored by min/max and get code 0; ties round away from zero;
    tiny and huge magnitudes; negative zero."""
    import KVmix

    x = np.zeros((1, 1, 4, 32), np.float32)
    x[0, 0, 0, :10] = [0, 15, 0.5, 1.5, 2.5, 3.5, 6.5, 13.5, 14.5, 0.49999997]
    x[0, 0, 1, :] = np.linspace(-3, 3, 32)
    x[0, 0, 1, 5] = np.nan
    x[0, 0, 2, :] = np.linspace(1e-30, 3e-30, 32)
    x[0, 0, 3, :] = np.linspace(-1e30, 2e30, 32)
    x[0, 0, 3, 0] = -0.0
    for bits in (1, 2, 4):
        got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(x).to(dev), 32, bits)
        want = oracle.quantize_pack_last_dim(x, 32, bits)
        check_triplet(got, want)
    h = x[:, :, :2].astype(np.float16)
    got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(h).to(dev), 32, 4)
    check_triplet(got, oracle.quantize_pack_last_dim(h, 32, 4))
    assert list(oracle.unpack_np(to_np(got[0]), 4)[0, 0, 0, :9]) == [0, 15, 1, 2, 3, 4, 7, 14, 15]


def test_every_fp16_pair_step(oracle, dev):
    """All 2-value 1-bit/4-bit groups built from a sweep of fp16 bit patterns: exercises the
    division and rounding over the whole fp16 range (padding keeps min/max inside the group)."""
    import KVmix

    rng = np.random.default_rng(3)
    bits16 = rng.integers(0, 0x7C00, size=(64, 64, 32), dtype=np.uint16)  # finite positives
    sign = rng.integers(0, 2, size=bits16.shape, dtype=np.uint16) << 15
    x = (bits16 | sign).view(np.float16).reshape(1, 64, 64, 32)
    for bits in (2, 4):
        got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(x).to(dev), 32, bits)
        check_triplet(got, oracle.quantize_pack_last_dim(x, 32, bits))


def test_non_contiguous_and_empty_inputs(oracle, dev):
    import KVmix

    rng = np.random.default_rng(4)
    big = kv_like(rng, (2, 3, 10, 256))
    t = torch.from_numpy(big).to(dev)
    view = t[:, :, 2:9, 64:192]                       # strided rows, offset start
    got = KVmix.quantize_pack_last_dim_cuda(view, 32, 4)
    check_triplet(got, oracle.quantize_pack_last_dim(np.ascontiguousarray(big[:, :, 2:9, 64:192]), 32, 4))
    tr = t.transpose(2, 3)                            # last stride != 1 -> copied like the reference does
    got = KVmix.quantize_pack_last_dim_cuda(tr[..., :8], 8, 4)
    check_triplet(got, oracle.quantize_pack_last_dim(np.ascontiguousarray(big.transpose(0, 1, 3, 2)[..., :8]), 8, 4))
    empty = torch.zeros((2, 3, 0, 64), dtype=torch.float16, device=dev)
    c, s, m = KVmix.quantize_pack_last_dim_cuda(empty, 32, 4)
    assert c.shape == (2, 3, 0, 8) and s.shape == (2, 3, 0, 2) and m.shape == (2, 3, 0, 2)
    empty = torch.zeros((2, 3, 4, 0), dtype=torch.float16, device=dev)
    c, s, m = KVmix.quantize_pack_last_dim_cuda(empty, 32, 4)
    assert c.shape == (2, 3, 4, 0) and s.shape == (2, 3, 4, 0)


@pytest.mark.parametrize("bits,g", [(4, 32), (2, 32), (1, 32), (3, 11), (4, 8)])
def test_append_variants_match_oracle(oracle, dev, bits, g):
    import KVmix

    rng = np.random.default_rng(bits + 60)
    unit = int(np.lcm(g, oracle.values_per_word(bits)))
    B, H, D = 2, 2, 16
    old = kv_like(rng, (B, H, D, unit * 2))
    new = kv_like(rng, (B, H, D, unit * 3))
    c0, s0, z0 = oracle.quantize_pack_last_dim(old, g, bits, oracle.SCALE_DIVIDE)
    want = oracle.process_key_quantization(new, c0, s0, z0, g, bits)
    tt = lambda a: torch.from_numpy(a).to(dev)
    got = KVmix.process_key_quantization_cuda(tt(new), tt(c0), tt(s0), tt(z0), g, bits)
    check_triplet(got, want, "key append")
    got = KVmix.process_key_quantization_cuda(tt(new), tt(c0[..., :0]), tt(s0[..., :0]), tt(z0[..., :0]), g, bits)
    check_triplet(got, oracle.process_key_quantization(new, c0[..., :0], s0[..., :0], z0[..., :0], g, bits))
    if bits != 3:
        Dv = 64
        oldv = kv_like(rng, (B, H, 5, Dv))
        newv = kv_like(rng, (B, H, 7, Dv))
        c0, s0, z0 = oracle.quantize_pack_last_dim(oldv, g, bits, oracle.SCALE_DIVIDE)
        want = oracle.process_value_quantization(newv, c0, s0, z0, g, bits)
        got = KVmix.process_value_quantization_cuda(tt(newv), tt(c0), tt(s0), tt(z0), g, bits)
        check_triplet(got, want, "value append")


def test_value_append_3bit_placeholder(oracle, dev):
    import KVmix

    rng = np.random.default_rng(9)
    B, H, D = 1, 2, 44
    oldv = kv_like(rng, (B, H, 3, D), dtype=np.float32)
    newv = kv_like(rng, (B, H, 4, D), dtype=np.float32)
    e = np.zeros((B, H, 0, D // 11), np.int32)
    ef = np.zeros((B, H, 0, D // 11), np.float32)
    c0, s0, z0 = oracle.process_value_quantization(oldv, e, ef, ef, 11, 3)
    want = oracle.process_value_quantization(newv, c0, s0, z0, 11, 3)
    tt = lambda a: torch.from_numpy(a).to(dev)
    got = KVmix.process_value_quantization_cuda(tt(newv), tt(c0), tt(s0), tt(z0), 11, 3)
    check_triplet(got, want)


@pytest.mark.parametrize("bits,g,fmt,groups", [(4, 32, 0, 4), (2, 32, 0, 4), (1, 32, 0, 4), (3, 11, 0, 4),
                                               (3, 11, 0, 11), (3, 11, 0, 25)])
def test_key_tokens_kernel_equals_transpose_then_quantize(oracle, dev, bits, g, fmt, groups):
    """C ABI kvmix_quant_pack_key_tokens == quantize_pack_last_dim(tail[:, :, :n].transpose(2,3))
    written at an offset into a larger channel-major cache.  (The reference 3-bit kernel takes the groups of a
    slice eleven at a time: fewer than, exactly and more than eleven, the last chunk ragged.)"""
    from kvmix_amd import _lib

    L = _lib.load()
    rng = np.random.default_rng(bits + 70)
    B, H, D = 2, 3, 128
    n = g * groups
    cap_tokens = g * (groups + 6)
    vpw = oracle.values_per_word(bits)
    tail = kv_like(rng, (B, H, n + 5, D), outlier_axis=3)     # longer tail, only n flushed
    t = torch.from_numpy(tail).to(dev)
    capw, capg = cap_tokens // vpw, cap_tokens // g
    code = torch.full((B, H, D, capw), -1, dtype=torch.int32, device=dev)
    scale = torch.full((B, H, D, capg), -1.0, dtype=torch.float16, device=dev)
    zero = torch.full((B, H, D, capg), -1.0, dtype=torch.float16, device=dev)
    off = 2 * g
    cv, sv, zv = code[..., off // vpw:], scale[..., off // g:], zero[..., off // g:]
    rc = L.kvmix_quant_pack_key_tokens(t.data_ptr(), B * H, n, D, t.stride(1), t.stride(2), g, bits, fmt,
                                       _lib.SCALE_RECIPROCAL, cv.data_ptr(), code.stride(1), code.stride(2),
                                       sv.data_ptr(), zv.data_ptr(), scale.stride(1), scale.stride(2),
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    want = oracle.quantize_pack_last_dim(np.ascontiguousarray(tail[:, :, :n].transpose(0, 1, 3, 2)), g, bits)
    assert same_bits(to_np(code[..., off // vpw: (off + n) // vpw]), want[0])
    assert same_bits(to_np(scale[..., off // g: (off + n) // g]), want[1])
    assert same_bits(to_np(zero[..., off // g: (off + n) // g]), want[2])
    # nothing outside the target window was touched
    assert (to_np(code[..., : off // vpw]) == -1).all() and (to_np(code[..., (off + n) // vpw:]) == -1).all()
    assert (to_np(scale[..., : off // g]) == -1).all() and (to_np(scale[..., (off + n) // g:]) == -1).all()


def test_key_tokens_kernel_with_more_slices_than_one_grid_dimension_holds(oracle, dev):
    """kvmix_quant_pack_key_tokens with more than 65535 (batch, head) slices: several launches."""
    from kvmix_amd import _lib

    L = _lib.load()
    rng = np.random.default_rng(77)
    outer, n, D, g, bits = 65539, 32, 16, 32, 4
    tail = rng.standard_normal((outer, n, D)).astype(np.float16)
    t = torch.from_numpy(tail).to(dev)
    code = torch.zeros((outer, D, n // 8), dtype=torch.int32, device=dev)
    scale = torch.zeros((outer, D, 1), dtype=torch.float16, device=dev)
    zero = torch.zeros_like(scale)
    rc = L.kvmix_quant_pack_key_tokens(t.data_ptr(), outer, n, D, t.stride(0), t.stride(1), g, bits, 0,
                                       _lib.SCALE_RECIPROCAL, code.data_ptr(), code.stride(0), code.stride(1),
                                       scale.data_ptr(), zero.data_ptr(), scale.stride(0), scale.stride(1),
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    want = oracle.quantize_pack_last_dim(np.ascontiguousarray(tail.transpose(0, 2, 1))[None], g, bits)
    assert same_bits(to_np(code)[None], want[0]) and same_bits(to_np(scale)[None], want[1])
    assert same_bits(to_np(zero)[None], want[2])


def test_scale_matches_torch_division_by_scalar_on_gpu(oracle, dev):
    """The returned scale is what `(max - min) / qmax` gives when torch evaluates that line
    (quantization_cuda.cu:711) on the GPU."""
    import KVmix

    rng = np.random.default_rng(12)
    x = kv_like(rng, (2, 8, 256, 256), dtype=np.float32) * np.float32(3.7)
    t = torch.from_numpy(x).to(dev)
    for bits in (2, 4):
        _, scale, mn = KVmix.quantize_pack_last_dim_cuda(t, 32, bits)
        g = t.reshape(2, 8, 256, 8, 32)
        want = (g.max(-1).values - g.min(-1).values) / ((1 << bits) - 1)
        assert torch.equal(scale, want)
        assert torch.equal(mn, g.min(-1).values)


def test_full_size_flush_properties(dev):
    """BASELINE-size flush (B=8, 32 heads, 128 tokens, head_dim 128): size-independent
    properties checked on the GPU -- min -> code 0, max -> qmax, |dequant - x| <= scale/2."""
    import KVmix

    torch.manual_seed(0)
    B, H, n, D = 8, 32, 128, 128
    v = torch.randn(B, H, n, D, device=dev, dtype=torch.float16)
    v[..., ::37] *= 10
    for bits in (1, 2, 4):
        qmax = (1 << bits) - 1
        code, scale, mn = KVmix.quantize_pack_last_dim_cuda(v, 32, bits)
        shifts = torch.arange(0, 32, bits, device=dev, dtype=torch.int32)
        q = ((code.unsqueeze(-1) >> shifts) & qmax).reshape(B, H, n, D // 32, 32)
        xg = v.float().reshape(B, H, n, D // 32, 32)
        assert torch.equal(mn.float(), xg.min(-1).values)
        assert (torch.gather(q, -1, xg.argmin(-1, keepdim=True)) == 0).all()
        assert (torch.gather(q, -1, xg.argmax(-1, keepdim=True)) == qmax).all()
        deq = scale.float().unsqueeze(-1) * q + mn.float().unsqueeze(-1)
        bound = scale.float().unsqueeze(-1) * 0.5 + 2.0 ** -10 * (mn.float().abs().unsqueeze(-1) + qmax * scale.float().unsqueeze(-1))
        assert ((deq - xg).abs() <= bound).all()


@pytest.mark.parametrize("bits", [4, 2, 1, 3])
def test_prompt_size_inputs_take_the_streaming_kernels(oracle, dev, bits):
    """Inputs of prompt size (2 M groups and more) go through the one-thread-per-group kernels;
    bits = 3 covers both the dense stream (group 32) and the reference format (group 11, fp16)."""
    import KVmix
    from kvmix_amd import ops

    rng = np.random.default_rng(bits)
    x = kv_like(rng, (4, 8, 2048 * 4 + 3, 256)).astype(np.float16)  # 2 098 944 groups of 32, rows not a block multiple
    xt = torch.from_numpy(x).to(dev)
    if bits == 3:
        code, scale, mn = ops.quantize_pack_dense3(xt, 32)
        oc, osc, omn = oracle.quantize_pack_dense3(x, 32)
    else:
        code, scale, mn = KVmix.quantize_pack_last_dim_cuda(xt, 32, bits)
        oc, osc, omn = oracle.quantize_pack_last_dim(x, 32, bits)
    assert same_bits(code.cpu().numpy(), oc) and same_bits(scale.cpu().numpy(), osc) and same_bits(mn.cpu().numpy(), omn)
    if bits == 3:
        x11 = np.ascontiguousarray(x[..., :253])  # 23 words per row: odd row length, 2-byte aligned rows
        code, scale, mn = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(x11).to(dev), 11, 3)
        oc, osc, omn = oracle.quantize_pack_last_dim(x11, 11, 3)
        assert same_bits(code.cpu().numpy(), oc) and same_bits(scale.cpu().numpy(), osc) and same_bits(mn.cpu().numpy(), omn)


@pytest.mark.parametrize("bits", [4, 2, 3])
def test_values_at_and_next_to_rounding_ties(oracle, dev, bits):
    """The kernels decide most codes from (x - min) * (1 / scale) and fall back to the division only
    near a tie: values exactly on k + 0.5, and a few ulps to either side, must still give the
    division's code.  fp32 input (every ulp reachable) and fp16 input (exact ties)."""
    import KVmix

    rng = np.random.default_rng(40 + bits)
    g = 11 if bits == 3 else 32
    qmax = 7 if bits == 3 else (1 << bits) - 1
    rows = 4096
    x = np.empty((1, 1, rows, g), np.float32)
    for r in range(rows):
        mn = np.float32(rng.uniform(-8, 8))
        scale = np.float32(2.0 ** rng.integers(-12, 6)) * np.float32(rng.uniform(1, 2))
        mx = np.float32(mn + np.float32(qmax) * scale)
        k = rng.integers(0, qmax, g).astype(np.float32)
        v = (mn + (k + np.float32(0.5)) * scale).astype(np.float32)
        ulps = rng.integers(-3, 4, g)
        v = (v.view(np.int32) + (ulps * np.sign(v)).astype(np.int32)).astype(np.int32).view(np.float32)
        v[0], v[1] = mn, mx  # pin the group's min and max
        x[0, 0, r] = np.clip(v, mn, mx)
    got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(x).to(dev), g, bits)
    check_triplet(got, oracle.quantize_pack_last_dim(x, g, bits), "fp32 ties")
    # fp16: min 0, max qmax * 2^e -> every k + 0.5 step is an exact tie
    xh = np.empty((1, 1, 64, g), np.float16)
    for r in range(64):
        s = 2.0 ** (r % 8 - 3)
        k = rng.integers(0, qmax, g)
        v = (k + 0.5) * s
        v[0], v[1] = 0.0, qmax * s
        xh[0, 0, r] = v
    got = KVmix.quantize_pack_last_dim_cuda(torch.from_numpy(xh).to(dev), g, bits)
    check_triplet(got, oracle.quantize_pack_last_dim(xh, g, bits), "fp16 ties")
