"""The fused key+value flush against the two separate operators and the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from helpers import kv_like, same_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("k_bits,v_bits", [(4, 4), (2, 4), (3, 2), (4, 3), (1, 1), (3, 3)])
@pytest.mark.parametrize("shape", [(2, 3, 64, 128, 32), (1, 2, 128, 128, 96), (2, 1, 32, 64, 1)])
def test_fused_flush_matches_separate(k_bits, v_bits, shape):
    from kvmix_amd import ops
    from oracle import kvmix_oracle as O

    B, H, n, D, nv = shape
    rng = np.random.default_rng(k_bits * 100 + v_bits * 10 + n)
    k_group = 11 if k_bits == 3 else 32
    nk = (n // k_group) * k_group if k_bits != 3 else 66 if n >= 66 else 33
    k_np = kv_like(rng, (B, H, nk, D)).astype(np.float16)
    v_np = kv_like(rng, (B, H, nv, D)).astype(np.float16)
    k = torch.from_numpy(k_np).cuda()
    v = torch.from_numpy(v_np).cuda()
    v_fmt = ops.FMT_DENSE3 if v_bits == 3 else ops.FMT_REF
    kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(k, k_group, k_bits, v, 32, v_bits, ops.FMT_REF, v_fmt)
    # separate operators
    kc2, ks2, km2 = ops.quantize_pack_last_dim_cuda(k.transpose(2, 3).contiguous(), k_group, k_bits)
    if v_bits == 3:
        vc2, vs2, vm2 = ops.quantize_pack_dense3(v, 32)
    else:
        vc2, vs2, vm2 = ops.quantize_pack_last_dim_cuda(v, 32, v_bits)
    torch.cuda.synchronize()
    for got, want in ((kc, kc2), (ks, ks2), (km, km2), (vc, vc2), (vs, vs2), (vm, vm2)):
        assert got.shape == want.shape
        assert same_bits(got.cpu().numpy(), want.cpu().numpy())
    # and the oracle for the key half (the transposed call is what the reference runs)
    oc, osc, omn = O.quantize_pack_last_dim(np.ascontiguousarray(k_np.transpose(0, 1, 3, 2)), k_group, k_bits)
    assert same_bits(kc.cpu().numpy(), oc) and same_bits(ks.cpu().numpy(), osc) and same_bits(km.cpu().numpy(), omn)


def test_fused_flush_rejects_bad_halves_before_launching():
    from kvmix_amd import ops

    k = torch.zeros(1, 1, 32, 64, dtype=torch.float16, device="cuda")
    v = torch.zeros(1, 1, 4, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.quantize_kv_flush(k, 32, 4, v, 48, 4)  # 64 not divisible by 48
    with pytest.raises(RuntimeError):
        ops.quantize_kv_flush(k, 11, 3, v, 32, 4)  # 32 tokens not divisible by 11


def test_fused_flush_empty_half():
    from kvmix_amd import ops

    k = torch.randn(1, 2, 0, 64, dtype=torch.float16, device="cuda")
    v = torch.randn(1, 2, 8, 64, dtype=torch.float16, device="cuda")
    kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(k, 32, 4, v, 32, 4)
    vc2, vs2, vm2 = ops.quantize_pack_last_dim_cuda(v, 32, 4)
    assert kc.shape == (1, 2, 64, 0)
    assert torch.equal(vc, vc2) and torch.equal(vs, vs2) and torch.equal(vm, vm2)
