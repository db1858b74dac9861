"""ops.rope_append against the torch composition it replaces (x * cos + rotate_half(x) * sin in
fp16 tensor arithmetic, then a copy into the tail slot): bit-identical, and nothing else in the
windows is touched."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def torch_rope(x, cos, sin):
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos + rot * sin


@pytest.mark.parametrize("B,nh,nkv,D", [(4, 32, 32, 128), (3, 8, 2, 128), (2, 4, 4, 64), (1, 6, 3, 256), (5, 1, 1, 16)])
def test_rope_append_matches_torch_bit_for_bit(dev, B, nh, nkv, D):
    from kvmix_amd import ops

    gen = torch.Generator(device=dev).manual_seed(B * 1000 + D)
    qkv = (torch.randn(B, 1, (nh + 2 * nkv) * D, device=dev, generator=gen) * 3).half()
    ang = torch.rand(D // 2, device=dev, generator=gen) * 6.283
    cos = torch.cat([ang, ang]).cos().half()
    sin = torch.cat([ang, ang]).sin().half()
    slots, ks, vs = 9, 3, 7
    # windows are views into longer buffers (as the cache hands them out): token stride = D, but
    # batch and head strides belong to the larger allocation
    kbuf = torch.full((B, nkv, slots + 5, D), 7.0, dtype=torch.float16, device=dev)
    vbuf = torch.full((B, nkv, slots + 2, D), -7.0, dtype=torch.float16, device=dev)
    kwin, vwin = kbuf[:, :, 2:2 + slots], vbuf[:, :, 1:1 + slots]
    heads = qkv.view(B, nh + 2 * nkv, D)
    want_q = torch_rope(heads[:, :nh], cos, sin)
    want_k = torch_rope(heads[:, nh:nh + nkv], cos, sin)
    want_v = heads[:, nh + nkv:]
    for device_slots in (False, True):
        kbuf.fill_(7.0)
        vbuf.fill_(-7.0)
        k_slot = torch.tensor([ks], dtype=torch.int64, device=dev) if device_slots else ks
        v_slot = torch.tensor([vs], dtype=torch.int64, device=dev) if device_slots else vs
        q = ops.rope_append(qkv, cos, sin, nh, nkv, kwin, vwin, k_slot, v_slot)
        assert q.shape == (B, nh, 1, D) and torch.equal(q[:, :, 0], want_q)
        assert torch.equal(kwin[:, :, ks], want_k) and torch.equal(vwin[:, :, vs], want_v)
        kbuf[:, :, 2 + ks] = 7.0
        vbuf[:, :, 1 + vs] = -7.0
        assert bool((kbuf == 7.0).all()) and bool((vbuf == -7.0).all())  # nothing else was written


def test_rope_append_slot_checks(dev):
    from kvmix_amd import ops

    qkv = torch.zeros(1, 1, 3 * 32, dtype=torch.float16, device=dev) + 1
    cs = torch.ones(32, dtype=torch.float16, device=dev)
    win = torch.zeros(1, 1, 4, 32, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):
        ops.rope_append(qkv, cs, cs, 1, 1, win, win.clone(), 4, 0)           # host slot outside the window
    far = torch.tensor([99], dtype=torch.int64, device=dev)
    k, v = win.clone(), win.clone()
    ops.rope_append(qkv, cs, cs, 1, 1, k, v, far, 1)                          # device slot outside: no write
    assert float(k.abs().sum()) == 0.0 and float(v[:, :, 1].sum()) == 32.0
    with pytest.raises(RuntimeError):
        ops.rope_append(qkv.float(), cs, cs, 1, 1, win, win, 0, 0)
    with pytest.raises(RuntimeError):
        ops.rope_append(qkv, cs[:16], cs, 1, 1, win, win, 0, 0)
