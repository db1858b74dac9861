"""Host logic of the in-place cache that needs no GPU: the flush policy against hand-worked cases
of the reference's rule (models/modeling_llama_KVmix.py:119-127,152-155,219-224) and the tail
buffer's append / drop / compaction bookkeeping."""
import numpy as np
import pytest
import torch

from kvmix_amd.cache import PackedKVCache, _Tail, flush_length


def test_ratio_rule_hand_worked():
    # L = 39, ratio 0.2: keep int(7.8) = 7, quantize floor(32 / 32) * 32 = 32
    assert flush_length(39, 0.2, 32) == 32
    assert flush_length(38, 0.2, 32) == 0      # keep 7, 31 left: below one group
    assert flush_length(416 + 1, 0.2, 32) == 320  # first decode step after a 2080-token prompt keeps 83
    assert flush_length(300, 0.2, 11) == 231   # keep 60, 240 // 11 * 11
    assert flush_length(0, 0.2, 32) == 0
    assert flush_length(5, 1.0, 32) == 0       # keep everything


def test_fixed_window_rule():
    assert flush_length(128, 0.0, 32, residual_length=128) == 0
    assert flush_length(129, 0.0, 32, residual_length=128) == 128   # the newest token stays in fp16
    assert flush_length(129, 0.0, 11, residual_length=129) == 0
    assert flush_length(130, 0.0, 11, residual_length=129) == 121
    assert flush_length(1000, 0.0, 32, residual_length=128, prompt=True) == 864  # (1000 - 128) // 32 * 32
    assert flush_length(100, 0.0, 32, residual_length=128, prompt=True) == 0


def test_oracle_policy_is_the_same_rule(oracle):
    for L in range(0, 200):
        for ratio in (0.1, 0.2, 0.3):
            for g in (11, 32):
                assert flush_length(L, ratio, g) == oracle.flush_length(L, ratio, g)


def test_tail_buffer_bookkeeping():
    """Appends and front drops against a plain list of tokens, through wrap-around and growth."""
    rng = np.random.default_rng(0)
    tail, want = _Tail(), []
    caps = set()
    for step in range(400):
        n = 1 if step % 50 else 37
        new = torch.from_numpy(rng.standard_normal((2, 3, n, 8)).astype(np.float16))
        tail.append(new, reserve=16)
        want += [new[:, :, i] for i in range(n)]
        if len(want) >= 24 and step % 3 == 0:
            drop = 16 if step % 7 else len(want)
            tail.drop_front(drop)
            want = want[drop:]
        got = tail.view()
        assert got.shape[2] == len(want) == tail.len
        if want:
            assert torch.equal(got, torch.stack(want, 2))
        caps.add(tail.buf.shape[2])
    assert len(caps) > 1  # the buffer did grow at least once
    assert tail.start + tail.len <= tail.buf.shape[2]


def test_empty_cache_views():
    c = PackedKVCache(4, 2)
    assert c.as_tuple() == (None,) * 8 + (0,)
    assert c[-1] == 0 and len(c) == 9
    assert c.Kgroup_size == 32 and PackedKVCache(3, 2).Kgroup_size == 11
    with pytest.raises(RuntimeError, match="GPU only"):
        x = torch.zeros(1, 1, 1, 128, dtype=torch.float16)
        c.append(x, x)
