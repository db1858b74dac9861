"""An in-place, pre-allocated form of the reference's per-layer KV cache.

The reference keeps nine entries per layer (models/modeling_llama_KVmix.py:270-273) and grows
them with `torch.cat` on every append and every flush (:117-118,134-139,162-167), which copies
the whole packed cache each time.  `PackedKVCache` holds the same nine things in buffers
allocated once for a stated capacity; a flush quantizes the oldest tail tokens straight into
the packed buffers at the current write position (the quantizer takes output strides), so an
append costs O(new tokens).  `as_tuple()` hands out the reference's 9-tuple as views of those
buffers: same shapes, same contents bit for bit, no copies; the GEMV reads the views in place.

Flush policy: `flush_length` below, the reference's ratio rule or a fixed fp16 window.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops

# Residual ratio the reference's profiler assigns to each bit width (myprofileKV.py:75-80).
RESIDUAL_RATIO_BY_BITS = {4: 0.3, 3: 0.2, 2: 0.2, 1: 0.1}


def flush_length(tail_len: int, ratio: float, group: int, residual_length: Optional[int] = None,
                 prompt: bool = False) -> int:
    """Number of oldest tail tokens to quantize now.

    Ratio rule (models/modeling_llama_KVmix.py:119-127,152-155 and, for the prompt, :219-224):
    keep int(ratio * L) tokens in fp16, quantize the rest rounded down to a multiple of the group.
    Fixed window (residual_length = R): once the tail holds more than R tokens, flush the oldest
    floor(R/g)*g; for a prompt, everything but the newest R tokens, rounded down to a multiple of the
    group.  Under either rule the newest token stays in fp16 (the ratio rule keeps int(ratio * L) >= 1
    tokens whenever it flushes at all): what a decode step flushes are tokens of earlier steps, which is
    what lets the flushes of all layers of a step be issued together before its first layer runs
    (flush_ahead below)."""
    if residual_length is not None:
        if prompt:
            return (max(tail_len - residual_length, 0) // group) * group
        return (residual_length // group) * group if tail_len > residual_length else 0
    keep = int(ratio * tail_len)
    if tail_len > keep and keep >= 0:
        return ((tail_len - keep) // group) * group
    return 0


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


class _Tail:
    """fp16 tokens [B,Hkv,L,D] kept in a longer buffer: append at the end, drop from the front.
    The live region moves back to the front of the buffer only when the end is reached."""

    def __init__(self):
        self.buf: Optional[torch.Tensor] = None
        self.start = 0
        self.len = 0

    def view(self) -> Optional[torch.Tensor]:
        return None if self.buf is None else self.buf[:, :, self.start:self.start + self.len]

    def append(self, new: torch.Tensor, reserve: int) -> None:
        B, H, n, D = new.shape
        if self.buf is None:
            self.buf = torch.zeros((B, H, max(reserve, n), D), dtype=new.dtype, device=new.device)
        cap = self.buf.shape[2]
        if self.start + self.len + n > cap:
            live = self.view()
            if self.len + n > cap:  # the tail itself has outgrown the buffer: a longer one
                buf = torch.zeros((B, H, max(2 * cap, self.len + n), D), dtype=new.dtype, device=new.device)
                buf[:, :, :self.len].copy_(live)
                self.buf = buf
            else:  # room at the front: move the live tokens there (regions may overlap)
                self.buf[:, :, :self.len].copy_(live.clone())
            self.start = 0
        self.buf[:, :, self.start + self.len:self.start + self.len + n].copy_(new)
        self.len += n

    def drop_front(self, n: int) -> None:
        self.start += n
        self.len -= n

    def window(self, slots: int) -> torch.Tensor:
        """A fixed-size view [B,H,slots,D] that starts at the live region (which is moved to the front
        of the buffer first if the view would not fit): slots beyond the live tokens hold finite
        leftovers (the buffer starts out zeroed), never uninitialised memory."""
        if self.start + slots > self.buf.shape[2]:
            if slots > self.buf.shape[2]:
                raise RuntimeError("tail buffer shorter than the requested window")
            self.buf[:, :, :self.len].copy_(self.view().clone())
            self.start = 0
        return self.buf[:, :, self.start:self.start + slots]


class PackedKVCache:
    """One layer's KV cache, quantized part and fp16 tails, updated in place.

    capacity: quantized tokens the packed buffers hold before they have to be re-allocated
    (they then double, which copies once; give the longest context expected to avoid that).
    k_fmt / v_fmt: ops.FMT_REF (the reference's packing; 3-bit keys then use group 11) or
    ops.FMT_DENSE3 for 3 bits with group 32."""

    def __init__(self, k_bits: int, v_bits: int, group_size: int = 32, k_residual_ratio: Optional[float] = None,
                 v_residual_ratio: Optional[float] = None, residual_length: Optional[int] = None,
                 capacity: int = 4096, k_fmt: int = ops.FMT_REF, v_fmt: int = ops.FMT_REF):
        for bits in (k_bits, v_bits):
            if bits not in (1, 2, 3, 4):
                raise RuntimeError("Supported quantization bits: 1, 2, 3, 4")
        if v_bits == 3 and v_fmt == ops.FMT_REF:
            # head_dim would have to be a multiple of 11 (quantization_cuda.cu:649)
            raise RuntimeError("3-bit values need v_fmt=FMT_DENSE3 (the reference's 3-bit packing needs steps % 11 == 0)")
        self.k_bits, self.v_bits, self.k_fmt, self.v_fmt = k_bits, v_bits, k_fmt, v_fmt
        self.k_residual_ratio = RESIDUAL_RATIO_BY_BITS[k_bits] if k_residual_ratio is None else k_residual_ratio
        self.v_residual_ratio = RESIDUAL_RATIO_BY_BITS[v_bits] if v_residual_ratio is None else v_residual_ratio
        self.Vgroup_size = group_size
        self.Kgroup_size = 11 if (k_bits == 3 and k_fmt == ops.FMT_REF) else group_size  # llama:49-52
        self.residual_length = residual_length
        self.capacity = max(int(capacity), 1)
        self.kv_seq_len = 0
        self.k_tokens = 0  # quantized key tokens
        self.v_tokens = 0  # quantized value tokens
        self._k_tail, self._v_tail = _Tail(), _Tail()
        self._k: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None  # code, scale, min
        self._v: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None
        self._packed_views = (None,) * 6  # views of the quantized part, rebuilt after a flush
        self._flushed_ahead = False       # flush_ahead() has run the coming one-token append's flush

    # -- sizes -----------------------------------------------------------------------------
    def _words(self, n: int, bits: int, fmt: int) -> int:
        if bits == 3:
            return n * 3 // 32 if fmt == ops.FMT_DENSE3 else n // 11
        return n * bits // 32

    def _alloc_k(self, like: torch.Tensor, tokens: int):
        B, H, _, D = like.shape
        cap = _round_up(tokens, 32 * 11)
        code = torch.empty((B, H, D, self._words(cap, self.k_bits, self.k_fmt)), dtype=torch.int32, device=like.device)
        scale = torch.empty((B, H, D, cap // self.Kgroup_size), dtype=torch.float16, device=like.device)
        return code, scale, torch.empty_like(scale)

    def _alloc_v(self, like: torch.Tensor, tokens: int):
        B, H, _, D = like.shape
        code = torch.empty((B, H, tokens, self._words(D, self.v_bits, self.v_fmt)), dtype=torch.int32,
                           device=like.device)
        scale = torch.empty((B, H, tokens, D // self.Vgroup_size), dtype=torch.float16, device=like.device)
        return code, scale, torch.empty_like(scale)

    def _reserve(self, like: torch.Tensor, nk: int, nv: int) -> None:
        """Make room for nk more quantized key tokens and nv more value tokens."""
        if nk > 0:
            need = self.k_tokens + nk
            have = 0 if self._k is None else self._k[1].shape[3] * self.Kgroup_size
            if need > have:
                new = self._alloc_k(like, max(need, self.capacity, 2 * have))
                if self._k is not None:
                    w, g = self._words(self.k_tokens, self.k_bits, self.k_fmt), self.k_tokens // self.Kgroup_size
                    new[0][..., :w].copy_(self._k[0][..., :w])
                    new[1][..., :g].copy_(self._k[1][..., :g])
                    new[2][..., :g].copy_(self._k[2][..., :g])
                self._k = new
        if nv > 0:
            need = self.v_tokens + nv
            have = 0 if self._v is None else self._v[0].shape[2]
            if need > have:
                new = self._alloc_v(like, max(need, self.capacity, 2 * have))
                if self._v is not None:
                    for dst, src in zip(new, self._v):
                        dst[:, :, :self.v_tokens].copy_(src[:, :, :self.v_tokens])
                self._v = new

    # -- update ----------------------------------------------------------------------------
    def append(self, key_states: torch.Tensor, value_states: torch.Tensor, prompt: bool = False) -> None:
        """Add new tokens [B,Hkv,n,D] (fp16, after RoPE) and flush what the policy says.

        Same decisions and same packed bits as the reference's decode branch
        (models/modeling_llama_KVmix.py:117-167) and, with prompt=True, its prompt branch
        (:219-251)."""
        if key_states.dim() != 4 or value_states.shape != key_states.shape:
            raise RuntimeError("key_states and value_states must be 4-D and of equal shape")
        if key_states.dtype != torch.float16 or value_states.dtype != torch.float16:
            raise RuntimeError(f"expected scalar type Half but found {key_states.dtype}")
        if not key_states.is_cuda:
            raise RuntimeError("KVmix operators run on the GPU only: got a tensor on " + str(key_states.device))
        key_states, value_states = key_states.detach(), value_states.detach()  # the cache is not part of any autograd graph
        n = key_states.shape[2]
        steady = max((self.residual_length or 0) + self.Vgroup_size, 2 * self.Vgroup_size)  # a tail between two flushes
        # Many tokens onto empty tails (a prompt): what the policy flushes is quantized straight from
        # the incoming tensors and only the rest is kept in fp16, so the tails never hold the prompt.
        direct = n > 1 and self._k_tail.len == 0 and self._v_tail.len == 0
        if direct:
            nk = flush_length(n, self.k_residual_ratio, self.Kgroup_size, self.residual_length, prompt)
            nv = flush_length(n, self.v_residual_ratio, self.Vgroup_size, self.residual_length, prompt)
            reserve = max(steady, n - nk, n - nv) + 2 * self.Vgroup_size
            self._k_tail.append(key_states[:, :, nk:], reserve)
            self._v_tail.append(value_states[:, :, nv:], reserve)
        else:
            reserve = steady + 2 * self.Vgroup_size + n
            self._k_tail.append(key_states, reserve)
            self._v_tail.append(value_states, reserve)
            if self._flushed_ahead and n == 1:
                nk = nv = 0  # (flush_ahead has already run this step's flush)
            else:
                nk = flush_length(self._k_tail.len, self.k_residual_ratio, self.Kgroup_size, self.residual_length, prompt)
                nv = flush_length(self._v_tail.len, self.v_residual_ratio, self.Vgroup_size, self.residual_length, prompt)
        self._flushed_ahead = False
        self.kv_seq_len += n
        if nk == 0 and nv == 0:
            return
        self._reserve(key_states, nk, nv)
        ops.quantize_kv_flush_into(*self._flush_args(nk, nv, key_states if direct else None, value_states if direct else None))
        self._flush_done(nk, nv, direct)

    def _flush_args(self, nk: int, nv: int, k_src=None, v_src=None):
        """Arguments of ops.quantize_kv_flush_into for flushing nk key and nv value tokens into the packed buffers
        (already reserved) at the write position: from the front of the tails, or of k_src / v_src."""
        k_out = v_out = None
        k_chunk = v_chunk = None
        if nk > 0:
            w0, g0 = self._words(self.k_tokens, self.k_bits, self.k_fmt), self.k_tokens // self.Kgroup_size
            w1, g1 = self._words(self.k_tokens + nk, self.k_bits, self.k_fmt), (self.k_tokens + nk) // self.Kgroup_size
            k_out = (self._k[0][..., w0:w1], self._k[1][..., g0:g1], self._k[2][..., g0:g1])
            k_chunk = (k_src if k_src is not None else self._k_tail.view())[:, :, :nk]
        if nv > 0:
            v_out = tuple(t[:, :, self.v_tokens:self.v_tokens + nv] for t in self._v)
            v_chunk = (v_src if v_src is not None else self._v_tail.view())[:, :, :nv]
        return (k_chunk, self.Kgroup_size, self.k_bits, k_out, v_chunk, self.Vgroup_size, self.v_bits, v_out,
                self.k_fmt, self.v_fmt)

    def _flush_done(self, nk: int, nv: int, direct: bool) -> None:
        if not direct:
            self._k_tail.drop_front(nk)
            self._v_tail.drop_front(nv)
        self.k_tokens += nk
        self.v_tokens += nv
        kc = ks = km = vc = vs = vm = None
        if self.k_tokens > 0:
            w, g = self._words(self.k_tokens, self.k_bits, self.k_fmt), self.k_tokens // self.Kgroup_size
            kc, ks, km = self._k[0][..., :w], self._k[1][..., :g], self._k[2][..., :g]
        if self.v_tokens > 0:
            vc, vs, vm = (t[:, :, :self.v_tokens] for t in self._v)
        self._packed_views = (kc, ks, km, vc, vs, vm)

    # -- hooks for a decode step replayed from a captured graph --------------------------------
    def flushes_on_next_append(self) -> bool:
        """Would appending one token make either tail flush?"""
        if self._flushed_ahead:
            return False  # (flush_ahead has run it)
        nk = flush_length(self._k_tail.len + 1, self.k_residual_ratio, self.Kgroup_size, self.residual_length)
        nv = flush_length(self._v_tail.len + 1, self.v_residual_ratio, self.Vgroup_size, self.residual_length)
        return nk > 0 or nv > 0

    def tail_windows(self, slots: int):
        """(key window, value window, live key tokens, live value tokens): fixed-size views of the
        fp16 tails for a step whose append is done by the caller on the device (the token goes to
        slot `live tokens` of each window); follow every such step with note_device_append()."""
        return self._k_tail.window(slots), self._v_tail.window(slots), self._k_tail.len, self._v_tail.len

    def note_device_append(self) -> None:
        """Book-keeping for one token that a device-side step wrote into the tail windows."""
        self._k_tail.len += 1
        self._v_tail.len += 1
        self.kv_seq_len += 1
        self._flushed_ahead = False

    def reset(self) -> None:
        """Forget every token; the buffers stay allocated and are reused by the next prompt."""
        self.kv_seq_len = self.k_tokens = self.v_tokens = 0
        for tail in (self._k_tail, self._v_tail):
            tail.start = tail.len = 0
            if tail.buf is not None:
                tail.buf.zero_()  # window() relies on slots past the live length reading as zero
        self._packed_views = (None,) * 6
        self._flushed_ahead = False

    # -- views -----------------------------------------------------------------------------
    def as_tuple(self) -> Tuple:
        """The reference's 9-tuple (models/modeling_llama_KVmix.py:270-273) as views of the
        buffers; packed entries are None until the first flush, as in the reference."""
        kc, ks, km, vc, vs, vm = self._packed_views
        return (kc, self._k_tail.view(), ks, km, vc, self._v_tail.view(), vs, vm, self.kv_seq_len)

    def __getitem__(self, i):  # the model reads past_key_values[layer][-1] for the length (llama:428,646)
        return self.as_tuple()[i]

    def __len__(self) -> int:
        return 9


def flush_ahead(caches) -> int:
    """Run now, batched over the caches (kvmix_quant_pack_kv_flush_batch: eight to a launch), the flush that the
    next ONE-token append of each of them would run, and mark those appends as flushed.  Call it right before a
    decode step: what a layer flushes in a step are the oldest tokens of its tails, tokens of earlier steps
    (models/modeling_llama_KVmix.py:122-127,152-156: `[:, :, :to_quantize_length]`), and how many follows from the
    tails' lengths alone, so nothing of the step itself is needed -- and the packed bits, the tails and every later
    decision are those of flushing inside the appends (a cache whose rule would take the coming token itself is left
    to its append).  Returns the number of caches flushed."""
    todo = []
    for c in caches:
        if not isinstance(c, PackedKVCache) or c._k_tail.buf is None or c._flushed_ahead:
            continue
        nk = flush_length(c._k_tail.len + 1, c.k_residual_ratio, c.Kgroup_size, c.residual_length)
        nv = flush_length(c._v_tail.len + 1, c.v_residual_ratio, c.Vgroup_size, c.residual_length)
        if (nk == 0 and nv == 0) or nk > c._k_tail.len or nv > c._v_tail.len:
            continue
        c._reserve(c._k_tail.buf, nk, nv)
        todo.append((c, nk, nv))
    if todo:
        ops.quantize_kv_flush_batch([c._flush_args(nk, nv) for c, nk, nv in todo])
        for c, nk, nv in todo:
            c._flush_done(nk, nv, direct=False)
            c._flushed_ahead = True
    return len(todo)
