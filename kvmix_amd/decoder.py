"""A plain Llama-shaped decoder stack around the KV-cache path, for the end-to-end decode
measurement (random-init Llama-2-7B shape, greedy decoding) and its parity test.

Only what the measurement needs: token embedding, per layer RMSNorm -> q/k/v projections -> RoPE
-> the attention step over the quantized cache -> output projection -> SwiGLU MLP, final norm,
LM head.  It stands where LlamaDecoderLayer_KVmix / LlamaModel_KVmix stand in the reference
(models/modeling_llama_KVmix.py:286-370, 373-543); the attention step itself is the `attention`
object of each layer (kvmix_amd.attention.KVmixAttention on the GPU), called with the same
arguments the reference's attention forward receives after RoPE (:103-105).
Weights are plain tensors; there is no checkpoint loading and no tokenizer here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence

import torch
import torch.nn.functional as F


@dataclass
class DecoderConfig:
    """Llama-2-7B by default."""
    hidden_size: int = 4096
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 32
    intermediate_size: int = 11008
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_heads


def init_weights(cfg: DecoderConfig, device, dtype=torch.float16, std: float = 0.02, seed: int = 4) -> dict:
    """Random weights ~N(0, std) (norm weights = 1), generated on `device` from `seed`."""
    gen = torch.Generator(device=device).manual_seed(seed)

    def w(*shape):
        return (torch.randn(*shape, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)

    h, kvh = cfg.hidden_size, cfg.num_kv_heads * cfg.head_dim
    layers = []
    for _ in range(cfg.num_layers):
        layers.append({
            "input_norm": torch.ones(h, device=device, dtype=dtype),
            # q, k and v projections stacked into one matrix (rows: q heads, k heads, v heads), and
            # gate over up likewise: a single-token step is bound by kernel count and weight streaming
            "wqkv": w(h + 2 * kvh, h), "wo": w(h, h),
            "post_norm": torch.ones(h, device=device, dtype=dtype),
            "w_gate_up": w(2 * cfg.intermediate_size, h),
            "w_down": w(h, cfg.intermediate_size),
        })
    return {"embed": w(cfg.vocab_size, h), "layers": layers, "norm": torch.ones(h, device=device, dtype=dtype),
            "lm_head": w(cfg.vocab_size, h)}


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS normalisation over the last dimension (one library kernel)."""
    return F.rms_norm(x, (x.shape[-1],), weight, eps)


def project_qkv(cfg: DecoderConfig, h: torch.Tensor, wqkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """h [B,Q,hidden] -> q [B,nh,Q,D], k, v [B,nkv,Q,D] with RoPE applied to q and k (one pass over both)."""
    B, Q, _ = h.shape
    nh, nkv = cfg.num_heads, cfg.num_kv_heads
    qkv = F.linear(h, wqkv).view(B, Q, nh + 2 * nkv, cfg.head_dim).transpose(1, 2)
    qk = apply_rope(qkv[:, :nh + nkv], cos, sin)
    return qk[:, :nh], qk[:, nh:], qkv[:, nh + nkv:]


def mlp(h: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    gu = F.linear(h, w_gate_up)
    half = gu.shape[-1] // 2
    return F.linear(F.silu(gu[..., :half]) * gu[..., half:], w_down)


def rope_tables(cfg: DecoderConfig, positions: torch.Tensor, dtype) -> tuple:
    """cos/sin [1,1,Q,D] for integer positions [Q] (rotate-half convention, fp32 angles)."""
    D = cfg.head_dim
    inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, device=positions.device, dtype=torch.float32) / D))
    ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos()[None, None].to(dtype), emb.sin()[None, None].to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos + rot * sin


class Decoder:
    """weights: the dict of init_weights; attention: one callable per layer with the signature
    attention(q [B,nh,Q,D], k [B,nkv,Q,D], v [B,nkv,Q,D], cache, attention_mask=..., need_weights=False) ->
    (out [B,nh,Q,D], attn_weights or None, cache);  caches: the per-layer cache objects to start from
    (None = the reference's "no past" prompt call)."""

    def __init__(self, cfg: DecoderConfig, weights: dict, attention: Sequence[Callable],
                 caches: Optional[List] = None):
        self.cfg, self.w, self.attention = cfg, weights, list(attention)
        self.caches: List = list(caches) if caches is not None else [None] * cfg.num_layers
        self.position = 0

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [B,Q] (prompt when nothing is cached yet, else the new tokens) -> logits of the
        last position [B, vocab] in fp32."""
        cfg = self.cfg
        B, Q = input_ids.shape
        x = self.w["embed"][input_ids]
        pos = torch.arange(self.position, self.position + Q, device=x.device)
        cos, sin = rope_tables(cfg, pos, x.dtype)
        mask = None
        if Q > 1:  # causal mask of the prompt, as the model builds it: 0 / dtype-min, fp32 logits
            mask = torch.full((Q, Q), torch.finfo(torch.float32).min, device=x.device, dtype=torch.float32)
            mask = torch.triu(mask, 1)[None, None]
        if Q == 1:
            # what the layers would flush in this step are tokens of earlier steps: all layers' flushes in one
            # batched launch sequence, before the first layer runs (in-place caches; others flush in their append)
            from .cache import flush_ahead

            flush_ahead(self.caches)
        for li, lw in enumerate(self.w["layers"]):
            h = rms_norm(x, lw["input_norm"], cfg.rms_norm_eps)
            q, k, v = project_qkv(cfg, h, lw["wqkv"], cos, sin)
            out, _, self.caches[li] = self.attention[li](q, k, v, self.caches[li], attention_mask=mask, need_weights=False)
            out = out.transpose(1, 2).reshape(B, Q, cfg.hidden_size)
            x = x + F.linear(out, lw["wo"])
            h = rms_norm(x, lw["post_norm"], cfg.rms_norm_eps)
            x = x + mlp(h, lw["w_gate_up"], lw["w_down"])
        self.position += Q
        x = rms_norm(x[:, -1], self.w["norm"], cfg.rms_norm_eps)
        return F.linear(x, self.w["lm_head"]).to(torch.float32)

    def generate(self, prompt_ids: torch.Tensor, new_tokens: int, on_step: Optional[Callable] = None) -> torch.Tensor:
        """Greedy decoding: returns the new token ids [B, new_tokens].  on_step(step, logits) is
        called after every forward (step 0 = the prompt)."""
        logits = self.forward(prompt_ids)
        if on_step is not None:
            on_step(0, logits)
        out = []
        for step in range(1, new_tokens + 1):
            nxt = logits.argmax(-1, keepdim=True)
            out.append(nxt)
            if step == new_tokens:
                break
            logits = self.forward(nxt)
            if on_step is not None:
                on_step(step, logits)
        return torch.cat(out, dim=1)


class GraphDecoder(Decoder):
    """Decoder whose single-token steps are replayed from a captured HIP graph.

    A decode step launches about forty small kernels per layer, so an eager host loop is bound by
    launch overhead, not by the GPU.  Between two flushes everything about a step is static except
    three numbers (the position and the lengths of the two fp16 tails); those live in device
    counters that the graph itself increments, the new token goes to slot `tail length` of a
    fixed-size tail window through an indexed copy, and the attention step reads the tail lengths
    from the counters, so that the window's unused slots get probability zero.  Before a step in which layers flush, the flushes of all
    layers are run at once (cache.flush_ahead: they take tokens of earlier steps only); the flush changes the packed
    lengths, which are launch arguments, so that step is captured anew and replayed like the others.
    Needs in-place caches (PackedKVCache) that all follow the same kind of flush policy: one fixed residual window,
    or the reference's ratio rule (models/modeling_llama_KVmix.py:119-127,152-155: residual_length None) -- there the
    tails stay short (a flush every group / (1 - ratio) tokens per layer, every 14 tokens with the reference's
    3-bit keys), so a graph lives for fewer steps and the window is sized at every capture."""

    def __init__(self, cfg: DecoderConfig, weights: dict, attention: Sequence, caches: List):
        super().__init__(cfg, weights, attention, caches)
        windows = {c.residual_length for c in caches}
        if len(windows) != 1:
            raise RuntimeError("GraphDecoder needs in-place caches that share one flush policy: one fixed residual "
                               "window, or the ratio rule for all")
        self.window = windows.pop()   # None: the ratio rule, the window is set at every capture
        self._graph = None
        self._stale = True
        self._warm = False
        self._ids = self._logits = None
        self._pos = self._len = None
        self._counters = {}
        self.graph_steps = self.eager_steps = self.captures = self.flush_steps = 0

    # one decode step with static shapes; mutates the device counters
    def _static_step(self, ids: torch.Tensor) -> torch.Tensor:
        from . import ops

        cfg, R = self.cfg, self.window
        B = ids.shape[0]
        dev = ids.device
        x = self.w["embed"][ids]
        D = cfg.head_dim
        inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
        ang = self._pos.to(torch.float32)[:, None] * inv_freq[None, :]
        emb = torch.cat([ang, ang], dim=-1)
        cos, sin = emb.cos()[None, None].to(x.dtype), emb.sin()[None, None].to(x.dtype)
        for li, lw in enumerate(self.w["layers"]):
            cache = self.caches[li]
            h = rms_norm(x, lw["input_norm"], cfg.rms_norm_eps)
            kwin, vwin, _, _ = cache.tail_windows(R)
            (kslot, klive), (vslot, vlive) = self._len[li]
            # rotary embedding of q and k and the append of k and v to the tail windows: one launch
            q = ops.rope_append(F.linear(h, lw["wqkv"]), cos, sin, cfg.num_heads, cfg.num_kv_heads, kwin, vwin, kslot, vslot)
            kc, _, ks, km, vc, _, vs, vm, _ = cache.as_tuple()
            width = max(cache.k_tokens, cache.v_tokens) + R
            single = ops.prefer_single_pass(B, cfg.num_heads, cfg.num_kv_heads, D, width, cache.k_bits, cache.k_fmt,
                                            cache.Kgroup_size, cache.v_bits, cache.v_fmt, cache.Vgroup_size,
                                            k_tokens=cache.k_tokens, v_tokens=cache.v_tokens)
            out, _ = ops.decode_attention(q, (kc, ks, km), (vc, vs, vm), kwin, vwin, cache.Kgroup_size, cache.k_bits,
                                          cache.Vgroup_size, cache.v_bits, cache.k_fmt, cache.v_fmt,
                                          k_tail_len=klive, v_tail_len=vlive, single_pass=single)
            out = out.transpose(1, 2).reshape(B, 1, cfg.hidden_size)
            x = x + F.linear(out, lw["wo"])
            h = rms_norm(x, lw["post_norm"], cfg.rms_norm_eps)
            x = x + mlp(h, lw["w_gate_up"], lw["w_down"])
        self._pos.add_(1)
        for slot, live in self._counters.values():
            slot.add_(1)
            live.add_(1)
        x = rms_norm(x[:, -1], self.w["norm"], cfg.rms_norm_eps)
        return F.linear(x, self.w["lm_head"]).to(torch.float32)

    def _sync_counters(self) -> None:
        """Device counters for the coming steps.  Tails of equal length stay equal until the next
        flush, so they share one pair of counters (slot of the next token, live slots once it is
        written): a step then increments a handful of counters instead of two per layer."""
        dev = self._pos.device
        self._pos.fill_(self.position)
        lengths = []
        for cache in self.caches:
            _, _, nk, nv = cache.tail_windows(self.window)
            lengths.append((nk, nv))
        for n in {n for pair in lengths for n in pair}:
            if n not in self._counters:
                self._counters[n] = (torch.empty(1, dtype=torch.int64, device=dev), torch.empty(1, dtype=torch.int64, device=dev))
        self._counters = {n: c for n, c in self._counters.items() if any(n in pair for pair in lengths)}
        for n, (slot, live) in self._counters.items():
            slot.fill_(n)
            live.fill_(n + 1)
        self._len = [(self._counters[nk], self._counters[nv]) for nk, nv in lengths]

    def _ratio_window(self) -> int:
        """Slots the tail windows need until the next flush under the ratio rule: every tail grows one token a
        step until the first length at which its rule flushes; that step runs eagerly, so the replayed steps
        write slots below it.  (A multiple of 8, so that windows change less often between captures.)"""
        from .cache import flush_length

        need = 1
        for c in self.caches:
            for tail, ratio, group in ((c._k_tail, c.k_residual_ratio, c.Kgroup_size), (c._v_tail, c.v_residual_ratio, c.Vgroup_size)):
                n = tail.len + 1
                while flush_length(n, ratio, group) == 0:
                    n += 1
                need = max(need, n)
        return (need + 7) // 8 * 8

    def _capture(self, ids: torch.Tensor) -> None:
        dev = ids.device
        if self._ids is None:
            self._ids = torch.zeros_like(ids)
            self._pos = torch.zeros(1, dtype=torch.int64, device=dev)
        self._ids.copy_(ids)
        if self.caches[0].residual_length is None:
            self.window = self._ratio_window()
        self._sync_counters()  # (also settles where the tail windows lie before anything is recorded)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            if not self._warm:
                # once: let the libraries set themselves up outside a capture; the step's writes go to
                # the slots the real step will overwrite, and the counters are set back afterwards
                self._static_step(self._ids)
                self._sync_counters()
                self._warm = True
            self._graph = None  # release the previous graph's memory first
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                self._logits = self._static_step(self._ids)
        torch.cuda.current_stream(dev).wait_stream(side)
        self._graph = graph
        self._stale = False
        self.captures += 1

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        if input_ids.shape[1] == 1 and self.position > 0 and any(c.flushes_on_next_append() for c in self.caches):
            # a step in which layers flush: the flushes of all layers now, batched (they take tokens of earlier
            # steps only); the packed lengths have changed, so the step is captured anew
            from .cache import flush_ahead

            flush_ahead(self.caches)
            self._stale = True
            self.flush_steps += 1
        if input_ids.shape[1] != 1 or self.position == 0 or any(c.flushes_on_next_append() for c in self.caches):
            # (a prompt, or a cache whose rule takes the coming token itself: the eager loop)
            self._stale = True
            self.eager_steps += 1
            return super().forward(input_ids)
        if self._stale:
            self._capture(input_ids)
        else:
            self._ids.copy_(input_ids)
        self._graph.replay()
        for cache in self.caches:
            cache.note_device_append()
        self.position += 1
        self.graph_steps += 1
        return self._logits.clone()


def kvmix_layers(cfg: DecoderConfig, k_bits: Sequence[int], v_bits: Sequence[int], residual_length: Optional[int] = 128,
                 group_size: int = 32, capacity: int = 4096):
    """Per-layer KVmixAttention objects and in-place caches for mixed per-layer bit widths.
    3-bit keys use the reference's 11-per-word format, 3-bit values the dense stream (the
    reference's 3-bit packing cannot hold head_dim 128)."""
    from . import ops
    from .attention import KVmixAttention

    atts = [KVmixAttention(kb, vb, group_size=group_size, residual_length=residual_length)
            for kb, vb in zip(k_bits, v_bits)]
    caches = [a.new_cache(capacity, v_fmt=ops.FMT_DENSE3 if a.v_bits == 3 else ops.FMT_REF) for a in atts]
    return atts, caches


__all__ = ["DecoderConfig", "Decoder", "GraphDecoder", "init_weights", "kvmix_layers", "rms_norm", "rope_tables", "apply_rope"]
