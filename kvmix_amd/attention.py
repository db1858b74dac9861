"""Host-side mirror of the reference's attention glue around the KVmix operators.

`KVmixAttention.forward` reproduces what `LlamaAttention_KVmix.forward`
(models/modeling_llama_KVmix.py:105-283) and `MistralAttention_KVmix.forward`
(models/modeling_mistral_KVmix.py:150-329) do between RoPE and the output projection:
append to the fp16 tails, flush the oldest tail tokens through the quantizer, q.K^T over the
packed keys + fp16 tail, fp32 softmax, p.V over the packed values + fp16 tail, and hand back the
reference's 9-entry cache tuple

    (Kcode [B,Hkv,D,Tqk/vpw] i32, K_tail [B,Hkv,Lk,D] f16, Kscale [B,Hkv,D,Tqk/g] f16, Kmin,
     Vcode [B,Hkv,Tqv,D/vpw] i32, V_tail [B,Hkv,Lv,D] f16, Vscale [B,Hkv,Tqv,D/g] f16, Vmin, kv_seq_len)

Projections, RoPE and the decoder stack belong to the model and are not part of this module.
Differences from the reference, all of them copies it makes and this does not:
GQA operands go to `quantized_gemm` un-repeated (the kernel maps query head h to kv head
h // n_rep; the reference materialises n_rep copies, models/modeling_llama_KVmix.py:176-178),
and the fp16 tail is multiplied through a grouped view instead of a repeated tensor.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import ops
from .cache import RESIDUAL_RATIO_BY_BITS, PackedKVCache, flush_length  # noqa: F401 (re-exported)


# longest fp16 tail for which a decode step goes through the library's fused step (one block per
# (batch, head) walks the tail; measured faster than torch's composition up to a few thousand tokens)
LIBRARY_STEP_MAX_TAIL = 16384


def repeat_kv_quant(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """models/modeling_llama_KVmix.py:19-28 (kept for callers that still want the copy)."""
    batch, num_key_value_heads, slen, head_dim = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    hidden_states = hidden_states[:, :, None, :, :].expand(batch, num_key_value_heads, n_rep, slen, head_dim)
    return hidden_states.reshape(batch, num_key_value_heads * n_rep, slen, head_dim)


def _cat(old: Optional[torch.Tensor], new: torch.Tensor, dim: int) -> torch.Tensor:
    return new if old is None else torch.cat([old, new], dim=dim)


def _grouped_matmul_qk(q: torch.Tensor, k_tail: torch.Tensor, n_rep: int) -> torch.Tensor:
    """q [B,nh,Q,D] x k_tail [B,Hkv,L,D]^T -> [B,nh,Q,L] without repeating k_tail."""
    B, nh, Q, D = q.shape
    Hkv, L = k_tail.shape[1], k_tail.shape[2]
    if n_rep == 1:
        return torch.matmul(q, k_tail.transpose(2, 3))
    out = torch.matmul(q.reshape(B, Hkv, n_rep * Q, D), k_tail.transpose(2, 3))
    return out.reshape(B, nh, Q, L)


def _grouped_matmul_pv(p: torch.Tensor, v_tail: torch.Tensor, n_rep: int) -> torch.Tensor:
    """p [B,nh,Q,L] x v_tail [B,Hkv,L,D] -> [B,nh,Q,D] without repeating v_tail."""
    B, nh, Q, L = p.shape
    Hkv, D = v_tail.shape[1], v_tail.shape[3]
    if n_rep == 1:
        return torch.matmul(p, v_tail)
    out = torch.matmul(p.reshape(B, Hkv, n_rep * Q, L), v_tail)
    return out.reshape(B, nh, Q, D)


class KVmixAttention:
    """The KV-cache part of one attention layer (no weights)."""

    def __init__(self, k_bits: int, v_bits: int, k_residual_ratio: Optional[float] = None,
                 v_residual_ratio: Optional[float] = None, group_size: int = 32,
                 residual_length: Optional[int] = None):
        self.k_bits, self.v_bits = k_bits, v_bits
        self.k_residual_ratio = RESIDUAL_RATIO_BY_BITS[k_bits] if k_residual_ratio is None else k_residual_ratio
        self.v_residual_ratio = RESIDUAL_RATIO_BY_BITS[v_bits] if v_residual_ratio is None else v_residual_ratio
        self.Vgroup_size = group_size
        self.Kgroup_size = 11 if k_bits == 3 else group_size  # models/modeling_llama_KVmix.py:49-52
        self.residual_length = residual_length

    # -- flush helpers ---------------------------------------------------------------------
    def _flush(self, k_tail, kq, v_tail, vq, prompt=False):
        """Quantize the oldest tokens of both tails.  kq / vq = (code, scale, min) so far (or Nones).
        When both tails flush in the same step the two quantizers run as one launch."""
        nk = flush_length(k_tail.shape[-2], self.k_residual_ratio, self.Kgroup_size, self.residual_length, prompt)
        nv = flush_length(v_tail.shape[-2], self.v_residual_ratio, self.Vgroup_size, self.residual_length, prompt)
        kc = vc = None
        if nk > 0 and nv > 0 and k_tail.dtype == torch.float16 and v_tail.shape[-1] % self.Vgroup_size == 0:
            kc, ks, km, vc, vs, vm = ops.quantize_kv_flush(k_tail[:, :, :nk, :], self.Kgroup_size, self.k_bits,
                                                           v_tail[:, :, :nv, :], self.Vgroup_size, self.v_bits)
        else:
            if nk > 0:
                kc, ks, km = ops.quantize_pack_last_dim_cuda(k_tail[:, :, :nk, :].transpose(2, 3).contiguous(),
                                                             self.Kgroup_size, self.k_bits)
            if nv > 0:
                vc, vs, vm = ops.quantize_pack_last_dim_cuda(v_tail[:, :, :nv, :].contiguous(), self.Vgroup_size,
                                                             self.v_bits)
        if kc is not None:
            k_tail = k_tail[:, :, nk:, :]
            kq = (_cat(kq[0], kc, 3), _cat(kq[1], ks, 3), _cat(kq[2], km, 3))
        if vc is not None:
            v_tail = v_tail[:, :, nv:, :]
            vq = (_cat(vq[0], vc, 2), _cat(vq[1], vs, 2), _cat(vq[2], vm, 2))
        return k_tail, kq, v_tail, vq

    def new_cache(self, capacity: int = 4096, k_fmt: int = ops.FMT_REF, v_fmt: int = ops.FMT_REF) -> PackedKVCache:
        """An empty in-place cache with this layer's bit widths and flush policy; pass it as
        past_key_value from the prompt on (the same object comes back, updated)."""
        return PackedKVCache(self.k_bits, self.v_bits, self.Vgroup_size, self.k_residual_ratio,
                             self.v_residual_ratio, self.residual_length, capacity, k_fmt, v_fmt)

    def _decode_with_torch_glue(self, query_states, kc, ks, km, k_tail, vc, vs, vm, v_tail, k_group, k_fmt, v_fmt, n_rep,
                                attention_mask):
        """The decode branch composed as the reference composes it (models/modeling_llama_KVmix.py:180-211):
        two quantized_gemm calls around torch's matmul / cat / softmax.  Used for several query
        positions at once and for masks or dtypes the library's fused step does not take."""
        D = query_states.shape[-1]
        att_full = _grouped_matmul_qk(query_states, k_tail, n_rep)
        if kc is not None:
            att_quant = ops.quantized_gemm(k_group, query_states, kc, ks, km, self.k_bits, k_fmt)
            attn_weights = torch.cat([att_quant.to(torch.float32), att_full.to(torch.float32)], dim=-1)
        else:
            attn_weights = att_full.to(torch.float32)
        attn_weights = attn_weights / math.sqrt(D)
        if attention_mask is not None:
            if attention_mask.shape[-2:] != attn_weights.shape[-2:]:
                raise ValueError(f"Attention mask shape {attention_mask.shape} does not match weights shape "
                                 f"{attn_weights.shape}")
            attn_weights = attn_weights + attention_mask
            attn_weights = torch.clamp(attn_weights, min=torch.finfo(attn_weights.dtype).min)
        attn_weights = F.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query_states.dtype)

        if vc is None:
            attn_output = _grouped_matmul_pv(attn_weights, v_tail, n_rep)
        else:
            lv = v_tail.shape[-2]
            tq = attn_weights.shape[-1] - lv
            out_quant = ops.quantized_gemm(self.Vgroup_size, attn_weights[..., :tq], vc, vs, vm, self.v_bits, v_fmt)
            out_full = _grouped_matmul_pv(attn_weights[..., tq:], v_tail, n_rep)
            attn_output = out_quant + out_full
        return attn_output, attn_weights

    # -- the step --------------------------------------------------------------------------
    def forward(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                past_key_value=None, attention_mask: Optional[torch.Tensor] = None, use_cache: bool = True,
                need_weights: bool = True):
        """query_states [B,nh,Q,D], key/value_states [B,Hkv,Q,D] (fp16, after RoPE).
        past_key_value: None (prompt), the reference's 9-tuple (a new tuple is returned, grown by
        concatenation as the reference does), or a PackedKVCache (updated in place and returned;
        an empty one means prompt).
        need_weights=False lets a single-token step run as one pass over the positions where that
        is the faster form; no probabilities exist then and attn_weights is None (the output differs
        from the other form by the reference's roundings after the softmax, about 2^-10 of the
        largest value).
        Returns (attn_output [B,nh,Q,D] fp16, attn_weights fp16 or None, past_key_value or None)."""
        B, nh, q_len, D = query_states.shape
        n_rep = nh // key_states.shape[1]
        inplace = past_key_value if isinstance(past_key_value, PackedKVCache) else None
        prompt = past_key_value is None or (inplace is not None and inplace.kv_seq_len == 0)
        k_fmt = inplace.k_fmt if inplace is not None else ops.FMT_REF
        v_fmt = inplace.v_fmt if inplace is not None else ops.FMT_REF
        k_group = inplace.Kgroup_size if inplace is not None else self.Kgroup_size

        if not prompt:
            if inplace is not None:
                inplace.append(key_states, value_states)
                kc, k_tail, ks, km, vc, v_tail, vs, vm, kv_seq_len = inplace.as_tuple()
            else:
                kv_seq_len = key_states.shape[-2] + past_key_value[-1]
                kc, k_tail, ks, km, vc, v_tail, vs, vm, _ = past_key_value
                k_tail = key_states if k_tail is None else torch.cat([k_tail, key_states], dim=2)
                v_tail = value_states if v_tail is None else torch.cat([v_tail, value_states], dim=2)
                k_tail, (kc, ks, km), v_tail, (vc, vs, vm) = self._flush(k_tail, (kc, ks, km), v_tail, (vc, vs, vm))

            mask_ok = attention_mask is None or (attention_mask.dtype == torch.float32 and attention_mask.dim() == 4
                                                 and attention_mask.shape[1] == 1)
            short_tails = max(k_tail.shape[2], v_tail.shape[2]) <= LIBRARY_STEP_MAX_TAIL
            if q_len == 1 and query_states.dtype == torch.float16 and D % 8 == 0 and mask_ok and short_tails:
                # the whole step in the library: logits over packed keys and fp16 tail, softmax,
                # output over packed values and fp16 tail
                if attention_mask is not None and attention_mask.shape[-2:] != (1, kv_seq_len):
                    raise ValueError(f"Attention mask shape {attention_mask.shape} does not match weights shape "
                                     f"{(B, nh, 1, kv_seq_len)}")
                single = (not need_weights) and ops.prefer_single_pass(
                    B, nh, key_states.shape[1], D, kv_seq_len, self.k_bits, k_fmt, k_group, self.v_bits, v_fmt,
                    self.Vgroup_size, k_tokens=kv_seq_len - k_tail.shape[2], v_tokens=kv_seq_len - v_tail.shape[2])
                attn_output, attn_weights = ops.decode_attention(
                    query_states, (kc, ks, km), (vc, vs, vm), k_tail, v_tail, k_group, self.k_bits, self.Vgroup_size,
                    self.v_bits, k_fmt, v_fmt, attention_mask, single_pass=single)
            else:
                attn_output, attn_weights = self._decode_with_torch_glue(
                    query_states, kc, ks, km, k_tail, vc, vs, vm, v_tail, k_group, k_fmt, v_fmt, n_rep, attention_mask)
        else:
            # prompt: dense fp16 attention; the cache keeps the oldest tokens quantized
            # (models/modeling_llama_KVmix.py:213-266)
            kv_seq_len = key_states.shape[-2]
            if inplace is not None:
                if use_cache:
                    inplace.append(key_states, value_states, prompt=True)
            elif use_cache:
                k_tail, (kc, ks, km), v_tail, (vc, vs, vm) = self._flush(key_states, (None,) * 3, value_states,
                                                                         (None,) * 3, prompt=True)
                k_tail, v_tail = k_tail.contiguous(), v_tail.contiguous()
            if not need_weights and query_states.dtype == torch.float16 and query_states.is_cuda:
                # nobody reads the probabilities: torch's fused attention, which never holds the
                # [Q, Q] matrix (fp32 accumulation throughout, where the composition below rounds the
                # logits and the probabilities to fp16)
                mask16 = None
                if attention_mask is not None:
                    if attention_mask.shape[-2:] != (q_len, kv_seq_len):
                        raise ValueError(f"Attention mask shape {attention_mask.shape} does not match weights shape "
                                         f"{(B, nh, q_len, kv_seq_len)}")
                    mask16 = attention_mask.clamp(min=torch.finfo(torch.float16).min).to(torch.float16)
                    # A query row whose every position is masked (a left-padding position): the reference adds
                    # the mask to its fp16 logits in the promoted dtype of the two and clamps
                    # (models/modeling_llama_KVmix.py:259-262).  With a half mask every entry of such a row ends
                    # at the lowest finite half, with a float mask of the lowest finite float the logit is
                    # absorbed: the softmax is uniform either way.  The fused routine adds in fp32 and would
                    # keep the logits' differences; a zero query makes them equal.  (A float mask holding
                    # -65504 keeps the differences in the reference too and is left alone.)
                    absorbed = torch.finfo(torch.float16).min if attention_mask.dtype == torch.float16 else -1e30
                    dead = attention_mask.amax(dim=-1, keepdim=True) <= absorbed
                    query_states = query_states.masked_fill(dead, 0)
                attn_output = F.scaled_dot_product_attention(query_states, key_states, value_states, attn_mask=mask16,
                                                             enable_gqa=n_rep > 1)
                cache = inplace if (use_cache and inplace is not None) else (
                    (kc, k_tail, ks, km, vc, v_tail, vs, vm, kv_seq_len) if use_cache else None)
                return attn_output, None, cache
            attn_weights = _grouped_matmul_qk(query_states, key_states, n_rep) / math.sqrt(D)
            if attention_mask is not None:
                if attention_mask.shape[-2:] != attn_weights.shape[-2:]:
                    raise ValueError(f"Attention mask shape {attention_mask.shape} does not match weights shape "
                                     f"{attn_weights.shape}")
                attn_weights = attn_weights + attention_mask
                attn_weights = torch.clamp(attn_weights, min=torch.finfo(attn_weights.dtype).min)
            attn_weights = F.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query_states.dtype)
            attn_output = _grouped_matmul_pv(attn_weights, value_states, n_rep)

        if not use_cache:
            cache = None
        elif inplace is not None:
            cache = inplace
        else:
            cache = (kc, k_tail, ks, km, vc, v_tail, vs, vm, kv_seq_len)
        return attn_output, attn_weights, cache

    __call__ = forward
