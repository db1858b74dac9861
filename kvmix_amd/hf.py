"""Causal-LM wrappers with the KVmix cache for the installed `transformers` (5.x, `Cache` API).

The reference ships forks of transformers 4.46's Llama and Mistral files
(models/modeling_llama_KVmix.py:29-283,515-537, models/modeling_mistral_KVmix.py:71-329) whose
attention layers keep a mixed-precision cache and whose model classes take a `quant_bits` argument:

    quant_bits[layer_idx] = {'k_bits': .., 'v_bits': .., 'k_residual_ratio': .., 'v_residual_ratio': ..}
    model = LlamaForCausalLM_KVmix.from_pretrained(path, config=config, attn_implementation="eager",
                                                   torch_dtype=torch.float16, quant_bits=quant_bits)
    model.generate(input_ids, attention_mask=mask, max_new_tokens=n)        # Inference-comparision.py:89-153

These classes keep that recipe (same class names, same `quant_bits` layout, `config.group_size`)
on top of the stock `LlamaForCausalLM` / `MistralForCausalLM`: each `self_attn` keeps the stock
projections and RoPE and hands q, k, v to `KVmixAttention`, and the cache object that travels
through `generate()` is a `KVmixCache` holding one in-place `PackedKVCache` per layer.  The stock
model code (embeddings, masks, norms, MLP, sampling) is untouched.

Not supported, and refused with an error rather than silently served from a dense cache: beam
search and assisted decoding (they reorder or crop the cache), other `Cache` classes, attention
implementations other than "eager" (the reference asks for eager too).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Union

import torch
from transformers import LlamaForCausalLM, MistralForCausalLM
from transformers.cache_utils import Cache, CacheLayerMixin
from transformers.models.llama.modeling_llama import LlamaAttention
from transformers.models.llama.modeling_llama import apply_rotary_pos_emb as llama_rope
from transformers.models.mistral.modeling_mistral import MistralAttention
from transformers.models.mistral.modeling_mistral import apply_rotary_pos_emb as mistral_rope

from . import ops
from .attention import KVmixAttention
from .cache import RESIDUAL_RATIO_BY_BITS, PackedKVCache

QuantBits = Union[Dict[int, dict], Sequence[dict], None]


def normalise_quant_bits(quant_bits: QuantBits, num_layers: int, default_bits: int = 4) -> Dict[int, dict]:
    """The reference's per-layer dictionary, completed: layers that are absent get `default_bits`,
    ratios that are absent get the reference's value for that bit width
    (models/modeling_llama_KVmix.py:36-39 reads the four keys unconditionally)."""
    if quant_bits is None:
        quant_bits = {}
    if not isinstance(quant_bits, dict):
        quant_bits = dict(enumerate(quant_bits))
    out = {}
    for i in range(num_layers):
        entry = dict(quant_bits.get(i, {}))
        kb, vb = int(entry.get("k_bits", default_bits)), int(entry.get("v_bits", default_bits))
        for name, bits in (("k_bits", kb), ("v_bits", vb)):
            if bits not in RESIDUAL_RATIO_BY_BITS:
                raise ValueError(f"quant_bits[{i}]['{name}'] = {bits}: supported widths are {sorted(RESIDUAL_RATIO_BY_BITS)}")
        out[i] = {"k_bits": kb, "v_bits": vb,
                  "k_residual_ratio": float(entry.get("k_residual_ratio", RESIDUAL_RATIO_BY_BITS[kb])),
                  "v_residual_ratio": float(entry.get("v_residual_ratio", RESIDUAL_RATIO_BY_BITS[vb]))}
    return out


class KVmixLayer(CacheLayerMixin):
    """One layer's slot in a `KVmixCache`: an in-place packed cache plus the bookkeeping the stock
    model code asks of a cache layer (lengths for position ids and masks)."""

    is_compileable = False
    supports_early_init = False
    is_sliding = False

    def __init__(self, packed: PackedKVCache):
        super().__init__()
        self.packed = packed
        self.is_initialized = True

    def lazy_initialization(self, key_states, value_states) -> None:  # buffers are created on first append
        return None

    def update(self, key_states, value_states, *args, **kwargs):
        raise RuntimeError("a KVmixCache is filled by the KVmix attention layers; the model it was passed to is not a "
                           "*_KVmix model")

    def get_seq_length(self) -> int:
        return int(self.packed.kv_seq_len)

    def get_mask_sizes(self, query_length: int):
        return self.get_seq_length() + query_length, 0

    def get_max_length(self) -> int:
        return -1

    def reset(self) -> None:
        self.packed.reset()

    def reorder_cache(self, beam_idx) -> None:
        raise NotImplementedError("beam search is not available with the KVmix cache")

    def crop(self, *args, **kwargs) -> None:
        raise NotImplementedError("the KVmix cache cannot give tokens back (quantized groups are not reversible)")

    batch_repeat_interleave = batch_select_indices = reorder_cache


class KVmixCache(Cache):
    """`past_key_values` for the *_KVmix models: one `PackedKVCache` per layer, with that layer's
    bit widths and residual policy.  `capacity` = tokens the packed buffers are allocated for up
    front (they grow when exceeded)."""

    def __init__(self, quant_bits: Dict[int, dict], group_size: int = 32, capacity: int = 4096,
                 residual_length: Optional[int] = None, three_bit_values_dense: bool = True):
        layers = []
        for i in range(len(quant_bits)):
            e = quant_bits[i]
            # the reference has no working 3-bit value format (quant_cuda/csrc/quantization_cuda.cu:413-537
            # rejects head_dim % 11); 3-bit values use this library's dense 32-per-3-words format
            v_fmt = ops.FMT_DENSE3 if (e["v_bits"] == 3 and three_bit_values_dense) else ops.FMT_REF
            layers.append(KVmixLayer(PackedKVCache(e["k_bits"], e["v_bits"], group_size, e["k_residual_ratio"],
                                                   e["v_residual_ratio"], residual_length, capacity, ops.FMT_REF, v_fmt)))
        super().__init__(layers=layers)

    def packed(self, layer_idx: int) -> PackedKVCache:
        return self.layers[layer_idx].packed

    def flush_ahead(self) -> int:
        """Run now, batched, the flushes the coming one-token step would run layer by layer (cache.flush_ahead)."""
        from .cache import flush_ahead

        return flush_ahead([layer.packed for layer in self.layers])

    def to_legacy_tuple(self, layer_idx: int):
        """The reference's 9-entry tuple for one layer (models/modeling_llama_KVmix.py:270-273), as views."""
        return self.layers[layer_idx].packed.as_tuple()


class _KVmixAttentionForward:
    """forward() shared by the Llama and Mistral attention subclasses: the stock projections and
    RoPE, then `KVmixAttention` instead of `past_key_values.update` + the attention interface."""

    _rope = None

    def _init_kvmix(self, entry: dict, group_size: int, residual_length: Optional[int]) -> None:
        self.kvmix = KVmixAttention(entry["k_bits"], entry["v_bits"], entry["k_residual_ratio"],
                                    entry["v_residual_ratio"], group_size, residual_length)

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None, **kwargs):
        input_shape = hidden_states.shape[:-1]
        hidden_shape = (*input_shape, -1, self.head_dim)
        query_states = self.q_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        key_states = self.k_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        value_states = self.v_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        cos, sin = position_embeddings
        query_states, key_states = type(self)._rope(query_states, key_states, cos, sin)

        if past_key_values is not None and not isinstance(past_key_values, KVmixCache):
            raise TypeError(f"{type(self).__name__} needs a KVmixCache as past_key_values, got "
                            f"{type(past_key_values).__name__}")
        q_len = query_states.shape[2]
        if attention_mask is None and q_len > 1:
            # the mask builder may leave a purely causal mask out; KVmixAttention applies what it is given
            seen = 0 if past_key_values is None else past_key_values.get_seq_length(self.layer_idx)
            attention_mask = torch.full((q_len, seen + q_len), torch.finfo(torch.float32).min, dtype=torch.float32,
                                        device=query_states.device).triu_(seen + 1)[None, None]
        if attention_mask is not None:
            # A prompt's mask stays in the model's dtype, as transformers builds it for the reference: the
            # prompt branch adds it to fp16 logits in fp16 (models/modeling_llama_KVmix.py:259-262), which is
            # what makes the rows of left-padding positions uniform.  A single-token step adds it to fp32
            # logits (:68-75,189-192), and the library's step takes fp32.
            mask_dtype = query_states.dtype if q_len > 1 else torch.float32
            if attention_mask.dtype == torch.bool:
                attention_mask = torch.zeros(attention_mask.shape, dtype=mask_dtype, device=attention_mask.device
                                             ).masked_fill_(~attention_mask, torch.finfo(mask_dtype).min)
            elif attention_mask.dtype != mask_dtype:
                attention_mask = attention_mask.clamp(min=torch.finfo(mask_dtype).min).to(mask_dtype)
        packed = None if past_key_values is None else past_key_values.packed(self.layer_idx)
        if packed is not None and q_len == 1 and self.layer_idx == 0:
            # a decode step: what its layers flush are tokens of earlier steps -- all layers' flushes at once,
            # batched, before the first layer runs (cache.flush_ahead)
            past_key_values.flush_ahead()
        attn_output, attn_weights, _ = self.kvmix(query_states, key_states, value_states, packed,
                                                  attention_mask=attention_mask, use_cache=packed is not None,
                                                  need_weights=bool(kwargs.get("output_attentions", False)))
        attn_output = attn_output.transpose(1, 2).reshape(*input_shape, -1).contiguous()
        return self.o_proj(attn_output), attn_weights


class LlamaAttention_KVmix(_KVmixAttentionForward, LlamaAttention):
    """models/modeling_llama_KVmix.py:29-283 on the stock LlamaAttention's weights."""
    _rope = staticmethod(llama_rope)


class MistralAttention_KVmix(_KVmixAttentionForward, MistralAttention):
    """models/modeling_mistral_KVmix.py:71-329 on the stock MistralAttention's weights."""
    _rope = staticmethod(mistral_rope)


class _KVmixCausalLM:
    """What the two model classes share: converting the attention layers, creating the cache."""

    _attention_class = None

    def _convert(self, config, quant_bits: QuantBits) -> None:
        if getattr(config, "_attn_implementation", "eager") not in (None, "eager"):
            # the KVmix layers never consult the attention interface; the mask they receive must be
            # the additive 4-D one that "eager" gets
            config._attn_implementation = "eager"
        self.quant_bits = normalise_quant_bits(quant_bits, config.num_hidden_layers)
        self.group_size = int(getattr(config, "group_size", 32))       # Inference-comparision.py:15
        self.residual_length = getattr(config, "residual_length", None)
        for i, layer in enumerate(self.model.layers):
            layer.self_attn.__class__ = self._attention_class          # same weights, new forward
            layer.self_attn._init_kvmix(self.quant_bits[i], self.group_size, self.residual_length)

    def new_cache(self, capacity: int = 4096) -> KVmixCache:
        return KVmixCache(self.quant_bits, self.group_size, capacity, self.residual_length)

    def _with_cache(self, kwargs: dict, capacity: int) -> dict:
        pkv = kwargs.get("past_key_values")
        if pkv is None:
            kwargs["past_key_values"] = self.new_cache(capacity)
        elif not isinstance(pkv, KVmixCache):
            raise TypeError(f"{type(self).__name__} needs a KVmixCache as past_key_values, got {type(pkv).__name__}")
        return kwargs

    def forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                inputs_embeds=None, labels=None, use_cache=None, **kwargs):
        # a cache is created when the caller asks for one (or leaves it to the config) and is not
        # computing a loss; a cache that is passed in is always used
        use = self.config.use_cache if use_cache is None else use_cache
        if use_cache is None and labels is not None:
            use = False
        if use or past_key_values is not None:
            n = input_ids.shape[1] if input_ids is not None else inputs_embeds.shape[1]
            past_key_values = self._with_cache({"past_key_values": past_key_values}, max(4096, 2 * n))["past_key_values"]
        return super().forward(input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids,
                               past_key_values=past_key_values, inputs_embeds=inputs_embeds, labels=labels,
                               use_cache=use, **kwargs)

    def generate(self, inputs=None, **kwargs):
        if kwargs.get("num_beams", 1) != 1 or kwargs.get("assistant_model") is not None:
            raise NotImplementedError("beam search and assisted decoding are not available with the KVmix cache")
        ids = inputs if inputs is not None else kwargs.get("input_ids")
        prompt_len = int(ids.shape[1]) if ids is not None else 0
        new = kwargs.get("max_new_tokens")
        if new is None:
            gc = kwargs.get("generation_config") or self.generation_config
            new = getattr(gc, "max_new_tokens", None) or max(int(getattr(gc, "max_length", 20) or 20) - prompt_len, 0)
        kwargs = self._with_cache(kwargs, prompt_len + int(new) + 1)
        return super().generate(inputs, **kwargs)


class LlamaForCausalLM_KVmix(_KVmixCausalLM, LlamaForCausalLM):
    """Drop-in for the reference's class of the same name (models/modeling_llama_KVmix.py:515-537)."""
    _attention_class = LlamaAttention_KVmix

    def __init__(self, config, quant_bits: QuantBits = None, **kwargs):
        super().__init__(config)
        self._convert(config, quant_bits)


class MistralForCausalLM_KVmix(_KVmixCausalLM, MistralForCausalLM):
    """Drop-in for the reference's class of the same name (models/modeling_mistral_KVmix.py)."""
    _attention_class = MistralAttention_KVmix

    def __init__(self, config, quant_bits: QuantBits = None, **kwargs):
        super().__init__(config)
        self._convert(config, quant_bits)
