"""Host logic of the transformers wrappers (kvmix_amd.hf): what can be checked without a GPU.
A forward without a cache never touches the quantized operators, so it must reproduce the stock
model to fp32 rounding; any cached forward needs the GPU and must say so instead of falling back."""
import pytest
import torch


def _pair(kind):
    from transformers import LlamaConfig, LlamaForCausalLM, MistralConfig, MistralForCausalLM

    from kvmix_amd.hf import LlamaForCausalLM_KVmix, MistralForCausalLM_KVmix

    cls, stock_cls, mix_cls = ((LlamaConfig, LlamaForCausalLM, LlamaForCausalLM_KVmix) if kind == "llama" else
                               (MistralConfig, MistralForCausalLM, MistralForCausalLM_KVmix))
    extra = {} if kind == "llama" else {"sliding_window": 16}
    cfg = cls(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              vocab_size=300, max_position_embeddings=256, **extra)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    stock = stock_cls(cfg).eval()
    model = mix_cls(cfg, quant_bits={0: {"k_bits": 2, "v_bits": 4}}).eval()
    model.load_state_dict(stock.state_dict())
    return stock, model


@pytest.mark.parametrize("kind", ["llama", "mistral"])
def test_forward_without_cache_is_the_stock_model(kind):
    stock, model = _pair(kind)
    ids = torch.randint(0, 300, (2, 40), generator=torch.Generator().manual_seed(1))
    mask = torch.ones(2, 40, dtype=torch.long)
    mask[1, :9] = 0
    with torch.no_grad():
        want = stock(ids, attention_mask=mask, use_cache=False).logits
        got = model(ids, attention_mask=mask, use_cache=False).logits
    torch.testing.assert_close(got, want, rtol=0, atol=2e-6)  # fp32; only the grouping of the head matmuls differs


def test_quant_bits_and_cache_bookkeeping():
    from kvmix_amd import ops
    from kvmix_amd.hf import KVmixCache, normalise_quant_bits

    stock, model = _pair("llama")
    # layer 0 as given with the reference's ratios filled in (myprofileKV.py:75-80), layer 1 defaulted
    assert model.quant_bits == {0: {"k_bits": 2, "v_bits": 4, "k_residual_ratio": 0.2, "v_residual_ratio": 0.3},
                                1: {"k_bits": 4, "v_bits": 4, "k_residual_ratio": 0.3, "v_residual_ratio": 0.3}}
    assert model.model.layers[0].self_attn.kvmix.k_bits == 2 and model.group_size == 32
    assert type(model.model.layers[1].self_attn).__name__ == "LlamaAttention_KVmix"
    assert normalise_quant_bits([{"k_bits": 3, "v_bits": 1}], 1)[0]["v_residual_ratio"] == 0.1
    with pytest.raises(ValueError):
        normalise_quant_bits({0: {"k_bits": 5}}, 1)

    cache = model.new_cache(capacity=100)
    assert isinstance(cache, KVmixCache) and len(cache) == 2
    assert cache.get_seq_length() == 0 and cache.get_mask_sizes(7, 1) == (7, 0) and cache.get_max_length() == -1
    assert cache.packed(0).k_bits == 2 and cache.packed(1).capacity == 100
    three = KVmixCache(normalise_quant_bits([{"k_bits": 3, "v_bits": 3}], 1))
    assert three.packed(0).v_fmt == ops.FMT_DENSE3 and three.packed(0).Kgroup_size == 11
    with pytest.raises(NotImplementedError):
        cache.reorder_cache(torch.tensor([0]))
    with pytest.raises(NotImplementedError):
        cache.crop(1)


def test_cached_forward_needs_the_gpu_and_the_right_cache():
    from transformers import DynamicCache

    stock, model = _pair("llama")
    ids = torch.randint(0, 300, (1, 12), generator=torch.Generator().manual_seed(2))
    model = model.half()
    with pytest.raises(RuntimeError, match="GPU"):
        model(ids)  # use_cache defaults to True: the prompt's flush calls the quantizer
    with pytest.raises(TypeError, match="KVmixCache"):
        model(ids, past_key_values=DynamicCache(config=model.config))
    with pytest.raises(RuntimeError, match="KVmix"):
        stock(ids, past_key_values=model.new_cache())
    with pytest.raises(NotImplementedError):
        model.generate(ids, num_beams=4, max_new_tokens=2)
    # a loss computation creates no cache (and therefore runs anywhere), as the stock model's does
    fp32 = _pair("llama")[1]
    out = fp32(ids, labels=ids)
    assert out.past_key_values is None and out.loss.requires_grad
