"""The transformers wrappers (kvmix_amd.hf) on the GPU: `generate()` of a small random-weight model.

What is compared, and against what:
  * every layer's attention calls are recorded during `generate()` and replayed on the CPU oracle
    with the same q/k/v (ratio flush policy, the one the reference's models use): caches agree bit
    for bit at the end, attention outputs within the GEMV tolerance at every step;
  * a left-padded batch: with nothing quantized the logits of a teacher-forced decode agree with
    the stock fp16 model (positions, masks); with quantized layers the calls, masks included, are
    replayed on the oracle;
  * `from_pretrained(..., quant_bits=...)` builds the same model as the constructor.
No checkpoint of the reference can be loaded here (none is shipped, none can be fetched): weights
are random, N(0, 0.02) scaled up in the attention projections so that logits depend on the cache."""
import math

import numpy as np
import pytest
import torch

from test_gpu_attention import same_cache
from test_gpu_decoder import OracleAttention, replay_layer

pytestmark = pytest.mark.gpu

BITS = {0: {"k_bits": 4, "v_bits": 2, "k_residual_ratio": 0.3, "v_residual_ratio": 0.2},
        1: {"k_bits": 3, "v_bits": 4, "k_residual_ratio": 0.2, "v_residual_ratio": 0.3},
        2: {"k_bits": 2, "v_bits": 1, "k_residual_ratio": 0.2, "v_residual_ratio": 0.1},
        3: {"k_bits": 1, "v_bits": 4, "k_residual_ratio": 0.1, "v_residual_ratio": 0.3}}


class RatioOracle(OracleAttention):
    """OracleAttention with the reference's ratio policy instead of a fixed window."""

    def __init__(self, oracle, entry, group=32):
        super().__init__(oracle, entry["k_bits"], entry["v_bits"], None, group)
        self.k_ratio, self.v_ratio = entry["k_residual_ratio"], entry["v_residual_ratio"]

    def prompt(self, q, k, v, mask):
        from kvmix_amd.cache import flush_length

        o = self.o
        T = k.shape[2]
        out, _ = o.attention_prompt(q, k, v, mask)
        kg = 11 if self.k_bits == 3 else self.group
        nk = flush_length(T, self.k_ratio, kg, None, prompt=True)
        nv = flush_length(T, self.v_ratio, self.group, None, prompt=True)
        kc, ks, km = o.quantize_pack_last_dim(np.ascontiguousarray(k[:, :, :nk].transpose(0, 1, 3, 2)), kg, self.k_bits)
        vc, vs, vm = o.quantize_pack_last_dim(np.ascontiguousarray(v[:, :, :nv]), self.group, self.v_bits)
        return out, (kc, k[:, :, nk:], ks, km, vc, v[:, :, nv:], vs, vm, T)

    def step(self, q, k, v, cache, compute_output=True):
        return self.o.attention_decode_step(q, k, v, cache, self.k_bits, self.v_bits, self.k_ratio, self.v_ratio,
                                            group_size=self.group, v_dense3=self.v_dense3, compute_output=compute_output)


class Tap:
    """Stands in for a layer's KVmixAttention and keeps what went in and what came out."""

    def __init__(self, att, keep_masks=False):
        self.att, self.calls, self.keep_masks = att, [], keep_masks

    def __call__(self, q, k, v, cache, attention_mask=None, use_cache=True, need_weights=True):
        out, p, cache = self.att(q, k, v, cache, attention_mask=attention_mask, use_cache=use_cache, need_weights=need_weights)
        rec = tuple(t.contiguous().cpu().numpy() for t in (q, k, v, out))
        if self.keep_masks:
            rec += (None if attention_mask is None else attention_mask.cpu().numpy(),)
        self.calls.append(rec)
        return out, p, cache


def small_config(kind, layers=4, **extra):
    from transformers import LlamaConfig, MistralConfig

    cls = LlamaConfig if kind == "llama" else MistralConfig
    cfg = cls(hidden_size=512, intermediate_size=1024, num_hidden_layers=layers, num_attention_heads=4,
              num_key_value_heads=2, vocab_size=1000, max_position_embeddings=2048, eos_token_id=None, **extra)  # (no token ends a generation early)
    cfg._attn_implementation = "eager"
    return cfg


def build_pair(kind, dev, quant_bits, seed=5, **extra):
    """(stock model, KVmix model) with the same fp16 weights."""
    from transformers import LlamaForCausalLM, MistralForCausalLM

    from kvmix_amd.hf import LlamaForCausalLM_KVmix, MistralForCausalLM_KVmix

    cfg = small_config(kind, layers=len(quant_bits), **extra)
    torch.manual_seed(seed)
    stock = (LlamaForCausalLM if kind == "llama" else MistralForCausalLM)(cfg)
    with torch.no_grad():  # default init (std 0.02) leaves attention nearly uniform; sharpen it
        for layer in stock.model.layers:
            layer.self_attn.q_proj.weight.mul_(4.0)
            layer.self_attn.k_proj.weight.mul_(4.0)
    stock = stock.half().to(dev).eval()
    model = (LlamaForCausalLM_KVmix if kind == "llama" else MistralForCausalLM_KVmix)(cfg, quant_bits=quant_bits)
    model.load_state_dict(stock.state_dict())
    return stock, model.half().to(dev).eval()


@pytest.mark.parametrize("kind", ["llama", "mistral"])
def test_generate_replayed_on_the_oracle(oracle, dev, kind):
    stock, model = build_pair(kind, dev, BITS)
    taps = []
    for layer in model.model.layers:
        layer.self_attn.kvmix = Tap(layer.self_attn.kvmix)
        taps.append(layer.self_attn.kvmix)
    B, T, new = 2, 150, 70
    ids = torch.randint(0, 1000, (B, T), generator=torch.Generator().manual_seed(1)).to(dev)
    cache = model.new_cache(capacity=64)  # small on purpose: the packed buffers have to grow
    out = model.generate(ids, max_new_tokens=new, do_sample=False, past_key_values=cache, pad_token_id=0)
    assert out.shape == (B, T + new) and torch.equal(out[:, :T], ids)
    assert cache.get_seq_length() == T + new - 1  # the last sampled token was never fed back
    for li, tap in enumerate(taps):
        assert len(tap.calls) == new and tap.calls[0][0].shape[2] == T and tap.calls[1][0].shape[2] == 1
        final = tuple(x.cpu().numpy() if torch.is_tensor(x) else x for x in cache.to_legacy_tuple(li))
        replay_layer(RatioOracle(oracle, BITS[li]), tap.calls, {new - 1}, {new - 1: final})
        assert final[0] is not None and final[4] is not None

    # greedy tokens of the stock model from the same prompt: the first one comes from the prompt
    # forward, which uses no quantized data, and must be identical
    ref = stock.generate(ids, max_new_tokens=1, do_sample=False, pad_token_id=0)
    assert torch.equal(ref[:, T], out[:, T])


def _teacher_forced(model, ids, mask, T, cache):
    """Logits of a prompt forward followed by single-token forwards over ids[:, T:]."""
    logits = []
    with torch.no_grad():
        o = model(ids[:, :T], attention_mask=mask[:, :T], past_key_values=cache, use_cache=True)
        cache = o.past_key_values
        logits.append(o.logits[:, -1].float())
        for t in range(T, ids.shape[1]):
            o = model(ids[:, t:t + 1], attention_mask=mask[:, :t + 1], past_key_values=cache, use_cache=True)
            logits.append(o.logits[:, -1].float())
    return torch.stack(logits, 1), cache


@pytest.mark.parametrize("kind,extra", [("llama", {}), ("mistral", {"sliding_window": 64})])
def test_left_padded_batch(oracle, dev, kind, extra):
    """Positions and masks of a left-padded batch (what the tokenizer in Inference-comparision.py:101
    produces).  Random weights make the dense-cache model a poor yardstick for quantized layers (their
    noise is a large part of a signal that is itself noise), so the check is split in two:
    with ratios of 1.0 nothing is ever quantized and the logits must match the stock model's closely,
    which pins positions, masks and head mapping; with 4-bit layers the recorded calls, masks
    included, are replayed on the oracle."""
    B, T, n = 3, 90, 60
    ids = torch.randint(0, 1000, (B, T + n), generator=torch.Generator().manual_seed(2)).to(dev)
    mask = torch.ones(B, T + n, dtype=torch.long, device=dev)
    mask[1, :17] = 0
    mask[2, :40] = 0

    keep = {i: {"k_bits": 4, "v_bits": 2, "k_residual_ratio": 1.0, "v_residual_ratio": 1.0} for i in range(3)}
    stock, model = build_pair(kind, dev, keep, **extra)
    want, _ = _teacher_forced(stock, ids, mask, T, None)
    got, cache = _teacher_forced(model, ids, mask, T, model.new_cache())
    assert cache.get_seq_length() == T + n and cache.packed(0).k_tokens == 0
    spread = float(want.std())
    err = (got - want).abs()
    # fp16 model, different summation orders: measured max 0.03, rms 0.004 of the spread
    assert float(err.max()) <= 0.1 * spread and float(err.pow(2).mean().sqrt()) <= 0.01 * spread, (float(err.max()), spread)

    four = {0: {"k_bits": 4, "v_bits": 4}, 1: {"k_bits": 2, "v_bits": 4}, 2: {"k_bits": 3, "v_bits": 2}}
    stock, model = build_pair(kind, dev, four, **extra)
    taps = []
    for layer in model.model.layers:
        layer.self_attn.kvmix = Tap(layer.self_attn.kvmix, keep_masks=True)
        taps.append(layer.self_attn.kvmix)
    got, cache = _teacher_forced(model, ids, mask, T, model.new_cache())
    assert cache.packed(0).k_tokens > 0 and cache.packed(0).v_tokens > 0
    # gross errors only (a wrong position or mask moves logits by more than their spread)
    assert float((got - want).pow(2).mean().sqrt()) <= 0.6 * spread
    for li, tap in enumerate(taps):
        orc, state = RatioOracle(oracle, model.quant_bits[li]), None
        for step, (q, k, v, out_g, m) in enumerate(tap.calls):
            # (the prompt's mask arrives in the model's dtype, a single-token step's in fp32)
            assert m is not None and m.dtype == (np.float16 if step == 0 else np.float32)
            assert m.shape == (B, 1, q.shape[2], T + step)
            if state is None:
                out_o, state = orc.prompt(q, k, v, m)
            else:
                out_o, _, state = oracle.attention_decode_step(q, k, v, state, orc.k_bits, orc.v_bits, orc.k_ratio,
                                                               orc.v_ratio, group_size=32, attention_mask=m)
            np.testing.assert_allclose(out_g.astype(np.float64), out_o.astype(np.float64), rtol=5e-3, atol=5e-3,
                                       err_msg=f"layer {li} step {step}")
        same_cache(tuple(x.cpu().numpy() if torch.is_tensor(x) else x for x in cache.to_legacy_tuple(li)), state)


def test_from_pretrained_takes_quant_bits(dev, tmp_path):
    from kvmix_amd.hf import LlamaForCausalLM_KVmix

    stock, model = build_pair("llama", dev, {0: BITS[0], 1: BITS[2]})
    stock.save_pretrained(tmp_path)
    cfg = small_config("llama", layers=2)
    cfg.group_size = 32
    loaded = LlamaForCausalLM_KVmix.from_pretrained(tmp_path, config=cfg, attn_implementation="eager",
                                                    torch_dtype=torch.float16, quant_bits={0: BITS[0], 1: BITS[2]}).to(dev).eval()
    assert loaded.quant_bits == model.quant_bits
    assert loaded.model.layers[1].self_attn.kvmix.k_bits == 2 and loaded.model.layers[1].self_attn.kvmix.v_bits == 1
    for name, w in model.state_dict().items():
        assert torch.equal(w, loaded.state_dict()[name]), name
    # a model built by .half() and one loaded as fp16 differ in the rotary frequencies' rounding, so
    # generations are compared with a stock model loaded the same way: the first new token comes
    # from the prompt forward alone and must be the same
    from transformers import LlamaForCausalLM

    same_way = LlamaForCausalLM.from_pretrained(tmp_path, config=small_config("llama", layers=2), attn_implementation="eager",
                                                torch_dtype=torch.float16).to(dev).eval()
    ids = torch.randint(0, 1000, (1, 100), generator=torch.Generator().manual_seed(3)).to(dev)
    a = same_way.generate(ids, max_new_tokens=1, do_sample=False, pad_token_id=0)
    b = loaded.generate(ids, max_new_tokens=12, do_sample=False, pad_token_id=0)
    assert b.shape == (1, 112) and torch.equal(a[:, :101], b[:, :101])


def test_three_bit_values_and_refusals(dev):
    from transformers import DynamicCache

    stock, model = build_pair("llama", dev, {0: {"k_bits": 3, "v_bits": 3}, 1: {"k_bits": 4, "v_bits": 3}})
    ids = torch.randint(0, 1000, (2, 120), generator=torch.Generator().manual_seed(4)).to(dev)
    out = model.generate(ids, max_new_tokens=40, do_sample=False, pad_token_id=0)
    assert out.shape == (2, 160)
    with pytest.raises(NotImplementedError):
        model.generate(ids, max_new_tokens=4, num_beams=2)
    with pytest.raises(TypeError):
        model(ids, past_key_values=DynamicCache(config=model.config), use_cache=True)
    with pytest.raises(RuntimeError):
        stock(ids, past_key_values=model.new_cache(), use_cache=True)


def test_recipe_profile_then_generate(dev):
    """Inference-comparision.py:56-153 in small: profile the stock model, build the KVmix model
    from the bits it returns, generate from a padded batch."""
    from kvmix_amd.hf import LlamaForCausalLM_KVmix
    from kvmix_amd.profiler import profile_model

    stock, _ = build_pair("llama", dev, {i: {} for i in range(10)})
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 1000, (1, 64), generator=g).to(dev) for _ in range(2)]
    quant_bits = profile_model(stock, prompts, [torch.ones_like(p) for p in prompts], [p.clone() for p in prompts], 10)
    assert sorted(e["k_bits"] for e in quant_bits.values()) == [2] * 8 + [3] * 2
    assert sorted(e["v_bits"] for e in quant_bits.values()) == [2] * 8 + [4] * 2
    model = LlamaForCausalLM_KVmix(stock.config, quant_bits=quant_bits)
    model.load_state_dict(stock.state_dict())
    model = model.half().to(dev).eval()
    ids = torch.randint(0, 1000, (4, 200), generator=g).to(dev)
    mask = torch.ones_like(ids)
    mask[0, :30] = 0
    out = model.generate(ids, attention_mask=mask, max_new_tokens=48, do_sample=False, pad_token_id=0)
    assert out.shape == (4, 248)
    want = stock.eval().generate(ids, attention_mask=mask, max_new_tokens=1, do_sample=False, pad_token_id=0)
    assert torch.equal(out[:, 200], want[:, 200])
    # the profiler also runs on the converted model (a loss computation creates no cache) and, the
    # cache-less forward being the stock one, ranks the layers the same way
    again = profile_model(model, prompts, [torch.ones_like(p) for p in prompts], [p.clone() for p in prompts], 10)
    assert again == quant_bits


def test_cache_reuse_sampling_and_attentions(dev):
    stock, model = build_pair("llama", dev, BITS)
    ids = torch.randint(0, 1000, (2, 150), generator=torch.Generator().manual_seed(1)).to(dev)
    fresh = model.generate(ids, max_new_tokens=40, do_sample=False, pad_token_id=0)
    cache = model.new_cache(64)
    first = model.generate(ids, max_new_tokens=40, do_sample=False, pad_token_id=0, past_key_values=cache)
    cache.reset()
    assert cache.get_seq_length() == 0
    again = model.generate(ids, max_new_tokens=40, do_sample=False, pad_token_id=0, past_key_values=cache)
    assert torch.equal(fresh, first) and torch.equal(fresh, again)  # a reset cache behaves like a new one
    sampled = model.generate(ids, max_new_tokens=10, do_sample=True, top_k=5, pad_token_id=0)
    assert sampled.shape == (2, 160)
    cache = model.new_cache()
    with torch.no_grad():
        model(ids, past_key_values=cache, use_cache=True)
        step = model(ids[:, :1], past_key_values=cache, use_cache=True, output_attentions=True)
    assert len(step.attentions) == 4 and tuple(step.attentions[0].shape) == (2, 4, 1, 151)  # the four-launch step returns its probabilities
    assert float((step.attentions[0].float().sum(-1) - 1).abs().max()) < 2e-3
