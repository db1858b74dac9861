"""End-to-end decode loop (kvmix_amd.decoder.Decoder + KVmixAttention + in-place caches) on the GPU.

What is compared, and against what:
  * every sampled layer's attention step is replayed on the CPU oracle with the very q/k/v the
    GPU run produced: the caches must agree bit for bit and the attention outputs within the GEMV
    tolerance, at every step;
  * at the reduced size the whole model is also run on the CPU in fp32 with the oracle's attention,
    fed the GPU run's tokens: logits agree within what fp16 GEMMs allow (tolerance stated below).
The prompt branch of the oracle adapter restates models/modeling_llama_KVmix.py:213-266."""
import math

import numpy as np
import pytest
import torch

from helpers import same_bits
from test_gpu_attention import same_cache

pytestmark = pytest.mark.gpu


class Recorder:
    """Wraps one layer's attention; keeps what went in and what came out."""

    def __init__(self, att, keep_prompt_out=True):
        self.att, self.calls, self.keep_prompt_out = att, [], keep_prompt_out

    def __call__(self, q, k, v, cache, attention_mask=None, need_weights=True):
        out, p, cache = self.att(q, k, v, cache, attention_mask=attention_mask, need_weights=need_weights)
        keep_out = self.keep_prompt_out or q.shape[2] == 1
        self.calls.append((q.contiguous().cpu().numpy(), k.contiguous().cpu().numpy(), v.contiguous().cpu().numpy(),
                           out.cpu().numpy() if keep_out else None))
        return out, p, cache


class OracleAttention:
    """The oracle behind the attention-call signature, on CPU tensors."""

    def __init__(self, oracle, k_bits, v_bits, window, group=32, prompt_output=True):
        self.o, self.k_bits, self.v_bits, self.window, self.group = oracle, k_bits, v_bits, window, group
        self.prompt_output = prompt_output

    def prompt(self, q, k, v, mask):
        from kvmix_amd.cache import flush_length

        o = self.o
        B, nh, T, D = q.shape
        rep = nh // k.shape[1]
        out = None
        if self.prompt_output:
            w = o._matmul_f16(q, o.repeat_kv(k, rep).transpose(0, 1, 3, 2)).astype(np.float32) / np.float32(math.sqrt(D))
            if mask is not None:
                w = np.maximum(w + mask.astype(np.float32), np.finfo(np.float32).min)
            p = o._softmax_f32(w.astype(np.float32)).astype(np.float16)
            out = o._matmul_f16(p, o.repeat_kv(v, rep))
        kg = 11 if self.k_bits == 3 else self.group
        nk = flush_length(T, 0.0, kg, self.window, prompt=True)
        nv = flush_length(T, 0.0, self.group, self.window, prompt=True)
        kc = ks = km = vc = vs = vm = None
        if nk:
            kc, ks, km = o.quantize_pack_last_dim(np.ascontiguousarray(k[:, :, :nk].transpose(0, 1, 3, 2)), kg, self.k_bits)
        if nv:
            vc, vs, vm = o.quantize_pack_last_dim(np.ascontiguousarray(v[:, :, :nv]), self.group, self.v_bits)
        return out, (kc, k[:, :, nk:], ks, km, vc, v[:, :, nv:], vs, vm, T)

    def step(self, q, k, v, cache):
        return self.o.attention_decode_step(q, k, v, cache, self.k_bits, self.v_bits, 0.0, 0.0, group_size=self.group,
                                            fixed_window=self.window)

    def __call__(self, q, k, v, cache, attention_mask=None, need_weights=True):
        dt = q.dtype
        qn, kn, vn = (np.ascontiguousarray(t.to(torch.float16).numpy()) for t in (q, k, v))
        if cache is None:
            out, cache = self.prompt(qn, kn, vn, None if attention_mask is None else attention_mask.numpy())
        else:
            out, _, cache = self.step(qn, kn, vn, cache)
        return torch.from_numpy(out).to(dt), None, cache


def replay_layer(oracle_att, calls, check_steps, gpu_cache_at):
    """Feed the recorded inputs of one layer to the oracle; compare outputs at every decode step
    and caches at the steps in check_steps (gpu_cache_at[step] = the GPU cache tuple as numpy)."""
    cache = None
    worst = 0.0
    for step, (q, k, v, out_g) in enumerate(calls):
        if cache is None:
            out_o, cache = oracle_att.prompt(q, k, v, np.triu(np.full((q.shape[2],) * 2, np.finfo(np.float32).min, np.float32), 1)[None, None])
        else:
            out_o, _, cache = oracle_att.step(q, k, v, cache)
        if out_g is not None and out_o is not None:
            a, b = out_g.astype(np.float64), out_o.astype(np.float64)
            # fp16 probabilities times values: relative 5e-3 plus an absolute floor of 5e-3 (outputs are O(0.1..1))
            np.testing.assert_allclose(a, b, rtol=5e-3, atol=5e-3, err_msg=f"step {step}")
            worst = max(worst, float(np.abs(a - b).max()))
        if step in check_steps:
            same_cache(gpu_cache_at[step], cache)
    return worst


def run_gpu(cfg, kbits, vbits, window, B, T, new_tokens, dev, sample_layers, check_steps, keep_prompt_out=True):
    from kvmix_amd.decoder import Decoder, init_weights, kvmix_layers

    weights = init_weights(cfg, dev)
    atts, caches = kvmix_layers(cfg, kbits, vbits, residual_length=window, capacity=T + new_tokens)
    recs = {li: Recorder(atts[li], keep_prompt_out) for li in sample_layers}
    dec = Decoder(cfg, weights, [recs.get(li, a) for li, a in enumerate(atts)], caches)
    gen = torch.Generator(device="cpu").manual_seed(40)
    prompt = torch.randint(0, cfg.vocab_size, (B, T), generator=gen).to(dev)
    logits, snaps = {}, {li: {} for li in sample_layers}

    def on_step(step, lg):
        if step in check_steps:
            logits[step] = lg.cpu().numpy()
            for li in sample_layers:
                snaps[li][step] = tuple(x.cpu().numpy() if torch.is_tensor(x) else x for x in dec.caches[li].as_tuple())

    tokens = dec.generate(prompt, new_tokens, on_step)
    return weights, prompt, tokens, logits, snaps, recs


def test_small_model_against_the_oracle_end_to_end(oracle, dev):
    from kvmix_amd.decoder import Decoder, DecoderConfig

    cfg = DecoderConfig(hidden_size=512, num_layers=4, num_heads=4, num_kv_heads=2, intermediate_size=1024, vocab_size=1000)
    kbits, vbits, window = [4, 3, 2, 1], [2, 4, 4, 1], 64
    B, T, new = 2, 200, 141
    check = {0, 1, 64, 128, 140}
    weights, prompt, tokens, logits_g, snaps, recs = run_gpu(cfg, kbits, vbits, window, B, T, new, dev, range(4), check)
    assert tokens.shape == (B, new)
    for li in range(4):
        assert len(recs[li].calls) == new  # the prompt and new - 1 decode forwards
        replay_layer(OracleAttention(oracle, kbits[li], vbits[li], window), recs[li].calls, check, snaps[li])
        assert snaps[li][140][0] is not None and snaps[li][140][4] is not None  # both sides did flush

    # the whole model on the CPU in fp32 with the oracle's attention, fed the GPU's tokens
    w32 = {"embed": weights["embed"].float().cpu(), "norm": weights["norm"].float().cpu(),
           "lm_head": weights["lm_head"].float().cpu(),
           "layers": [{k: v.float().cpu() for k, v in lw.items()} for lw in weights["layers"]]}
    cpu = Decoder(cfg, w32, [OracleAttention(oracle, kb, vb, window) for kb, vb in zip(kbits, vbits)])
    ids = torch.cat([prompt.cpu(), tokens.cpu()], dim=1)
    lg = cpu.forward(ids[:, :T])
    for step in range(0, 141):
        if step:
            lg = cpu.forward(ids[:, T + step - 1:T + step])
        if step in check:
            want, got = lg.numpy().astype(np.float64), logits_g[step].astype(np.float64)
            # fp16 weights and activations on the GPU against fp32 on the CPU, four layers deep, and
            # quantization codes that flip where a value sits next to a rounding boundary (1-bit
            # layers turn such a flip into a full-scale change of that value): bounded relative to
            # the spread of the logits, in the maximum and, four times tighter, in the mean square
            spread = float(want.std())
            err = np.abs(got - want)
            print(f"step {step}: max {err.max() / spread:.4f} rms {np.sqrt((err ** 2).mean()) / spread:.4f} of the spread")
            assert err.max() <= 0.06 * spread and np.sqrt((err ** 2).mean()) <= 0.015 * spread, step
    # the caches of the two runs hold almost the same codes (inputs differ by fp16 GEMM rounding)
    kc_g = snaps[0][140][0]
    kc_c = cpu.caches[0][0]
    assert kc_g.shape == kc_c.shape
    diff = kc_g ^ kc_c  # 4-bit fields that differ
    fields = sum(int(((diff >> (4 * i)) & 15 != 0).sum()) for i in range(8))
    assert fields / (kc_g.size * 8) < 0.02


def test_llama2_7b_shape_decode_loop(oracle, dev):
    """BASELINE's end-to-end case at full size: random-init Llama-2-7B, prompt 2048, batch 4, 512 new
    tokens, mixed per-layer bits, 128-token window; three layers replayed on the oracle, caches
    compared at forwards 1 (the prompt), 128 and 512."""
    from bench import layer_bits
    from kvmix_amd.decoder import DecoderConfig

    cfg = DecoderConfig()
    kbits, vbits = layer_bits(32)
    sample = [li for li in range(32) if vbits[li] != 3]  # the oracle's step has the reference's formats only
    by_k = {}
    for li in sample:
        by_k.setdefault(kbits[li], li)  # one layer per key bit width
    sample = sorted(by_k.values())[:3]
    check = {0, 127, 511}
    B, T, new = 4, 2048, 512
    _, _, tokens, logits, snaps, recs = run_gpu(cfg, kbits, vbits, 128, B, T, new, dev, sample, check, keep_prompt_out=False)
    assert tokens.shape == (B, new) and set(logits) == check
    assert all(np.isfinite(v).all() for v in logits.values())
    for li in sample:
        assert len(recs[li].calls) == new
        replay_layer(OracleAttention(oracle, kbits[li], vbits[li], 128, prompt_output=False), recs[li].calls, check,
                     snaps[li])
        tq = snaps[li][511][4].shape[2]
        assert tq == 1920 + 4 * 128  # prompt flush, then one 128-token flush at decode forwards 1, 129, 257, 385


def test_graph_replayed_steps_match_eager_steps(dev):
    """GraphDecoder (decode steps replayed from a captured HIP graph, device-side counters, fixed-size
    tail windows) against the eager Decoder fed the same tokens: every step's logits, through
    several flushes and re-captures; layer 0, whose inputs do not depend on the attention
    arithmetic, must end with a bit-identical cache."""
    from kvmix_amd.decoder import Decoder, DecoderConfig, GraphDecoder, init_weights, kvmix_layers

    cfg = DecoderConfig(hidden_size=512, num_layers=4, num_heads=4, num_kv_heads=2, intermediate_size=1024, vocab_size=1000)
    kbits, vbits, window = [4, 3, 2, 1], [2, 4, 3, 1], 64
    B, T, new = 2, 200, 300
    weights = init_weights(cfg, dev)
    gen = torch.Generator(device="cpu").manual_seed(41)
    prompt = torch.randint(0, cfg.vocab_size, (B, T), generator=gen).to(dev)

    atts, caches = kvmix_layers(cfg, kbits, vbits, residual_length=window, capacity=T + new)
    gd = GraphDecoder(cfg, weights, atts, caches)
    seen = []
    def keep(step, lg):
        seen.append(lg.clone())
        torch.cuda.synchronize()  # (a synchronisation and eager work between every two replays)

    tokens = gd.generate(prompt, new, keep)
    assert gd.graph_steps + gd.eager_steps == new and gd.graph_steps > 0.85 * new and gd.captures >= 4

    atts2, caches2 = kvmix_layers(cfg, kbits, vbits, residual_length=window, capacity=T + new)
    ed = Decoder(cfg, weights, atts2, caches2)
    ids = torch.cat([prompt, tokens], dim=1)
    for step in range(new):
        lg = ed.forward(ids[:, :T] if step == 0 else ids[:, T + step - 1:T + step])
        spread = float(lg.std())
        # two GPU evaluations of the same step: they differ by the fp16 rounding of the tail products
        # (fixed-size window against exact-size tail) and the order of the softmax sums
        assert float((lg - seen[step]).abs().max()) <= 0.01 * spread, step
    for li in range(cfg.num_layers):
        a, b = caches[li].as_tuple(), caches2[li].as_tuple()
        assert a[-1] == b[-1] == T + new - 1
        for x, y in zip(a[:-1], b[:-1]):
            assert x.shape == y.shape
            if li == 0:
                assert torch.equal(x, y)
    # deeper layers see inputs that differ in the last fp16 bits: nearly all codes still agree
    diff = caches[3].as_tuple()[4] ^ caches2[3].as_tuple()[4]  # 1-bit value codes
    assert float((diff != 0).sum()) / diff.numel() < 0.2


def test_graph_decoder_needs_a_fixed_window(dev):
    from kvmix_amd.decoder import DecoderConfig, GraphDecoder, kvmix_layers

    cfg = DecoderConfig(hidden_size=256, num_layers=1, num_heads=2, num_kv_heads=2, intermediate_size=256, vocab_size=10)
    atts, caches = kvmix_layers(cfg, [4], [4], residual_length=None)
    with pytest.raises(RuntimeError, match="fixed residual window"):
        GraphDecoder(cfg, {}, atts, caches)
