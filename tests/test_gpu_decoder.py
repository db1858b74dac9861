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
    """Wraps one layer's attention; keeps what went in and what came out (of a prompt call only the
    keys and values unless keep_prompt_out: the cache does not depend on the queries)."""

    def __init__(self, att, keep_prompt_out=True):
        self.att, self.calls, self.keep_prompt_out = att, [], keep_prompt_out

    def __call__(self, q, k, v, cache, attention_mask=None, need_weights=True):
        out, p, cache = self.att(q, k, v, cache, attention_mask=attention_mask, need_weights=need_weights)
        keep_out = self.keep_prompt_out or q.shape[2] == 1
        self.calls.append((q.contiguous().cpu().numpy() if keep_out else None, k.contiguous().cpu().numpy(),
                           v.contiguous().cpu().numpy(), out.cpu().numpy() if keep_out else None))
        return out, p, cache


class OracleAttention:
    """The oracle behind the attention-call signature, on CPU tensors.  3-bit values are kept in the
    dense 3-bit stream, as kvmix_layers sets the GPU caches up (the reference's 3-bit words cannot
    hold head_dim 128); 3-bit keys in the reference's words."""

    def __init__(self, oracle, k_bits, v_bits, window, group=32, prompt_output=True):
        self.o, self.k_bits, self.v_bits, self.window, self.group = oracle, k_bits, v_bits, window, group
        self.prompt_output = prompt_output
        self.v_dense3 = v_bits == 3

    def prompt(self, q, k, v, mask):
        from kvmix_amd.cache import flush_length

        o = self.o
        T, D = k.shape[2], k.shape[3]
        out = None
        if self.prompt_output:
            out, _ = o.attention_prompt(q, k, v, mask)
        kg = 11 if self.k_bits == 3 else self.group
        nk = flush_length(T, 0.0, kg, self.window, prompt=True)
        nv = flush_length(T, 0.0, self.group, self.window, prompt=True)
        kc = ks = km = vc = vs = vm = None
        if nk:
            kc, ks, km = o.quantize_pack_last_dim(np.ascontiguousarray(k[:, :, :nk].transpose(0, 1, 3, 2)), kg, self.k_bits)
        if nv and self.v_dense3:
            vc, vs, vm = o.quantize_pack_dense3(np.ascontiguousarray(v[:, :, :nv]), self.group)
        elif nv:
            vc, vs, vm = o.quantize_pack_last_dim(np.ascontiguousarray(v[:, :, :nv]), self.group, self.v_bits)
        return out, (kc, k[:, :, nk:], ks, km, vc, v[:, :, nv:], vs, vm, T)

    def step(self, q, k, v, cache, compute_output=True):
        return self.o.attention_decode_step(q, k, v, cache, self.k_bits, self.v_bits, 0.0, 0.0, group_size=self.group,
                                            fixed_window=self.window, v_dense3=self.v_dense3,
                                            compute_output=compute_output)

    def __call__(self, q, k, v, cache, attention_mask=None, need_weights=True):
        dt = q.dtype
        qn, kn, vn = (np.ascontiguousarray(t.to(torch.float16).numpy()) for t in (q, k, v))
        if cache is None:
            out, cache = self.prompt(qn, kn, vn, None if attention_mask is None else attention_mask.numpy())
        else:
            out, _, cache = self.step(qn, kn, vn, cache)
        return torch.from_numpy(out).to(dt), None, cache


def replay_layer(oracle_att, calls, check_steps, gpu_cache_at, output_steps=None):
    """Feed the recorded inputs of one layer to the oracle; compare outputs at every decode step (or
    only at those in output_steps -- the cache is brought up to date at every step either way)
    and caches at the steps in check_steps (gpu_cache_at[step] = the GPU cache tuple as numpy)."""
    cache = None
    worst = 0.0
    for step, (q, k, v, out_g) in enumerate(calls):
        if cache is None:
            mask = None
            if q is not None:
                mask = np.triu(np.full((q.shape[2],) * 2, np.finfo(np.float32).min, np.float32), 1)[None, None]
            out_o, cache = oracle_att.prompt(q, k, v, mask)
        else:
            out_o, _, cache = oracle_att.step(q, k, v, cache, output_steps is None or step in output_steps)
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
    kbits, vbits, window = [4, 3, 2, 1], [2, 3, 4, 1], 64  # (3-bit values: the dense stream)
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


class TorchFp32Attention:
    """Reference for the floating-point half of a decode step, in plain torch on the GPU: the cache is
    kept by the library (its codes are compared with the oracle's bit for bit elsewhere in this file),
    the step itself is dense fp32 attention over the cache dequantized with torch integer ops --
    no kernel of the library's product or softmax path runs."""

    def __init__(self, att):
        self.att = att

    def __call__(self, q, k, v, cache, attention_mask=None, need_weights=True):
        from helpers import dequantize_torch
        from kvmix_amd import ops

        if cache.kv_seq_len == 0:
            return self.att(q, k, v, cache, attention_mask=attention_mask, need_weights=need_weights)
        cache.append(k, v)
        kc, k_tail, ks, km, vc, v_tail, vs, vm, _ = cache.as_tuple()
        D = q.shape[-1]
        parts = []
        if kc is not None:
            kd = dequantize_torch(kc, ks, km, cache.k_bits, cache.Kgroup_size, cache.k_fmt == ops.FMT_DENSE3)  # [B,H,D,Tq]
            parts.append(torch.matmul(q.float(), kd))
        parts.append(torch.matmul(q.float(), k_tail.float().transpose(2, 3)))
        p = torch.softmax(torch.cat(parts, -1) / math.sqrt(D), -1)
        lv = v_tail.shape[2]
        out = torch.matmul(p[..., p.shape[-1] - lv:], v_tail.float())
        if vc is not None:
            vd = dequantize_torch(vc, vs, vm, cache.v_bits, cache.Vgroup_size, cache.v_fmt == ops.FMT_DENSE3)  # [B,H,Tq,D]
            out = out + torch.matmul(p[..., : p.shape[-1] - lv], vd)
        return out.to(q.dtype), None, cache


def test_llama2_7b_shape_decode_loop(oracle, dev):
    """BASELINE's end-to-end case at full size: random-init Llama-2-7B, prompt 2048, batch 4, 512 new
    tokens, mixed per-layer bits (3-bit values in the dense stream), 128-token window.
    Every one of the 32 layers is replayed on the oracle with the q/k/v the GPU run produced: caches
    compared bit for bit at forwards 1 (the prompt), 128 and 512, attention outputs at the decode
    forwards next to them; three layers (one per key width, one of them with 3-bit values) have the
    output of every decode step compared.  The logits of the same forwards are compared with a second
    run of the stack whose attention step is plain fp32 torch over the dequantized cache."""
    from bench import layer_bits
    from kvmix_amd.decoder import Decoder, DecoderConfig, kvmix_layers

    cfg = DecoderConfig()
    kbits, vbits = layer_bits(32)
    layers = list(range(32))
    full = {}
    for li in layers:  # one fully replayed layer per key width, preferring 3-bit values
        if kbits[li] not in full or (vbits[li] == 3 and vbits[full[kbits[li]]] != 3):
            full[kbits[li]] = li
    full = set(full.values())
    assert any(vbits[li] == 3 for li in full) and any(kbits[li] == 3 for li in full)
    check = {0, 127, 511}
    near = {1, 2, 127, 128, 129, 511}
    B, T, new = 4, 2048, 512
    weights, prompt, tokens, logits, snaps, recs = run_gpu(cfg, kbits, vbits, 128, B, T, new, dev, layers, check,
                                                           keep_prompt_out=False)
    assert tokens.shape == (B, new) and set(logits) == check
    assert all(np.isfinite(v).all() for v in logits.values())
    for li in layers:
        assert len(recs[li].calls) == new
        replay_layer(OracleAttention(oracle, kbits[li], vbits[li], 128, prompt_output=False), recs[li].calls, check,
                     snaps[li], output_steps=None if li in full else near)
        tq = snaps[li][511][4].shape[2]
        assert tq == 1920 + 4 * 128  # prompt flush, then one 128-token flush at decode forwards 1, 129, 257, 385
        recs[li].calls.clear()
    del recs, snaps

    # logits: the same stack and tokens with the fp32 torch attention step
    atts, caches = kvmix_layers(cfg, kbits, vbits, residual_length=128, capacity=T + new)
    ref = Decoder(cfg, weights, [TorchFp32Attention(a) for a in atts], caches)
    ids = torch.cat([prompt, tokens], dim=1)
    worst = {}
    for step in range(new):
        lg = ref.forward(ids[:, :T] if step == 0 else ids[:, T + step - 1:T + step])
        if step in check:
            want, got = lg.cpu().numpy().astype(np.float64), logits[step].astype(np.float64)
            spread = float(want.std())
            err = np.abs(got - want)
            print(f"forward {step + 1}: logits max {err.max() / spread:.4f} rms {np.sqrt((err ** 2).mean()) / spread:.4f} of their spread")
            # the two runs share weights, tokens and quantizer and differ in the attention arithmetic (fp16
            # logits and probabilities against fp32) and, through it, in what the later layers cache: a value
            # next to a rounding boundary gets the neighbouring code (a full step of a 2-bit layer), 32 layers
            # deep.  Measured: 5 % of the spread at most, 1 % rms; the prompt forward is identical.
            worst[step] = (err.max() / spread, np.sqrt((err ** 2).mean()) / spread)
    for step, (mx, rms) in worst.items():
        assert mx <= 0.10 and rms <= 0.025, (step, mx, rms)
    assert worst[0][0] <= 1e-6


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


def test_graph_decoder_needs_one_flush_policy(dev):
    from kvmix_amd.decoder import DecoderConfig, GraphDecoder, kvmix_layers

    cfg = DecoderConfig(hidden_size=256, num_layers=2, num_heads=2, num_kv_heads=2, intermediate_size=256, vocab_size=10)
    atts, caches = kvmix_layers(cfg, [4, 4], [4, 4], residual_length=None)
    _, fixed = kvmix_layers(cfg, [4, 4], [4, 4], residual_length=64)
    with pytest.raises(RuntimeError, match="one flush policy"):
        GraphDecoder(cfg, {}, atts, [caches[0], fixed[1]])


def test_graph_replayed_steps_under_the_ratio_flush_rule(dev):
    """The reference's own flush rule (keep int(ratio * L) tail tokens, quantize the rest in whole groups:
    models/modeling_llama_KVmix.py:119-127,152-155) under graph replay: the tails stay short and flush every few
    steps (every 14 tokens with the reference's 3-bit keys), every flushing step runs eagerly and the graph is
    captured again with a window sized for the tails of that moment.  Against the eager decoder fed the same
    tokens: every step's logits, and the caches -- the same quantized lengths everywhere, layer 0 bit for bit."""
    from kvmix_amd.decoder import Decoder, DecoderConfig, GraphDecoder, init_weights, kvmix_layers

    cfg = DecoderConfig(hidden_size=512, num_layers=4, num_heads=4, num_kv_heads=2, intermediate_size=1024, vocab_size=1000)
    kbits, vbits = [4, 3, 2, 1], [2, 4, 3, 1]
    B, T, new = 2, 150, 120
    weights = init_weights(cfg, dev)
    gen = torch.Generator(device="cpu").manual_seed(43)
    prompt = torch.randint(0, cfg.vocab_size, (B, T), generator=gen).to(dev)

    atts, caches = kvmix_layers(cfg, kbits, vbits, residual_length=None, capacity=T + new)
    gd = GraphDecoder(cfg, weights, atts, caches)
    seen = []
    def keep(step, lg):
        seen.append(lg.clone())
        torch.cuda.synchronize()

    tokens = gd.generate(prompt, new, keep)
    assert gd.graph_steps + gd.eager_steps == new and gd.graph_steps > 0.5 * new and gd.captures >= 5, \
        (gd.graph_steps, gd.eager_steps, gd.captures)

    atts2, caches2 = kvmix_layers(cfg, kbits, vbits, residual_length=None, capacity=T + new)
    ed = Decoder(cfg, weights, atts2, caches2)
    ids = torch.cat([prompt, tokens], dim=1)
    for step in range(new):
        lg = ed.forward(ids[:, :T] if step == 0 else ids[:, T + step - 1:T + step])
        assert float((lg - seen[step]).abs().max()) <= 0.01 * float(lg.std()), step
    for li in range(cfg.num_layers):
        a, b = caches[li].as_tuple(), caches2[li].as_tuple()
        assert a[-1] == b[-1] == T + new - 1
        assert (caches[li].k_tokens, caches[li].v_tokens) == (caches2[li].k_tokens, caches2[li].v_tokens)
        for x, y in zip(a[:-1], b[:-1]):
            assert x.shape == y.shape
            if li == 0:
                assert torch.equal(x, y)
