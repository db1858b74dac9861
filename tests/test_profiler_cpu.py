"""kvmix_amd.profiler against what fixes its results without the reference running:
the class sizes and bit tables of myprofileKV.py:59-105 as hand-worked cases, the scores as
gradient norms (a central finite difference along the gradient equals its norm only if the
gradient is right), and the one-backward shortcut against the per-layer procedure of
myprofileKV.py:29-44 carried out with torch's ordinary backward()."""
import pytest
import torch


def _model(layers=4, dtype=torch.float64):
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(hidden_size=32, intermediate_size=64, num_hidden_layers=layers, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=50, max_position_embeddings=128)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg).to(dtype)


def _prompts(n, length, seed=1):
    g = torch.Generator().manual_seed(seed)
    ids = [torch.randint(0, 50, (1, length), generator=g) for _ in range(n)]
    return ids, [torch.ones_like(i) for i in ids], [i.clone() for i in ids]


def _loss64(model, ids, mask):
    """Next-token cross entropy in the model's own precision (the model's `.loss` is computed in
    fp32, too coarse for a finite difference)."""
    logits = model(input_ids=ids, attention_mask=mask).logits
    return torch.nn.functional.cross_entropy(logits[0, :-1], ids[0, 1:])


def test_classes_and_bit_table():
    from kvmix_amd.profiler import classify_layers, set_quant_bits

    scores = torch.arange(32, dtype=torch.float64)          # layer 31 matters most
    imp, gen, rest = classify_layers(scores, 32)
    assert imp == [31, 30, 29] and gen == [28, 27, 26] and rest == list(range(25, -1, -1))
    assert classify_layers(torch.tensor([3.0, 1.0, 2.0]), 3) == ([], [], [0, 2, 1])  # int(0.3) = 0
    qb = set_quant_bits([31, 30, 29], [28, 27, 26], list(range(26)), [0, 1, 2], [3, 4, 5], list(range(6, 32)))
    assert len(qb) == 32
    assert qb[31] == {"k_bits": 3, "v_bits": 2, "k_residual_ratio": 0.2, "v_residual_ratio": 0.2}
    assert qb[27] == {"k_bits": 3, "v_bits": 2, "k_residual_ratio": 0.2, "v_residual_ratio": 0.2}
    assert qb[0] == {"k_bits": 2, "v_bits": 4, "k_residual_ratio": 0.2, "v_residual_ratio": 0.3}
    assert qb[4] == {"k_bits": 2, "v_bits": 4, "k_residual_ratio": 0.2, "v_residual_ratio": 0.3}
    assert qb[10] == {"k_bits": 2, "v_bits": 2, "k_residual_ratio": 0.2, "v_residual_ratio": 0.2}
    assert sum(e["k_bits"] == 3 for e in qb.values()) == 6 and sum(e["v_bits"] == 4 for e in qb.values()) == 6


def test_scores_are_gradient_norms():
    from kvmix_amd.profiler import profile_importance

    model = _model()
    ids, masks, labels = _prompts(1, 24)
    k, v = profile_importance(model, ids, masks, labels, 4)
    assert k.shape == (4,) and v.shape == (4,) and bool((k > 0).all()) and bool((v > 0).all())
    model.zero_grad()
    model(input_ids=ids[0], attention_mask=masks[0], labels=labels[0]).loss.backward()
    for layer, proj, score in [(0, "k_proj", k[0]), (3, "k_proj", k[3]), (2, "v_proj", v[2])]:
        w = getattr(model.model.layers[layer].self_attn, proj).weight
        g = w.grad.clone()
        assert abs(float(g.norm()) - float(score)) <= 1e-6 * float(score)
        # the stock attention rounds its softmax to fp32 even in an fp64 model, so the loss carries
        # ~1e-8 of noise: a step large enough to stand above it, and a tolerance to match
        eps, d = 3e-3, g / g.norm()
        with torch.no_grad():
            w.add_(eps * d)
            up = float(_loss64(model, ids[0], masks[0]))
            w.sub_(2 * eps * d)
            down = float(_loss64(model, ids[0], masks[0]))
            w.add_(eps * d)
        assert abs((up - down) / (2 * eps) - float(score)) <= 2e-3 * float(score)


def test_one_backward_equals_the_per_layer_procedure_and_prompts_are_averaged():
    from kvmix_amd.profiler import profile_importance

    model = _model(layers=3)
    ids, masks, labels = _prompts(3, 40)
    ids[1], masks[1], labels[1] = (torch.cat([t, t], 1) for t in (ids[1], masks[1], labels[1]))  # 80 tokens, cut to 48
    k, v = profile_importance(model, ids, masks, labels, 3, max_length=48)
    assert model.training and all(p.grad is None for p in model.parameters())
    want_k, want_v = torch.zeros(3, dtype=torch.float64), torch.zeros(3, dtype=torch.float64)
    for i, m, l in zip(ids, masks, labels):
        i, m, l = i[:, :48], m[:, :48], l[:, :48]
        for layer in range(3):
            for proj, acc in (("k_proj", want_k), ("v_proj", want_v)):
                model.zero_grad()
                loss = model(input_ids=i, attention_mask=m, labels=l).loss
                w = getattr(model.model.layers[layer].self_attn, proj).weight
                loss.backward(inputs=[w])
                acc[layer] += float(w.grad.norm(2))
    torch.testing.assert_close(k, want_k / 3, rtol=1e-12, atol=0)
    torch.testing.assert_close(v, want_v / 3, rtol=1e-12, atol=0)


def test_profile_model_end_to_end():
    from kvmix_amd.hf import normalise_quant_bits
    from kvmix_amd.profiler import classify_layers, profile_importance, profile_model

    model = _model(layers=20, dtype=torch.float32)
    ids, masks, labels = _prompts(2, 32)
    qb = profile_model(model, ids, masks, labels, 20)
    k, v = profile_importance(model, ids, masks, labels, 20)
    k_top = set(classify_layers(k, 20)[0] + classify_layers(k, 20)[1])
    v_top = set(classify_layers(v, 20)[0] + classify_layers(v, 20)[1])
    assert len(k_top) == 4 and len(v_top) == 4
    assert {i for i, e in qb.items() if e["k_bits"] == 3} == k_top and {i for i, e in qb.items() if e["v_bits"] == 4} == v_top
    assert all(e["k_bits"] in (2, 3) and e["v_bits"] in (2, 4) for e in qb.values())
    assert normalise_quant_bits(qb, 20) == qb  # what the model classes take, unchanged
