"""kvmix_amd.profiler on the GPU (the device the reference's recipe runs it on,
Inference-comparision.py:56-87): the scores of a 4-layer and a 20-layer model on cuda:0 against
the same model profiled in float64 on the CPU, and the quant_bits table that comes out."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _model(layers, dtype):
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=layers, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=100, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    torch.manual_seed(3)
    return LlamaForCausalLM(cfg).to(dtype)


def _prompts(n, length, dev, seed=1):
    g = torch.Generator().manual_seed(seed)
    ids = [torch.randint(0, 100, (1, length), generator=g).to(dev) for _ in range(n)]
    return ids, [torch.ones_like(i) for i in ids], [i.clone() for i in ids]


@pytest.mark.parametrize("layers", [4, 20])
def test_profile_on_gpu_matches_float64_cpu(dev, layers):
    from kvmix_amd.profiler import classify_layers, profile_importance, profile_model, set_quant_bits

    cpu = _model(layers, torch.float64)
    gpu = _model(layers, torch.float32).to(dev)
    gpu.load_state_dict({k: v.to(torch.float32) for k, v in cpu.state_dict().items()})
    ids_c, m_c, l_c = _prompts(3, 48, "cpu")
    ids_g, m_g, l_g = _prompts(3, 48, dev)
    k_c, v_c = profile_importance(cpu, ids_c, m_c, l_c, layers)
    k_g, v_g = profile_importance(gpu, ids_g, m_g, l_g, layers)
    assert k_g.dtype == torch.float64 and k_g.shape == (layers,) and not k_g.is_cuda
    # fp32 forward and backward on the GPU against float64 on the CPU
    torch.testing.assert_close(k_g, k_c, rtol=2e-3, atol=1e-7)
    torch.testing.assert_close(v_g, v_c, rtol=2e-3, atol=1e-7)
    qb = profile_model(gpu, ids_g, m_g, l_g, layers)
    assert sorted(qb) == list(range(layers))
    # the table that the CPU scores give, unless two scores are too close for fp32 to order them
    ks, vs = torch.sort(k_c, descending=True).values, torch.sort(v_c, descending=True).values
    if (ks[:-1] - ks[1:]).min() > 1e-2 * ks[0] and (vs[:-1] - vs[1:]).min() > 1e-2 * vs[0]:
        assert qb == set_quant_bits(*classify_layers(k_c, layers), *classify_layers(v_c, layers))
    n_top = int(0.1 * layers)
    assert sum(e["k_bits"] == 3 for e in qb.values()) == 2 * n_top
    assert sum(e["v_bits"] == 4 for e in qb.values()) == 2 * n_top
    assert all(e["k_bits"] in (2, 3) and e["v_bits"] in (2, 4) for e in qb.values())
    # the model is left in train mode with cleared gradients, as the reference leaves it
    assert gpu.training and all(p.grad is None for p in gpu.parameters())
