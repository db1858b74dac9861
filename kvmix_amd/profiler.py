"""Per-layer bit-width assignment from gradient norms: the step that produces `quant_bits`.

Same functions, arguments and results as the reference's myprofileKV.py:13-115
(`profile_importance`, `classify_layers`, `set_quant_bits`, `profile_model`), which
Inference-comparision.py:56-87 runs on the stock fp16/fp32 model before loading the KVmix one:

  score_K[layer] = mean over prompts of || d loss / d W_k[layer] ||_2      (likewise V),
  the top int(0.1 L) layers by score are "important", the next int(0.1 L) "general", the rest
  "unimportant"; keys get 3 / 3 / 2 bits, values 4 / 4 / 2, and every width brings its fixed
  fp16 residual ratio.

One difference in how, none in what: the reference runs one forward and two backward passes per
layer and prompt (2 L backward passes over the same loss); the gradients of different weights do
not interact, so this runs one forward and one backward per prompt and reads all 2 L norms from
it.  Plain PyTorch autograd on whatever device the model is on; no kernels of this library are
involved (the model profiled is the stock one, without a quantized cache)."""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import torch

from .cache import RESIDUAL_RATIO_BY_BITS

# myprofileKV.py:83-97: bits for (important, general, unimportant) layers
K_BITS_BY_CLASS = (3, 3, 2)
V_BITS_BY_CLASS = (4, 4, 2)


def profile_importance(model, input_ids_list: Sequence[torch.Tensor], attention_mask_list: Sequence[torch.Tensor],
                       labels_list: Sequence[torch.Tensor], num_layers: int, max_length: int = 1024
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """(k_scores [L], v_scores [L]) as float64 tensors: the L2 norm of the loss gradient with respect
    to each layer's k_proj / v_proj weight, averaged over the prompts (myprofileKV.py:13-57).
    Prompts longer than max_length are cut to it.  Leaves the model in train mode with cleared
    gradients, as the reference does."""
    layers = model.model.layers
    weights = [layers[i].self_attn.k_proj.weight for i in range(num_layers)] + \
              [layers[i].self_attn.v_proj.weight for i in range(num_layers)]
    totals = torch.zeros(2 * num_layers, dtype=torch.float64)
    model.train()
    for input_ids, attention_mask, labels in zip(input_ids_list, attention_mask_list, labels_list):
        if input_ids.size(1) > max_length:
            input_ids, attention_mask, labels = input_ids[:, :max_length], attention_mask[:, :max_length], labels[:, :max_length]
        model.zero_grad(set_to_none=True)
        loss = model(input_ids=input_ids, attention_mask=attention_mask, labels=labels).loss
        grads = torch.autograd.grad(loss, weights, allow_unused=True)
        totals += torch.tensor([0.0 if g is None else g.norm(2).item() for g in grads], dtype=torch.float64)
        del loss, grads
    model.zero_grad(set_to_none=True)
    scores = totals / max(len(input_ids_list), 1)
    return scores[:num_layers].clone(), scores[num_layers:].clone()


def classify_layers(importance_scores: torch.Tensor, num_layers: int) -> Tuple[List[int], List[int], List[int]]:
    """(important, general, unimportant) layer indices by descending score: int(0.1 L), int(0.1 L)
    and the rest (myprofileKV.py:59-67; the shares are the code's, not its docstring's)."""
    order = torch.argsort(importance_scores, descending=True).tolist()
    n_important = int(0.1 * num_layers)
    n_general = int(0.1 * num_layers)
    return order[:n_important], order[n_important:n_important + n_general], order[n_important + n_general:]


def set_quant_bits(k_important, k_general, k_unimportant, v_important, v_general, v_unimportant) -> Dict[int, dict]:
    """The per-layer dictionary the model classes take (myprofileKV.py:70-105)."""
    total = len(k_important) + len(k_general) + len(k_unimportant)
    k_class = {**{i: 2 for i in k_unimportant}, **{i: 1 for i in k_general}, **{i: 0 for i in k_important}}
    v_class = {**{i: 2 for i in v_unimportant}, **{i: 1 for i in v_general}, **{i: 0 for i in v_important}}
    quant_bits = {}
    for layer in range(total):
        k_bits = K_BITS_BY_CLASS[k_class.get(layer, 2)]
        v_bits = V_BITS_BY_CLASS[v_class.get(layer, 2)]
        quant_bits[layer] = {"k_bits": k_bits, "v_bits": v_bits,
                             "k_residual_ratio": RESIDUAL_RATIO_BY_BITS[k_bits],
                             "v_residual_ratio": RESIDUAL_RATIO_BY_BITS[v_bits]}
    return quant_bits


def profile_model(model, input_ids_list, attention_mask_list, labels_list, num_layers: int) -> Dict[int, dict]:
    """myprofileKV.py:108-115: scores -> classes -> quant_bits."""
    k_scores, v_scores = profile_importance(model, input_ids_list, attention_mask_list, labels_list, num_layers,
                                            max_length=1024)
    return set_quant_bits(*classify_layers(k_scores, num_layers), *classify_layers(v_scores, num_layers))
