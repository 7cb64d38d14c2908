"""Block forward that routes the LoRA-wrapped expert MLP through the single ``fast_lora``
autograd function (reference: qwen3_moe_fused/fast_lora.py)."""
from __future__ import annotations

from typing import Any, Optional

import torch
from torch import nn

from .kernels.fast_lora import fast_lora
from .kernels.routing import combine_rows, gather_rows
from .modular_qwen3_moe_fused import Qwen3MoeFusedSparseMoeBlock, route_tokens


def get_lora_parameters(proj: nn.Module) -> tuple[torch.Tensor, Optional[Any], torch.Tensor, torch.Tensor, float]:
    """(base weight, its quant state or None, lora_A weight, lora_B weight, scaling) of a
    LoRA-wrapped projection with exactly one active, unmerged adapter and no dropout
    (fast_lora.py:13-36)."""
    if getattr(proj, "disable_adapters", False) or getattr(proj, "merged", False):
        raise NotImplementedError("fast LoRA needs the adapter enabled and unmerged")
    base = getattr(proj, "base_layer", proj)
    weight = base.weight
    active = getattr(proj, "active_adapters", None)
    if active is None:
        name = getattr(proj, "active_adapter", "default")
    else:
        assert len(active) == 1, "fast LoRA handles one adapter"
        name = active[0]
    assert isinstance(proj.lora_dropout[name], nn.Identity), "fast LoRA does not apply dropout"
    return (weight, getattr(weight, "quant_state", None), proj.lora_A[name].weight, proj.lora_B[name].weight,
            proj.scaling[name])


def fast_Qwen3MoeFusedSparseMoeBlock_forward(self: Qwen3MoeFusedSparseMoeBlock,
                                             hidden_states: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    batch, seq, hidden = hidden_states.shape
    tokens = hidden_states.reshape(batch * seq, hidden).contiguous()
    router_logits, routing_weights, m_sizes, sort_idx, inv_sort_idx = route_tokens(self, tokens)
    x = gather_rows(tokens, sort_idx, self.num_selected, inv_sort_idx)
    y = fast_lora(x, *get_lora_parameters(self.gate_proj), *get_lora_parameters(self.up_proj),
                  *get_lora_parameters(self.down_proj), m_sizes)
    out = combine_rows(y, inv_sort_idx, routing_weights, sort_idx)
    return out.view(batch, seq, hidden), router_logits


def patch_Qwen3MoeFusedSparseMoeBlock_forward() -> None:
    Qwen3MoeFusedSparseMoeBlock.forward = fast_Qwen3MoeFusedSparseMoeBlock_forward
