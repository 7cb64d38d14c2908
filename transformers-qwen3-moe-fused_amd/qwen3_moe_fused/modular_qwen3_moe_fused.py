"""Fused MoE modules (reference: qwen3_moe_fused/modular_qwen3_moe_fused.py).

``MoeFusedLinear`` keeps all experts of one projection in a single (E, out, in) parameter and
applies them with one grouped GEMM; ``Qwen3MoeFusedSparseMoeBlock`` is the whole sparse MLP:
router -> softmax/top-k -> stable expert sort -> gate/up GEMMs -> SiLU*mul -> down GEMM ->
un-sort + routing-weighted sum.  Parameter names and shapes match the reference so state dicts
load unchanged.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
from torch import nn

from .functional import moe_fused_linear
from .kernels.routing import combine_rows, gather_rows, route_and_sort
from .kernels.silu_mul import silu_mul


def moe_fused_kaiming_uniform_(weight: torch.Tensor) -> None:
    """Kaiming-uniform over in_features with gain a = sqrt(5), as nn.Linear initialises
    (modular_qwen3_moe_fused.py:21-26): U(-b, b) with b = sqrt(15 / in_features)."""
    fan_in = weight.shape[-1]
    limit = math.sqrt(15.0 / fan_in)
    with torch.no_grad():
        weight.uniform_(-limit, limit)


class MoeFusedLinear(nn.Module):
    __constants__ = ["in_features", "out_features", "num_experts"]

    def __init__(self, in_features: int, out_features: int, num_experts: int,
                 device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None) -> None:
        super().__init__()
        self.in_features, self.out_features, self.num_experts = in_features, out_features, num_experts
        self.weight = nn.Parameter(torch.empty((num_experts, out_features, in_features), device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        moe_fused_kaiming_uniform_(self.weight)

    def forward(self, input: torch.Tensor, m_sizes: torch.Tensor) -> torch.Tensor:
        return moe_fused_linear(input, self.weight, m_sizes)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, num_experts={self.num_experts}"


def route_tokens(block, hidden_2d: torch.Tensor):
    """Router half of the block, shared with the fast-LoRA forward: returns
    (router_logits, routing_weights (T,k), m_sizes, sort_idx, inv_sort_idx)."""
    router_logits = block.gate(hidden_2d)
    routing_weights, selected, m_sizes, sort_idx, inv_sort_idx = route_and_sort(
        router_logits.contiguous(), block.num_selected, block.norm_topk_prob, hidden_2d.dtype, block.num_experts)
    if getattr(block, "keep_routing", False):
        block.last_selected = selected  # (T, k) expert ids of this call, as the top-k kernel wrote them
    return router_logits, routing_weights, m_sizes, sort_idx, inv_sort_idx


class Qwen3MoeFusedRouter(nn.Linear):
    """The block's ``gate``: a plain bias-free linear layer (modular_qwen3_moe_fused.py:72 of the
    reference) under a class name of its own, so that transformers releases that collect
    ``router_logits`` with a forward hook on the router module (instead of from the block's return
    value, as the reference's release did) have a class to hook: its output is the raw logits."""


class Qwen3MoeFusedSparseMoeBlock(nn.Module):
    """``config`` needs: num_experts, num_experts_per_tok, norm_topk_prob, hidden_size,
    moe_intermediate_size, hidden_act == "silu" (a transformers ``Qwen3MoeConfig`` has them)."""

    def __init__(self, config) -> None:
        super().__init__()
        assert config.hidden_act == "silu"
        self.num_experts = config.num_experts
        self.num_selected = config.num_experts_per_tok
        self.norm_topk_prob = config.norm_topk_prob
        self.hidden_size = config.hidden_size
        self.moe_intermediate_size = config.moe_intermediate_size
        self.gate = Qwen3MoeFusedRouter(self.hidden_size, self.num_experts, bias=False)
        self.gate_proj = MoeFusedLinear(self.hidden_size, self.moe_intermediate_size, self.num_experts)
        self.up_proj = MoeFusedLinear(self.hidden_size, self.moe_intermediate_size, self.num_experts)
        self.down_proj = MoeFusedLinear(self.moe_intermediate_size, self.hidden_size, self.num_experts)

    # gather + gate_proj + up_proj + SiLU-mul as one kernel when both projections are plain (or
    # plain 4-bit) expert matrices in bf16; set to False to call the two modules one by one
    fuse_front = True
    # with fuse_front: set to True for the three projections as one node of the autograd graph, whose backward runs
    # the gated unit's backward inside the down projection's input gradient (dh is never written: 50 MB less memory
    # at 32768 routed rows).  Off by default: the kernel's epilogue then does the unit's arithmetic with the matrix
    # units idle, and a training step of the block takes 1.62-1.67 ms instead of 1.58-1.63 ms.
    fuse_backward = False
    # set to True to keep the expert ids of the last call in ``last_selected`` (tests read the block's own routing)
    keep_routing = False

    def _fused_front(self, tokens, m_sizes, sort_idx, inv_sort_idx) -> Optional[torch.Tensor]:
        from .fused_mlp import moe_fused_glu, moe_fused_glu_4bit
        from .quantize.layer import MoeFusedLinear4bit

        gate, up = self.gate_proj, self.up_proj
        if tokens.dtype != torch.bfloat16 or type(gate) is not type(up):
            return None
        if type(gate) is MoeFusedLinear:
            if gate.weight.dtype != torch.bfloat16 or up.weight.dtype != torch.bfloat16:
                return None
            return moe_fused_glu(tokens, gate.weight, up.weight, m_sizes, sort_idx, inv_sort_idx, self.num_selected)
        if type(gate) is MoeFusedLinear4bit:
            for proj in (gate, up):
                if getattr(proj.weight, "quant_state", None) is None or proj.compute_dtype not in (None, torch.bfloat16):
                    return None
            return moe_fused_glu_4bit(tokens, gate.weight, up.weight, m_sizes, sort_idx, inv_sort_idx,
                                      self.num_selected)
        return None

    def _fused_mlp(self, tokens, m_sizes, sort_idx, inv_sort_idx) -> Optional[torch.Tensor]:
        """The three projections as one node of the graph when all are plain bf16 expert matrices and a gradient
        will be asked for: the backward then runs the gated unit's backward inside the down projection's input
        gradient.  Without gradients the front half and the down projection are the same two launches anyway."""
        from .fused_mlp import moe_fused_mlp

        projs = (self.gate_proj, self.up_proj, self.down_proj)
        if not self.fuse_backward or tokens.dtype != torch.bfloat16 or not torch.is_grad_enabled():
            return None
        if any(type(p) is not MoeFusedLinear or p.weight.dtype != torch.bfloat16 for p in projs):
            return None
        if not (tokens.requires_grad or any(p.weight.requires_grad for p in projs)):
            return None
        return moe_fused_mlp(tokens, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, m_sizes,
                             sort_idx, inv_sort_idx, self.num_selected)

    def forward(self, hidden_states: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        batch, seq, hidden = hidden_states.shape
        tokens = hidden_states.reshape(batch * seq, hidden).contiguous()
        router_logits, routing_weights, m_sizes, sort_idx, inv_sort_idx = route_tokens(self, tokens)

        y = self._fused_mlp(tokens, m_sizes, sort_idx, inv_sort_idx) if self.fuse_front else None
        if y is None:
            h = self._fused_front(tokens, m_sizes, sort_idx, inv_sort_idx) if self.fuse_front else None
            if h is None:
                # every token once per selected expert, rows grouped by expert
                x = gather_rows(tokens, sort_idx, self.num_selected, inv_sort_idx)
                h = silu_mul(self.gate_proj(x, m_sizes), self.up_proj(x, m_sizes))
            y = self.down_proj(h, m_sizes)
        out = combine_rows(y, inv_sort_idx, routing_weights, sort_idx)
        return out.view(batch, seq, hidden), router_logits


def _hf_subclasses():
    """Model-level wiring (decoder layer / model / causal LM with the fused block swapped in),
    built on demand so that importing this module does not import transformers."""
    import inspect

    from transformers.models.qwen3_moe.modeling_qwen3_moe import (Qwen3MoeDecoderLayer, Qwen3MoeForCausalLM,
                                                                  Qwen3MoeMLP, Qwen3MoeModel, Qwen3MoeSparseMoeBlock)

    # The reference was written against a transformers revision whose sparse block returns
    # (hidden_states, router_logits) (modular_qwen3_moe_fused.py:1,118); later releases return the
    # hidden states alone and the decoder layer adds them to the residual as they come.
    block_cls = Qwen3MoeFusedSparseMoeBlock
    if inspect.signature(Qwen3MoeSparseMoeBlock.forward).return_annotation is torch.Tensor:
        class _TensorBlock(Qwen3MoeFusedSparseMoeBlock):
            def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
                return super().forward(hidden_states)[0]

        block_cls = _TensorBlock

    class Qwen3MoeFusedDecoderLayer(Qwen3MoeDecoderLayer):
        def __init__(self, config, layer_idx: int) -> None:
            super().__init__(config, layer_idx)
            sparse = (layer_idx not in config.mlp_only_layers and config.num_experts > 0
                      and (layer_idx + 1) % config.decoder_sparse_step == 0)
            self.mlp = (block_cls(config) if sparse
                        else Qwen3MoeMLP(config, intermediate_size=config.intermediate_size))

    # Releases that record outputs through forward hooks take the router logits from the stock router
    # class; the fused block's router is hooked the same way (output_router_logits, the auxiliary
    # load-balancing loss).  Older releases read them from the block's return value and have no table.
    record = {}
    if isinstance(getattr(Qwen3MoeModel, "_can_record_outputs", None), dict):
        # the recorder class has lived in two places; without it the model classes still build and the router
        # logits come from the block's return value only
        OutputRecorder = None
        for module in ("transformers.utils.output_capturing", "transformers.utils.generic"):
            try:
                OutputRecorder = getattr(__import__(module, fromlist=["OutputRecorder"]), "OutputRecorder")
                break
            except (ImportError, AttributeError):
                continue
        if OutputRecorder is not None:
            record = {"_can_record_outputs": {**Qwen3MoeModel._can_record_outputs,
                                              "router_logits": OutputRecorder(Qwen3MoeFusedRouter, index=0)}}

    class Qwen3MoeFusedModel(Qwen3MoeModel):
        locals().update(record)

        def __init__(self, config) -> None:
            super().__init__(config)
            self.layers = nn.ModuleList(Qwen3MoeFusedDecoderLayer(config, i) for i in range(config.num_hidden_layers))

    class Qwen3MoeFusedForCausalLM(Qwen3MoeForCausalLM):
        locals().update(record)

        def __init__(self, config) -> None:
            super().__init__(config)
            self.model = Qwen3MoeFusedModel(config)

    return Qwen3MoeFusedDecoderLayer, Qwen3MoeFusedModel, Qwen3MoeFusedForCausalLM


def __getattr__(name: str):
    names = ("Qwen3MoeFusedDecoderLayer", "Qwen3MoeFusedModel", "Qwen3MoeFusedForCausalLM")
    if name in names:
        classes = dict(zip(names, _hf_subclasses()))
        globals().update(classes)
        return classes[name]
    raise AttributeError(name)
