"""Front half of the sparse MLP block as one differentiable op:

    h = silu(xg @ w_gate[e]^T) * (xg @ w_up[e]^T),   xg = tokens[sort_idx // num_selected]

i.e. qwen3_moe_fused/modular_qwen3_moe_fused.py:95-108 (replicate, sort, gate_proj, up_proj,
SiLU-mul) in a single kernel launch; the reference names both fusions as possible (:101, :105).
The forward keeps the two products only when a gradient will be asked for; the backward
re-gathers the token rows instead of keeping a (rows, hidden) copy alive.
"""
from __future__ import annotations

import torch

from .grouped_gemm.backward_dw import grouped_gemm_backward_dw
from .grouped_gemm.forward import grouped_gemm_forward
from .grouped_gemm.fused import (grouped_gemm_forward_transposed_dual, grouped_gemm_forward_transposed_silu_bwd,
                                 grouped_glu_forward, grouped_glu_forward_4bit)
from .kernels.routing import _combine, _gather, _scatter
from .kernels.silu_mul import silu_mul_backward
from .grouped_gemm.forward_4bit import grouped_gemm_forward_transposed_4bit


class _GluGathered(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tokens, w_gate, w_up, m_sizes, sort_idx, inv_sort_idx, k):
        need = any(ctx.needs_input_grad[:3])
        out = grouped_glu_forward(tokens, w_gate, w_up, m_sizes, sort_idx, k, return_products=need)
        if not need:
            return out
        h, e, g = out
        ctx.save_for_backward(tokens, w_gate, w_up, m_sizes, sort_idx, inv_sort_idx, e, g)
        ctx.k = k
        return h

    @staticmethod
    def backward(ctx, dh):
        tokens, w_gate, w_up, m_sizes, sort_idx, inv_sort_idx, e, g = ctx.saved_tensors
        de, dg = silu_mul_backward(dh.contiguous(), e, g)
        d_tokens = d_gate = d_up = None
        if ctx.needs_input_grad[0]:
            # both terms of the input gradient in one reduction (one rounding), then each token's
            # k rows are summed
            dx = grouped_gemm_forward_transposed_dual(de, w_gate, dg, w_up, m_sizes, tokens.dtype)
            d_tokens = _combine(dx, inv_sort_idx, None, tokens.shape[0], ctx.k)
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            # the replicated, sorted rows again (the forward pass never wrote them), from the source's side: every
            # token row is read once and written k times
            xg = _scatter(tokens, inv_sort_idx, ctx.k, None) if ctx.k > 1 else _gather(tokens, sort_idx, ctx.k, None)
            if ctx.needs_input_grad[1]:
                d_gate = grouped_gemm_backward_dw(xg, de, m_sizes, w_gate.dtype)
            if ctx.needs_input_grad[2]:
                d_up = grouped_gemm_backward_dw(xg, dg, m_sizes, w_up.dtype)
        return d_tokens, d_gate, d_up, None, None, None, None


def moe_fused_glu(tokens: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, m_sizes: torch.Tensor,
                  sort_idx: torch.Tensor, inv_sort_idx: torch.Tensor, num_selected: int) -> torch.Tensor:
    """``tokens`` (T, hidden); ``w_gate``, ``w_up`` (E, intermediate, hidden); ``sort_idx`` /
    ``inv_sort_idx`` (T * num_selected,) int32 as ``get_expert_counts_and_idx`` returns them.
    Result (T * num_selected, intermediate), rows grouped by expert.  Differentiable in
    ``tokens``, ``w_gate`` and ``w_up``."""
    return _GluGathered.apply(tokens, w_gate, w_up, m_sizes, sort_idx, inv_sort_idx, num_selected)


class _MlpGathered(torch.autograd.Function):
    """``moe_fused_glu`` followed by the down projection, as one node of the graph: its backward runs the down
    projection's input gradient with the gated unit's backward in the epilogue (``dh`` is never written), then
    what ``_GluGathered.backward`` runs."""

    @staticmethod
    def forward(ctx, tokens, w_gate, w_up, w_down, m_sizes, sort_idx, inv_sort_idx, k):
        need = any(ctx.needs_input_grad[:4])
        out = grouped_glu_forward(tokens, w_gate, w_up, m_sizes, sort_idx, k, return_products=need)
        h, e, g = out if need else (out, None, None)
        y = grouped_gemm_forward(h, w_down, m_sizes)
        if need:
            ctx.save_for_backward(tokens, w_gate, w_up, w_down, m_sizes, sort_idx, inv_sort_idx, e, g, h)
            ctx.k = k
        return y

    @staticmethod
    def backward(ctx, dy):
        tokens, w_gate, w_up, w_down, m_sizes, sort_idx, inv_sort_idx, e, g, h = ctx.saved_tensors
        dy = dy.contiguous()
        d_tokens = d_gate = d_up = d_down = None
        if ctx.needs_input_grad[3]:
            d_down = grouped_gemm_backward_dw(h, dy, m_sizes, w_down.dtype)
        if any(ctx.needs_input_grad[:3]):
            de, dg = grouped_gemm_forward_transposed_silu_bwd(dy, w_down, e, g, m_sizes)
            if ctx.needs_input_grad[0]:
                dx = grouped_gemm_forward_transposed_dual(de, w_gate, dg, w_up, m_sizes, tokens.dtype)
                d_tokens = _combine(dx, inv_sort_idx, None, tokens.shape[0], ctx.k)
            if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
                xg = _scatter(tokens, inv_sort_idx, ctx.k, None) if ctx.k > 1 else _gather(tokens, sort_idx, ctx.k, None)
                if ctx.needs_input_grad[1]:
                    d_gate = grouped_gemm_backward_dw(xg, de, m_sizes, w_gate.dtype)
                if ctx.needs_input_grad[2]:
                    d_up = grouped_gemm_backward_dw(xg, dg, m_sizes, w_up.dtype)
        return d_tokens, d_gate, d_up, d_down, None, None, None, None


def moe_fused_mlp(tokens: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                  m_sizes: torch.Tensor, sort_idx: torch.Tensor, inv_sort_idx: torch.Tensor,
                  num_selected: int) -> torch.Tensor:
    """``moe_fused_linear(moe_fused_glu(tokens, w_gate, w_up, ...), w_down, m_sizes)``: the three expert
    projections of the block (modular_qwen3_moe_fused.py:95-110 of the reference) as one differentiable op.
    ``w_down`` (E, hidden, intermediate).  Result (T * num_selected, hidden), rows grouped by expert."""
    return _MlpGathered.apply(tokens, w_gate, w_up, w_down, m_sizes, sort_idx, inv_sort_idx, num_selected)


class _GluGathered4bit(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tokens, gate_packed, gate_state, up_packed, up_state, m_sizes, sort_idx, inv_sort_idx, k):
        need = ctx.needs_input_grad[0]
        out = grouped_glu_forward_4bit(tokens, gate_packed, gate_state, up_packed, up_state, m_sizes, sort_idx, k,
                                       return_products=need)
        if not need:
            return out
        h, e, g = out
        ctx.save_for_backward(gate_packed, up_packed, m_sizes, inv_sort_idx, e, g)
        ctx.states = (gate_state, up_state)
        ctx.k, ctx.n_tokens = k, tokens.shape[0]
        return h

    @staticmethod
    def backward(ctx, dh):
        gate_packed, up_packed, m_sizes, inv_sort_idx, e, g = ctx.saved_tensors
        de, dg = silu_mul_backward(dh.contiguous(), e, g)
        # frozen weights: only the tokens get a gradient
        dx = grouped_gemm_forward_transposed_4bit(de, gate_packed, ctx.states[0], m_sizes, de.dtype)
        grouped_gemm_forward_transposed_4bit(dg, up_packed, ctx.states[1], m_sizes, out=dx, accumulate=True)
        d_tokens = _combine(dx, inv_sort_idx, None, ctx.n_tokens, ctx.k)
        return d_tokens, None, None, None, None, None, None, None, None


def moe_fused_glu_4bit(tokens: torch.Tensor, gate_weight: torch.Tensor, up_weight: torch.Tensor,
                       m_sizes: torch.Tensor, sort_idx: torch.Tensor, inv_sort_idx: torch.Tensor,
                       num_selected: int) -> torch.Tensor:
    """``moe_fused_glu`` on packed NF4 weights carrying a ``quant_state`` (frozen)."""
    assert not gate_weight.requires_grad and not up_weight.requires_grad
    return _GluGathered4bit.apply(tokens, gate_weight.data, gate_weight.quant_state, up_weight.data,
                                  up_weight.quant_state, m_sizes, sort_idx, inv_sort_idx, num_selected)
