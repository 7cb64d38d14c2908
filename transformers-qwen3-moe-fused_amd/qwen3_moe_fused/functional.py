"""``moe_fused_linear`` and the naive reference trio it is checked against.

API of qwen3_moe_fused/functional.py: ``moe_fused_linear(input, weight, m_sizes)`` takes rows
already grouped by expert plus the per-expert row counts (functional.py:64-79); the three
``_moe_fused_linear_naive_*`` functions take per-row ``selected_experts`` in any order, run on
any device in plain torch and define the semantics (functional.py:7-61).
"""
from __future__ import annotations

import torch

from .grouped_gemm.interface import grouped_gemm


def _moe_fused_linear_naive_fwd(input: torch.Tensor, weight: torch.Tensor,
                                selected_experts: torch.Tensor) -> torch.Tensor:
    """output[b, o] = sum_i weight[selected_experts[b], o, i] * input[b, i], one mat-vec per row."""
    rows = [torch.mv(weight[int(e)], x_row) for e, x_row in zip(selected_experts.tolist(), input)]
    if not rows:
        return input.new_empty((0, weight.shape[1]))
    return torch.stack(rows, dim=0)


def _moe_fused_linear_naive_bwd_input(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                      selected_experts: torch.Tensor) -> torch.Tensor:
    """grad_input[b, i] = sum_o weight[selected_experts[b], o, i] * grad_output[b, o]."""
    grad_input = torch.empty_like(input)
    for b, e in enumerate(selected_experts.tolist()):
        grad_input[b] = torch.mv(weight[int(e)].t(), grad_output[b])
    return grad_input


def _moe_fused_linear_naive_bwd_weight(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                       selected_experts: torch.Tensor) -> torch.Tensor:
    """grad_weight[e, o, i] = sum over rows b routed to e of grad_output[b, o] * input[b, i]."""
    grad_weight = torch.zeros_like(weight)
    for b, e in enumerate(selected_experts.tolist()):
        grad_weight[int(e)].add_(torch.outer(grad_output[b], input[b]))
    return grad_weight


def moe_fused_linear(input: torch.Tensor, weight: torch.Tensor, m_sizes: torch.Tensor) -> torch.Tensor:
    """MoE linear layer as one grouped GEMM.

    ``input`` (rows, in_features) holds the rows of expert 0 first, then expert 1, ...;
    ``weight`` is (num_experts, out_features, in_features); ``m_sizes`` (num_experts,) integer
    row counts summing to ``rows``.  Differentiable in ``input`` and ``weight``.
    """
    return grouped_gemm(input, weight, m_sizes)


def moe_fused_linear_unsorted(input: torch.Tensor, weight: torch.Tensor,
                              selected_experts: torch.Tensor) -> torch.Tensor:
    """Same result as ``_moe_fused_linear_naive_fwd`` for rows in arbitrary expert order:
    sort by expert, grouped GEMM, un-sort.  Differentiable in ``input`` and ``weight``."""
    from .kernels.indexing import get_expert_counts_and_idx
    from .kernels.routing import gather_rows

    m_sizes, sort_idx, inv_sort_idx = get_expert_counts_and_idx(selected_experts, weight.shape[0])
    out_sorted = moe_fused_linear(gather_rows(input, sort_idx, 1, inv_sort_idx), weight, m_sizes)
    return gather_rows(out_sorted, inv_sort_idx, 1, sort_idx)
