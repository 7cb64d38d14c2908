"""Autograd glue of the grouped GEMM (reference: qwen3_moe_fused/grouped_gemm/interface.py:8-31).

Forward saves (x, w, m_sizes); backward runs the dX product only when x needs a gradient and
the dW product only when w does, and returns no gradient for m_sizes.
"""
from __future__ import annotations

import torch

from .backward_dw import grouped_gemm_backward_dw
from .forward import grouped_gemm_forward
from .forward_transposed import grouped_gemm_forward_transposed


class GroupedGemm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, m_sizes):
        ctx.save_for_backward(x, w, m_sizes)
        return grouped_gemm_forward(x, w, m_sizes)

    @staticmethod
    def backward(ctx, dy):
        x, w, m_sizes = ctx.saved_tensors
        dy = dy.contiguous()
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        dx = grouped_gemm_forward_transposed(dy, w, m_sizes, x.dtype) if need_dx else None
        dw = grouped_gemm_backward_dw(x, dy, m_sizes, w.dtype) if need_dw else None
        return dx, dw, None


grouped_gemm = GroupedGemm.apply
