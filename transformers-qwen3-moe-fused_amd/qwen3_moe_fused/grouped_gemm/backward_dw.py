"""w[e, n, k] = sum_{m in e} y[m, n] * x[m, k] -- the dW product of moe_fused_linear.

Host wrapper over ``mfl_gemm_dw``; contract of the reference's ``grouped_gemm_backward_dw``
(qwen3_moe_fused/grouped_gemm/backward_dw.py:92-134).  The kernel writes every element of
the result, zeros included, so the output is allocated uninitialised where the reference
pre-zeroes it (:110).
"""
from __future__ import annotations

from typing import Optional

import torch

from ._common import check_operands, launch


def grouped_gemm_backward_dw(x: torch.Tensor, y: torch.Tensor, m_sizes: torch.Tensor, dtype: torch.dtype, *,
                             out: Optional[torch.Tensor] = None, alpha: float = 1.0,
                             accumulate: bool = False) -> torch.Tensor:
    check_operands(m_sizes, x, y)
    assert x.ndim == 2 and y.ndim == 2
    rows, k = x.shape
    rows_y, n = y.shape
    assert rows_y == rows
    experts = m_sizes.numel()
    if out is None:
        assert not accumulate, "accumulate needs an existing output"
        out = torch.empty((experts, n, k), device=x.device, dtype=dtype)
    else:
        assert out.shape == (experts, n, k) and out.is_contiguous() and out.device == x.device
    # the C entry point takes (x, dy); launch() passes its first two tensors in order
    return launch("mfl_gemm_dw", x, y, m_sizes, out, rows, n, k, experts, alpha, accumulate)
