"""y[m, n] = sum_k w[e(m), k, n] * x[m, k] -- the dX product of moe_fused_linear.

Host wrapper over ``mfl_gemm_dx``; contract of the reference's
``grouped_gemm_forward_transposed`` (qwen3_moe_fused/grouped_gemm/forward_transposed.py:107-151).
"""
from __future__ import annotations

from typing import Optional

import torch

from ._common import check_operands, launch, out_dtype


def grouped_gemm_forward_transposed(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor,
                                    dtype: Optional[torch.dtype] = None, *, out: Optional[torch.Tensor] = None,
                                    alpha: float = 1.0, accumulate: bool = False) -> torch.Tensor:
    check_operands(m_sizes, x, w)
    assert x.ndim == 2 and w.ndim == 3
    rows, k = x.shape
    experts, k_w, n = w.shape
    assert k_w == k
    assert m_sizes.numel() == experts
    if out is None:
        assert not accumulate, "accumulate needs an existing output"
        out = torch.empty((rows, n), device=x.device, dtype=out_dtype(dtype, x))
    else:
        assert out.shape == (rows, n) and out.is_contiguous() and out.device == x.device
    return launch("mfl_gemm_dx", x, w, m_sizes, out, rows, n, k, experts, alpha, accumulate)
