"""y[m, n] = sum_k w[e(m), n, k] * x[m, k] -- rows of x grouped by expert.

Host wrapper over ``mfl_gemm_fwd``; same contract as the reference's
``grouped_gemm_forward`` (qwen3_moe_fused/grouped_gemm/forward.py:116-160): output is
freshly allocated, rows past ``sum(m_sizes)`` are left unwritten, ``m_sizes`` stays on
the device.
"""
from __future__ import annotations

from typing import Optional

import torch

from ._common import check_operands, is_int_tensor, launch, out_dtype  # noqa: F401  (is_int_tensor re-exported)


def grouped_gemm_forward(x: torch.Tensor, w: torch.Tensor, m_sizes: torch.Tensor,
                         dtype: Optional[torch.dtype] = None, *, out: Optional[torch.Tensor] = None,
                         alpha: float = 1.0, accumulate: bool = False) -> torch.Tensor:
    check_operands(m_sizes, x, w)
    assert x.ndim == 2 and w.ndim == 3
    rows, k = x.shape
    experts, n, k_w = w.shape
    assert k_w == k
    assert m_sizes.numel() == experts
    if out is None:
        assert not accumulate, "accumulate needs an existing output"
        out = torch.empty((rows, n), device=x.device, dtype=out_dtype(dtype, x))
    else:
        assert out.shape == (rows, n) and out.is_contiguous() and out.device == x.device
    return launch("mfl_gemm_fwd", x, w, m_sizes, out, rows, n, k, experts, alpha, accumulate)
