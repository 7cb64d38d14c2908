"""w[e, n, k] = sum_{m in e} y[m, n] * x[m, k] -- the dW product of moe_fused_linear.

Host wrapper over ``mfl_gemm_dw``; contract of the reference's ``grouped_gemm_backward_dw``
(qwen3_moe_fused/grouped_gemm/backward_dw.py:92-134).  The kernel writes every element of
the result, zeros included, so the output is allocated uninitialised where the reference
pre-zeroes it (:110).
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ._common import check_operands, launch

# below this many rows the general kernel is as fast and needs no workspace
_SPLIT_MIN_ROWS = 4096


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
    if not accumulate and rows >= _SPLIT_MIN_ROWS and x.dtype == torch.bfloat16:
        # one side as thin as a LoRA rank: the rows are dealt out evenly over the workgroups, so that the
        # expert with the most rows does not decide the time of the launch
        ws_bytes = int(_lib.lib().mfl_gemm_dw_split_workspace(rows, n, k, experts))
        if ws_bytes > 0 and out.dtype in (torch.bfloat16, torch.float32):
            ws = torch.empty(ws_bytes, device=x.device, dtype=torch.uint8)
            ms = _lib.as_index_tensor(m_sizes)
            rc = _lib.lib().mfl_gemm_dw_split(_lib.ptr(x), _lib.ptr(y), _lib.ptr(ms), _lib.itype_code(ms.dtype),
                                              _lib.ptr(out), rows, n, k, experts, _lib.dtype_code(x.dtype),
                                              _lib.dtype_code(out.dtype), float(alpha), _lib.ptr(ws), ws_bytes,
                                              _lib.stream())
            _lib.check(rc, "mfl_gemm_dw_split")
            return out
    # the C entry point takes (x, dy); launch() passes its first two tensors in order
    return launch("mfl_gemm_dw", x, y, m_sizes, out, rows, n, k, experts, alpha, accumulate)
