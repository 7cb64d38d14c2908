"""Argument checks and the single launch helper shared by the three grouped-GEMM wrappers.

The reference wrappers validate with bare ``assert`` (AssertionError on misuse) --
qwen3_moe_fused/grouped_gemm/forward.py:119-132 -- and so do these.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib

_INT_DTYPES = (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64)


def is_int_tensor(x: torch.Tensor) -> bool:
    return x.dtype in _INT_DTYPES


def check_operands(m_sizes: torch.Tensor, *tensors: torch.Tensor) -> None:
    first = tensors[0]
    assert first.is_cuda, "grouped GEMM runs on the GPU only"
    for t in tensors[1:] + (m_sizes,):
        assert t.device == first.device
    assert is_int_tensor(m_sizes)
    for t in tensors + (m_sizes,):
        assert t.is_contiguous()
    assert m_sizes.ndim == 1
    for t in tensors[1:]:
        assert t.dtype == first.dtype, "both GEMM operands must share one element type"


def launch(entry: str, a: torch.Tensor, b: torch.Tensor, m_sizes: torch.Tensor, out: torch.Tensor,
           R: int, N: int, K: int, E: int, alpha: float = 1.0, accumulate: bool = False) -> torch.Tensor:
    ms = _lib.as_index_tensor(m_sizes)
    fn = getattr(_lib.lib(), entry)
    rc = fn(_lib.ptr(a), _lib.ptr(b), _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(out), R, N, K, E,
            _lib.dtype_code(a.dtype), _lib.dtype_code(out.dtype), float(alpha), int(bool(accumulate)), _lib.stream())
    _lib.check(rc, entry)
    return out


def out_dtype(requested: Optional[torch.dtype], like: torch.Tensor) -> torch.dtype:
    return like.dtype if requested is None else requested
