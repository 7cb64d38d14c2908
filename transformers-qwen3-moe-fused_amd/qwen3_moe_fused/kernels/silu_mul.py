"""h = silu(e) * g and its backward (reference: qwen3_moe_fused/kernels/silu_mul.py).

Rounding chain kept from the reference kernels: the SiLU is evaluated in fp32, rounded to the
tensor dtype, then multiplied (silu_mul.py:34-39); the backward follows :62-73 and the in-place
variant overwrites (dh, e, g) with (h, de, dg) (:95-111).
"""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib


def _check(*ts: torch.Tensor) -> None:
    first = ts[0]
    assert first.is_cuda
    for t in ts:
        assert t.device == first.device
        assert t.is_contiguous()
        assert t.numel() == first.numel()
        assert t.dtype == first.dtype


def silu_mul_forward(e: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    _check(e, g)
    h = torch.empty_like(e)
    rc = _lib.lib().mfl_silu_mul_fwd(_lib.ptr(e), _lib.ptr(g), _lib.ptr(h), e.numel(), _lib.dtype_code(e.dtype),
                                     _lib.stream())
    _lib.check(rc, "mfl_silu_mul_fwd")
    return h


def silu_mul_backward(dh: torch.Tensor, e: torch.Tensor, g: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _check(e, g, dh)
    de, dg = torch.empty_like(e), torch.empty_like(g)
    rc = _lib.lib().mfl_silu_mul_bwd(_lib.ptr(dh), _lib.ptr(e), _lib.ptr(g), _lib.ptr(de), _lib.ptr(dg), None,
                                     e.numel(), _lib.dtype_code(e.dtype), _lib.stream())
    _lib.check(rc, "mfl_silu_mul_bwd")
    return de, dg


def silu_mul_backward_inplace(dh: torch.Tensor, e: torch.Tensor, g: torch.Tensor) -> None:
    """Overwrites ``dh, e, g`` with ``h, de, dg``."""
    _check(e, g, dh)
    rc = _lib.lib().mfl_silu_mul_bwd(_lib.ptr(dh), _lib.ptr(e), _lib.ptr(g), _lib.ptr(e), _lib.ptr(g), _lib.ptr(dh),
                                     e.numel(), _lib.dtype_code(e.dtype), _lib.stream())
    _lib.check(rc, "mfl_silu_mul_bwd")


class SiluMul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, e, g):
        ctx.save_for_backward(e, g)
        return silu_mul_forward(e, g)

    @staticmethod
    def backward(ctx, dh):
        e, g = ctx.saved_tensors
        return silu_mul_backward(dh.contiguous(), e, g)


silu_mul = SiluMul.apply
