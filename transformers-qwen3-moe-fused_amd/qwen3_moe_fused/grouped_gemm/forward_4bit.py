"""Forward grouped GEMM with NF4 weights decoded inside the K loop.

Host wrapper over ``mfl_gemm_fwd_nf4``; contract of the reference's ``grouped_gemm_forward_4bit``
(qwen3_moe_fused/grouped_gemm/forward_4bit.py:135-208): ``w_quant`` is the packed uint8 tensor,
``w_quant_state`` an NF4 quant state whose ``shape`` is (E, N, K); a double-quantised absmax is
un-nested first (:149-152); the state's own dtype is ignored and weights are rounded to
``x.dtype`` (:103-104).  Inputs the fused kernels do not take (status UNSUPPORTED: rows that are
not bf16, K not a multiple of 8, quantisation blocks under 8) are served by the dequantise kernel
followed by the plain product, so the wrapper accepts what the reference's accepts.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ..quantize.nf4 import resolve_absmax, tiled_absmax
from ._common import is_int_tensor


def grouped_gemm_forward_4bit(x: torch.Tensor, w_quant: torch.Tensor, w_quant_state, m_sizes: torch.Tensor,
                              dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    assert w_quant_state.quant_type in ("nf4", "fp4")
    blocksize = int(w_quant_state.blocksize)
    assert blocksize > 0 and blocksize & (blocksize - 1) == 0, "blocksize must be a power of two"
    code = w_quant_state.code
    assert code.dtype == torch.float32
    absmax = resolve_absmax(w_quant_state)

    assert x.is_cuda
    for t in (w_quant, code, absmax, m_sizes):
        assert t.device == x.device
    assert is_int_tensor(w_quant) and is_int_tensor(m_sizes)
    for t in (x, w_quant, code, absmax, m_sizes):
        assert t.is_contiguous()
    assert x.ndim == 2 and m_sizes.ndim == 1 and len(w_quant_state.shape) == 3
    rows, k = x.shape
    experts, n, k_w = w_quant_state.shape
    assert k_w == k and k % 2 == 0
    total = experts * n * k
    assert total % blocksize == 0
    assert w_quant.numel() == total // 2
    assert absmax.numel() == total // blocksize
    assert m_sizes.numel() == experts

    y = torch.empty((rows, n), device=x.device, dtype=x.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    tiled = tiled_absmax(w_quant_state, absmax, rows)  # decode-sized batches: scales in the order of consumption
    if tiled is not None:
        rc = _lib.lib().mfl_gemm_fwd_nf4_tiled(_lib.ptr(x), rows, None, 1, _lib.ptr(w_quant), _lib.ptr(code),
                                               _lib.ptr(absmax), _lib.ptr(tiled), blocksize, _lib.ptr(ms),
                                               _lib.itype_code(ms.dtype), _lib.ptr(y), rows, n, k, experts,
                                               _lib.dtype_code(x.dtype), _lib.dtype_code(y.dtype), _lib.stream())
    else:
        rc = _lib.lib().mfl_gemm_fwd_nf4(_lib.ptr(x), _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), blocksize,
                                         _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(y), rows, n, k, experts,
                                         _lib.dtype_code(x.dtype), _lib.dtype_code(y.dtype), _lib.stream())
    if rc == -6:  # MFL_ERR_UNSUPPORTED (fp32 / fp16 rows, K % 8 != 0, blocksize < 8): dequantise, then the plain product
        from ..quantize.nf4 import dequantize_nf4
        from .forward import grouped_gemm_forward

        return grouped_gemm_forward(x, dequantize_nf4(w_quant, w_quant_state, x.dtype), m_sizes, y.dtype)
    _lib.check(rc, "mfl_gemm_fwd_nf4")
    return y


def grouped_gemm_forward_transposed_4bit(dy: torch.Tensor, w_quant: torch.Tensor, w_quant_state,
                                         m_sizes: torch.Tensor, dtype: Optional[torch.dtype] = None, *,
                                         out: Optional[torch.Tensor] = None, alpha: float = 1.0,
                                         accumulate: bool = False) -> torch.Tensor:
    """``grouped_gemm_forward_transposed(dy, W, m_sizes)`` with ``W`` = the NF4 weight of shape
    (E, out, in) = ``w_quant_state.shape``: dx (rows, in) = dy (rows, out) @ W[e].  The weight is
    decoded inside the kernel; for shapes the fused kernel does not take (status UNSUPPORTED) it
    is dequantised first, as the reference always does (kernels/fast_lora.py:57-62,127-131)."""
    from ..quantize.nf4 import dequantize_nf4
    from .forward_transposed import grouped_gemm_forward_transposed

    assert w_quant_state.quant_type in ("nf4", "fp4")
    blocksize = int(w_quant_state.blocksize)
    code = w_quant_state.code
    absmax = resolve_absmax(w_quant_state)
    assert dy.is_cuda and dy.ndim == 2 and dy.is_contiguous() and m_sizes.is_contiguous()
    assert is_int_tensor(w_quant) and is_int_tensor(m_sizes) and w_quant.is_contiguous()
    experts, k, n = w_quant_state.shape
    rows = dy.shape[0]
    assert dy.shape[1] == k and m_sizes.numel() == experts
    if out is None:
        assert not accumulate, "accumulate needs an existing output"
        out = torch.empty((rows, n), device=dy.device, dtype=dy.dtype if dtype is None else dtype)
    else:
        assert out.shape == (rows, n) and out.is_contiguous() and out.device == dy.device
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_dx_nf4(_lib.ptr(dy), _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), blocksize,
                                    _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(out), rows, n, k, experts,
                                    _lib.dtype_code(dy.dtype), _lib.dtype_code(out.dtype), float(alpha),
                                    int(bool(accumulate)), _lib.stream())
    if rc == -6:  # MFL_ERR_UNSUPPORTED
        w = dequantize_nf4(w_quant, w_quant_state, dy.dtype)
        return grouped_gemm_forward_transposed(dy, w, m_sizes, dtype, out=out, alpha=alpha, accumulate=accumulate)
    _lib.check(rc, "mfl_gemm_dx_nf4")
    return out
