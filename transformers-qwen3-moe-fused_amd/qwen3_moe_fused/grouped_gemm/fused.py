"""Forward products fused with their neighbours in the sparse MLP block.

The reference keeps these steps apart and names both fusions as possible
(qwen3_moe_fused/modular_qwen3_moe_fused.py:100-101 "fuse a sort and a MoeFusedLinear layer",
:105 "fuse gate_h and up_h"):

* gathered rows: ``y = grouped_gemm_forward(x_src[row_idx // idx_div], w, m_sizes)`` without
  writing the gathered matrix (with ``row_idx = sort_idx``, ``idx_div = num_selected`` this is the
  replicate-and-sort of :95-103 folded into the GEMM's operand load);
* gated linear unit: ``silu(x @ w_gate^T) * (x @ w_up^T)`` in one kernel (:106-108), with the
  rounding steps of the separate kernels, so the result is bit-identical to them.

Each wrapper calls the fused entry point and, when the library answers that it has no fused
kernel for the request (status ``UNSUPPORTED``: odd sizes, fp32, ...), runs the separate HIP
kernels instead.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from ..kernels.routing import _gather as gather_kernel
from ..kernels.silu_mul import silu_mul_forward
from ..quantize.nf4 import resolve_absmax, tiled_absmax
from ._common import check_operands, is_int_tensor
from .forward import grouped_gemm_forward
from .forward_4bit import grouped_gemm_forward_4bit

UNSUPPORTED = -6  # MFL_ERR_UNSUPPORTED


def _gather(x_src: torch.Tensor, row_idx: torch.Tensor, idx_div: int) -> torch.Tensor:
    return gather_kernel(x_src, row_idx, idx_div, None)


def _check_gather(x_src: torch.Tensor, row_idx: Optional[torch.Tensor], idx_div: int) -> int:
    """Number of rows of the (virtual) left operand."""
    assert x_src.ndim == 2
    if row_idx is None:
        return x_src.shape[0]
    assert row_idx.dtype == torch.int32 and row_idx.ndim == 1 and row_idx.is_contiguous()
    assert row_idx.device == x_src.device and idx_div >= 1
    return row_idx.numel()


def _nf4_args(w_quant: torch.Tensor, state, x: torch.Tensor, k: int):
    assert state.quant_type in ("nf4", "fp4")
    blocksize = int(state.blocksize)
    assert blocksize > 0 and blocksize & (blocksize - 1) == 0, "blocksize must be a power of two"
    code = state.code
    assert code.dtype == torch.float32
    absmax = resolve_absmax(state)
    for t in (w_quant, code, absmax):
        assert t.device == x.device and t.is_contiguous()
    assert is_int_tensor(w_quant) and len(state.shape) == 3
    experts, n, k_w = state.shape
    assert k_w == k and k % 2 == 0
    total = experts * n * k
    assert total % blocksize == 0 and w_quant.numel() == total // 2 and absmax.numel() == total // blocksize
    return code, absmax, blocksize, experts, n


def grouped_gemm_forward_gathered(x_src: torch.Tensor, row_idx: torch.Tensor, idx_div: int, w: torch.Tensor,
                                  m_sizes: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward(x_src[row_idx // idx_div], w, m_sizes, dtype)``."""
    check_operands(m_sizes, x_src, w)
    rows = _check_gather(x_src, row_idx, idx_div)
    assert w.ndim == 3
    experts, n, k = w.shape
    assert x_src.shape[1] == k and m_sizes.numel() == experts
    y = torch.empty((rows, n), device=x_src.device, dtype=x_src.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_fwd_gather(_lib.ptr(x_src), x_src.shape[0], _lib.ptr(row_idx), idx_div, _lib.ptr(w),
                                        _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(y), rows, n, k, experts,
                                        _lib.dtype_code(x_src.dtype), _lib.dtype_code(y.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        return grouped_gemm_forward(_gather(x_src, row_idx, idx_div), w, m_sizes, dtype)
    _lib.check(rc, "mfl_gemm_fwd_gather")
    return y


def grouped_gemm_forward_4bit_gathered(x_src: torch.Tensor, row_idx: torch.Tensor, idx_div: int,
                                       w_quant: torch.Tensor, w_quant_state, m_sizes: torch.Tensor,
                                       dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward_4bit(x_src[row_idx // idx_div], w_quant, w_quant_state, m_sizes, dtype)``."""
    assert x_src.is_cuda and x_src.is_contiguous() and m_sizes.is_contiguous() and is_int_tensor(m_sizes)
    rows = _check_gather(x_src, row_idx, idx_div)
    k = x_src.shape[1]
    code, absmax, blocksize, experts, n = _nf4_args(w_quant, w_quant_state, x_src, k)
    assert m_sizes.numel() == experts
    y = torch.empty((rows, n), device=x_src.device, dtype=x_src.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    tiled = tiled_absmax(w_quant_state, absmax, rows)
    if tiled is not None:
        rc = _lib.lib().mfl_gemm_fwd_nf4_tiled(_lib.ptr(x_src), x_src.shape[0], _lib.ptr(row_idx), idx_div,
                                               _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), _lib.ptr(tiled),
                                               blocksize, _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(y), rows,
                                               n, k, experts, _lib.dtype_code(x_src.dtype),
                                               _lib.dtype_code(y.dtype), _lib.stream())
    else:
        rc = _lib.lib().mfl_gemm_fwd_nf4_gather(_lib.ptr(x_src), x_src.shape[0], _lib.ptr(row_idx), idx_div,
                                                _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), blocksize,
                                                _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(y), rows, n, k,
                                                experts, _lib.dtype_code(x_src.dtype), _lib.dtype_code(y.dtype),
                                                _lib.stream())
    if rc == UNSUPPORTED:
        return grouped_gemm_forward_4bit(_gather(x_src, row_idx, idx_div), w_quant, w_quant_state, m_sizes, dtype)
    _lib.check(rc, "mfl_gemm_fwd_nf4_gather")
    return y


def grouped_glu_forward(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, m_sizes: torch.Tensor,
                        row_idx: Optional[torch.Tensor] = None, idx_div: int = 1,
                        return_products: bool = False):
    """``h = silu(e) * g`` with ``e = grouped_gemm_forward(xg, w_gate, m_sizes)``,
    ``g = grouped_gemm_forward(xg, w_up, m_sizes)`` and ``xg = x`` or, with ``row_idx``,
    ``x[row_idx // idx_div]``.  Returns ``h`` or ``(h, e, g)``."""
    check_operands(m_sizes, x, w_gate, w_up)
    rows = _check_gather(x, row_idx, idx_div)
    assert w_gate.ndim == 3 and w_up.shape == w_gate.shape
    experts, n, k = w_gate.shape
    assert x.shape[1] == k and m_sizes.numel() == experts
    h = torch.empty((rows, n), device=x.device, dtype=x.dtype)
    e = torch.empty_like(h) if return_products else None
    g = torch.empty_like(h) if return_products else None
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_glu_fwd(_lib.ptr(x), x.shape[0], _lib.ptr(row_idx), idx_div, _lib.ptr(w_gate), _lib.ptr(w_up),
                                _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(h), _lib.ptr(e), _lib.ptr(g), rows, n,
                                k, experts, _lib.dtype_code(x.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        xg = x if row_idx is None else _gather(x, row_idx, idx_div)
        e = grouped_gemm_forward(xg, w_gate, m_sizes)
        g = grouped_gemm_forward(xg, w_up, m_sizes)
        h = silu_mul_forward(e, g)
    else:
        _lib.check(rc, "mfl_glu_fwd")
    return (h, e, g) if return_products else h


def grouped_glu_forward_4bit(x: torch.Tensor, gate_quant: torch.Tensor, gate_state, up_quant: torch.Tensor, up_state,
                             m_sizes: torch.Tensor, row_idx: Optional[torch.Tensor] = None, idx_div: int = 1,
                             return_products: bool = False):
    """``grouped_glu_forward`` with NF4 gate and up weights, each with its own quant state."""
    assert x.is_cuda and x.is_contiguous() and m_sizes.is_contiguous() and is_int_tensor(m_sizes)
    rows = _check_gather(x, row_idx, idx_div)
    k = x.shape[1]
    code_g, absmax_g, bs_g, experts, n = _nf4_args(gate_quant, gate_state, x, k)
    code_u, absmax_u, bs_u, experts_u, n_u = _nf4_args(up_quant, up_state, x, k)
    assert (experts_u, n_u) == (experts, n) and m_sizes.numel() == experts
    h = torch.empty((rows, n), device=x.device, dtype=x.dtype)
    e = torch.empty_like(h) if return_products else None
    g = torch.empty_like(h) if return_products else None
    ms = _lib.as_index_tensor(m_sizes)
    tiled_g, tiled_u = tiled_absmax(gate_state, absmax_g, rows), tiled_absmax(up_state, absmax_u, rows)
    rc = _lib.lib().mfl_glu_fwd_nf4_tiled(_lib.ptr(x), x.shape[0], _lib.ptr(row_idx), idx_div,
                                          _lib.ptr(gate_quant), _lib.ptr(code_g), _lib.ptr(absmax_g), _lib.ptr(tiled_g),
                                          bs_g, _lib.ptr(up_quant), _lib.ptr(code_u), _lib.ptr(absmax_u),
                                          _lib.ptr(tiled_u), bs_u, _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(h),
                                          _lib.ptr(e), _lib.ptr(g), rows, n, k, experts, _lib.dtype_code(x.dtype),
                                          _lib.stream())
    if rc == UNSUPPORTED:
        xg = x if row_idx is None else _gather(x, row_idx, idx_div)
        e = grouped_gemm_forward_4bit(xg, gate_quant, gate_state, m_sizes)
        g = grouped_gemm_forward_4bit(xg, up_quant, up_state, m_sizes)
        h = silu_mul_forward(e, g)
    else:
        _lib.check(rc, "mfl_glu_fwd_nf4_tiled")
    return (h, e, g) if return_products else h


def grouped_gemm_forward_transposed_dual(dy1: torch.Tensor, w1: torch.Tensor, dy2: torch.Tensor, w2: torch.Tensor,
                                         m_sizes: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward_transposed(dy1, w1, m_sizes) + grouped_gemm_forward_transposed(dy2, w2,
    m_sizes)`` in one kernel (one reduction over both terms, one rounding): the input gradient of
    the gated unit, ``de @ w_gate + dg @ w_up``."""
    from .forward_transposed import grouped_gemm_forward_transposed

    check_operands(m_sizes, dy1, w1, dy2, w2)
    assert dy1.ndim == 2 and w1.ndim == 3 and dy2.shape == dy1.shape and w2.shape == w1.shape
    rows, k = dy1.shape
    experts, k_w, n = w1.shape
    assert k_w == k and m_sizes.numel() == experts
    dx = torch.empty((rows, n), device=dy1.device, dtype=dy1.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_dx_dual(_lib.ptr(dy1), _lib.ptr(w1), _lib.ptr(dy2), _lib.ptr(w2), _lib.ptr(ms),
                                     _lib.itype_code(ms.dtype), _lib.ptr(dx), rows, n, k, experts,
                                     _lib.dtype_code(dy1.dtype), _lib.dtype_code(dx.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        grouped_gemm_forward_transposed(dy1, w1, m_sizes, dtype, out=dx)
        return grouped_gemm_forward_transposed(dy2, w2, m_sizes, dtype, out=dx, accumulate=True)
    _lib.check(rc, "mfl_gemm_dx_dual")
    return dx


def grouped_gemm_forward_transposed_silu_bwd(dy: torch.Tensor, w: torch.Tensor, e: torch.Tensor, g: torch.Tensor,
                                             m_sizes: torch.Tensor, return_h: bool = False):
    """``silu_mul_backward(grouped_gemm_forward_transposed(dy, w, m_sizes), e, g)`` in one kernel: the input
    gradient of the down projection never reaches memory, its pieces meet those of ``e`` and ``g`` in the
    product's epilogue.  Returns ``(de, dg)`` or ``(de, dg, h)``; the same bits as the two kernels."""
    from ..kernels.silu_mul import silu_mul_forward
    from .forward_transposed import grouped_gemm_forward_transposed

    check_operands(m_sizes, dy, w, e, g)
    assert dy.ndim == 2 and w.ndim == 3 and e.shape == g.shape
    rows, k = dy.shape
    experts, k_w, n = w.shape
    assert k_w == k and m_sizes.numel() == experts and e.shape == (rows, n)
    de, dg = torch.empty_like(e), torch.empty_like(g)
    h = torch.empty_like(e) if return_h else None
    ms = _lib.as_index_tensor(m_sizes)
    rc = UNSUPPORTED
    if dy.dtype == torch.bfloat16 and w.dtype == dy.dtype and e.dtype == dy.dtype and g.dtype == dy.dtype:
        rc = _lib.lib().mfl_gemm_dx_silu_bwd(_lib.ptr(dy), _lib.ptr(w), _lib.ptr(e), _lib.ptr(g), _lib.ptr(ms),
                                             _lib.itype_code(ms.dtype), _lib.ptr(de), _lib.ptr(dg), _lib.ptr(h), rows, n,
                                             k, experts, _lib.dtype_code(dy.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        from ..kernels.silu_mul import silu_mul_backward

        dh = grouped_gemm_forward_transposed(dy, w, m_sizes, e.dtype)
        de, dg = silu_mul_backward(dh, e, g)
        if return_h:
            h = silu_mul_forward(e, g)
    else:
        _lib.check(rc, "mfl_gemm_dx_silu_bwd")
    return (de, dg, h) if return_h else (de, dg)


def grouped_gemm_forward_lora(x: torch.Tensor, w: torch.Tensor, xt: torch.Tensor, wt: torch.Tensor,
                              m_sizes: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward(x, w, m_sizes) + grouped_gemm_forward(xt, wt, m_sizes)`` in one kernel: a product
    with the rank-r term of a LoRA adapter in the same reduction (``xt = s * x A^T`` (rows, r), ``wt = B``
    (E, N, r)); the reference adds the two (qwen3_moe_fused/lora.py:134, kernels/fast_lora.py:65-88)."""
    check_operands(m_sizes, x, w, xt, wt)
    assert x.ndim == 2 and w.ndim == 3 and xt.ndim == 2 and wt.ndim == 3
    rows, k = x.shape
    experts, n, k_w = w.shape
    r = xt.shape[1]
    assert k_w == k and m_sizes.numel() == experts and xt.shape[0] == rows and wt.shape == (experts, n, r)
    y = torch.empty((rows, n), device=x.device, dtype=x.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_fwd_lora(_lib.ptr(x), _lib.ptr(w), _lib.ptr(xt), _lib.ptr(wt), r, _lib.ptr(ms),
                                      _lib.itype_code(ms.dtype), _lib.ptr(y), rows, n, k, experts,
                                      _lib.dtype_code(x.dtype), _lib.dtype_code(y.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        grouped_gemm_forward(x, w, m_sizes, dtype, out=y)
        return grouped_gemm_forward(xt, wt, m_sizes, dtype, out=y, accumulate=True)
    _lib.check(rc, "mfl_gemm_fwd_lora")
    return y


def grouped_gemm_forward_transposed_lora(dy: torch.Tensor, w: torch.Tensor, xt: torch.Tensor, wt: torch.Tensor,
                                         m_sizes: torch.Tensor, dtype: Optional[torch.dtype] = None, *,
                                         dy2: Optional[torch.Tensor] = None,
                                         w2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``dy @ w (+ dy2 @ w2) + xt @ wt`` per expert in one kernel: an input gradient with the rank-r term of a
    LoRA adapter in the same reduction (``xt = s * dy B`` (rows, r), ``wt = A`` (E, r, N)), optionally over
    both weights of the gated unit (qwen3_moe_fused/kernels/fast_lora.py:127-131,151-152)."""
    from .forward_transposed import grouped_gemm_forward_transposed

    check_operands(m_sizes, dy, w, xt, wt)
    assert dy.ndim == 2 and w.ndim == 3 and xt.ndim == 2 and wt.ndim == 3
    rows, k = dy.shape
    experts, k_w, n = w.shape
    r = xt.shape[1]
    assert k_w == k and m_sizes.numel() == experts and xt.shape[0] == rows and wt.shape == (experts, r, n)
    assert (dy2 is None) == (w2 is None)
    if dy2 is not None:
        check_operands(m_sizes, dy, dy2, w2)
        assert dy2.shape == dy.shape and w2.shape == w.shape
    dx = torch.empty((rows, n), device=dy.device, dtype=dy.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_dx_lora(_lib.ptr(dy), _lib.ptr(w), _lib.ptr(dy2) if dy2 is not None else None,
                                     _lib.ptr(w2) if w2 is not None else None, _lib.ptr(xt), _lib.ptr(wt), r,
                                     _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(dx), rows, n, k, experts,
                                     _lib.dtype_code(dy.dtype), _lib.dtype_code(dx.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        if dy2 is None:
            grouped_gemm_forward_transposed(dy, w, m_sizes, dtype, out=dx)
        else:
            dx = grouped_gemm_forward_transposed_dual(dy, w, dy2, w2, m_sizes, dtype)
        return grouped_gemm_forward_transposed(xt, wt, m_sizes, dtype, out=dx, accumulate=True)
    _lib.check(rc, "mfl_gemm_dx_lora")
    return dx


def grouped_gemm_forward_4bit_lora(x: torch.Tensor, w_quant: torch.Tensor, w_quant_state, xt: torch.Tensor,
                                   wt: torch.Tensor, m_sizes: torch.Tensor,
                                   dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward_lora`` over NF4 base weights: ``x W^T + xt wt^T`` with ``W`` decoded inside the
    kernel (the QLoRA forward product; the reference dequantises, multiplies and adds:
    qwen3_moe_fused/kernels/fast_lora.py:57-63,65-88)."""
    assert x.is_cuda and x.ndim == 2 and x.is_contiguous() and m_sizes.is_contiguous() and is_int_tensor(m_sizes)
    rows, k = x.shape
    code, absmax, blocksize, experts, n = _nf4_args(w_quant, w_quant_state, x, k)
    r = xt.shape[1]
    assert m_sizes.numel() == experts and xt.shape == (rows, r) and wt.shape == (experts, n, r)
    assert xt.is_contiguous() and wt.is_contiguous() and xt.dtype == x.dtype and wt.dtype == x.dtype
    y = torch.empty((rows, n), device=x.device, dtype=x.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_fwd_nf4_lora(_lib.ptr(x), _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), blocksize,
                                          _lib.ptr(xt), _lib.ptr(wt), r, _lib.ptr(ms), _lib.itype_code(ms.dtype),
                                          _lib.ptr(y), rows, n, k, experts, _lib.dtype_code(x.dtype),
                                          _lib.dtype_code(y.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        y = grouped_gemm_forward_4bit(x, w_quant, w_quant_state, m_sizes, dtype)
        return grouped_gemm_forward(xt, wt, m_sizes, dtype, out=y, accumulate=True)
    _lib.check(rc, "mfl_gemm_fwd_nf4_lora")
    return y


def grouped_gemm_forward_transposed_4bit_lora(dy: torch.Tensor, w_quant: torch.Tensor, w_quant_state, xt: torch.Tensor,
                                              wt: torch.Tensor, m_sizes: torch.Tensor,
                                              dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``grouped_gemm_forward_transposed_lora`` over NF4 base weights of shape (E, out, in) =
    ``w_quant_state.shape``: dx (rows, in) = dy (rows, out) @ W[e] + xt (rows, r) @ wt[e], wt (E, r, in)
    (qwen3_moe_fused/kernels/fast_lora.py:57-63,127-131)."""
    from .forward_4bit import grouped_gemm_forward_transposed_4bit
    from .forward_transposed import grouped_gemm_forward_transposed

    assert dy.is_cuda and dy.ndim == 2 and dy.is_contiguous() and m_sizes.is_contiguous() and is_int_tensor(m_sizes)
    assert w_quant_state.quant_type in ("nf4", "fp4") and is_int_tensor(w_quant) and w_quant.is_contiguous()
    blocksize = int(w_quant_state.blocksize)
    code, absmax = w_quant_state.code, resolve_absmax(w_quant_state)
    experts, k, n = w_quant_state.shape
    rows, r = dy.shape[0], xt.shape[1]
    assert dy.shape[1] == k and m_sizes.numel() == experts and xt.shape == (rows, r) and wt.shape == (experts, r, n)
    assert xt.is_contiguous() and wt.is_contiguous() and xt.dtype == dy.dtype and wt.dtype == dy.dtype
    dx = torch.empty((rows, n), device=dy.device, dtype=dy.dtype if dtype is None else dtype)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_gemm_dx_nf4_lora(_lib.ptr(dy), _lib.ptr(w_quant), _lib.ptr(code), _lib.ptr(absmax), blocksize,
                                         _lib.ptr(xt), _lib.ptr(wt), r, _lib.ptr(ms), _lib.itype_code(ms.dtype),
                                         _lib.ptr(dx), rows, n, k, experts, _lib.dtype_code(dy.dtype),
                                         _lib.dtype_code(dx.dtype), _lib.stream())
    if rc == UNSUPPORTED:
        grouped_gemm_forward_transposed_4bit(dy, w_quant, w_quant_state, m_sizes, dtype, out=dx)
        return grouped_gemm_forward_transposed(xt, wt, m_sizes, dtype, out=dx, accumulate=True)
    _lib.check(rc, "mfl_gemm_dx_nf4_lora")
    return dx


def grouped_glu_forward_lora(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, xt: torch.Tensor,
                             wt_gate: torch.Tensor, wt_up: torch.Tensor, m_sizes: torch.Tensor):
    """``(h, e, g)`` with ``e = x w_gate^T + xt wt_gate^T``, ``g = x w_up^T + xt wt_up^T``, ``h = silu(e) * g`` in
    one kernel: the gate and up projections of the LoRA MLP with their rank-r terms and the SiLU-mul
    (qwen3_moe_fused/kernels/fast_lora.py:68-95).  ``xt`` (rows, r_g + r_u) holds both adapters' scaled
    activations side by side; ``wt_gate`` / ``wt_up`` (E, N, r_g + r_u) hold each adapter's B over its own columns
    and zeros over the other's."""
    check_operands(m_sizes, x, w_gate, w_up, xt, wt_gate, wt_up)
    assert x.ndim == 2 and w_gate.ndim == 3 and w_up.shape == w_gate.shape
    rows, k = x.shape
    experts, n, k_w = w_gate.shape
    kt = xt.shape[1]
    assert k_w == k and m_sizes.numel() == experts and xt.shape[0] == rows
    assert wt_gate.shape == (experts, n, kt) and wt_up.shape == (experts, n, kt)
    h = torch.empty((rows, n), device=x.device, dtype=x.dtype)
    e, g = torch.empty_like(h), torch.empty_like(h)
    ms = _lib.as_index_tensor(m_sizes)
    rc = _lib.lib().mfl_glu_fwd_lora(_lib.ptr(x), _lib.ptr(w_gate), _lib.ptr(w_up), _lib.ptr(xt), _lib.ptr(wt_gate),
                                     _lib.ptr(wt_up), kt, _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(h),
                                     _lib.ptr(e), _lib.ptr(g), rows, n, k, experts, _lib.dtype_code(x.dtype),
                                     _lib.stream())
    if rc == UNSUPPORTED:
        e = grouped_gemm_forward_lora(x, w_gate, xt, wt_gate, m_sizes)
        g = grouped_gemm_forward_lora(x, w_up, xt, wt_up, m_sizes)
        return silu_mul_forward(e, g), e, g
    _lib.check(rc, "mfl_glu_fwd_lora")
    return h, e, g
