"""Router-side kernels of the sparse MoE block: fused softmax + top-k, the token gather that
feeds the experts and the weighted combine that follows them.

The reference does these with stock torch ops inline in the block forward
(qwen3_moe_fused/modular_qwen3_moe_fused.py:87-103,112-115, same in fast_lora.py:52-78); here
each is one library call with an autograd wrapper.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _lib


def softmax_topk_raw(logits: torch.Tensor, k: int, renorm: bool,
                     out_dtype: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (weights fp32 (T,k), weights cast to ``out_dtype`` (T,k), expert ids int64 (T,k)).
    Softmax in fp32 over the last dim, top-k sorted descending, equal probabilities resolved to the
    lower expert id, optional renormalisation over the k kept."""
    assert logits.is_cuda and logits.ndim == 2 and logits.is_contiguous()
    T, E = logits.shape
    out_dtype = logits.dtype if out_dtype is None else out_dtype
    w32 = torch.empty((T, k), device=logits.device, dtype=torch.float32)
    wc = torch.empty((T, k), device=logits.device, dtype=out_dtype)
    idx = torch.empty((T, k), device=logits.device, dtype=torch.int64)
    rc = _lib.lib().mfl_route_softmax_topk(_lib.ptr(logits), _lib.dtype_code(logits.dtype), T, E, k, int(bool(renorm)),
                                           _lib.ptr(w32), _lib.ptr(wc), _lib.dtype_code(out_dtype), _lib.ptr(idx),
                                           _lib.stream())
    _lib.check(rc, "mfl_route_softmax_topk")
    return w32, wc, idx


class _SoftmaxTopk(torch.autograd.Function):
    """Differentiable in the logits (the router trains through the routing weights)."""

    @staticmethod
    def forward(ctx, logits, k, renorm, out_dtype):
        w32, wc, idx = softmax_topk_raw(logits, k, renorm, out_dtype)
        ctx.save_for_backward(logits, idx, w32)
        ctx.renorm = renorm
        ctx.mark_non_differentiable(idx)
        return wc, idx

    @staticmethod
    def backward(ctx, dw, _didx):
        # Not on the hot path (a (T, E) problem; the frozen-router LoRA recipes never reach it).
        logits, idx, w32 = ctx.saved_tensors
        return _softmax_topk_backward(logits, idx, w32, ctx.renorm, dw), None, None, None


def _softmax_topk_backward(logits, idx, w32, renorm, dw):
    T, E = logits.shape
    k = idx.shape[1]
    if logits.is_cuda and E <= 1024 and k <= 64 and dw.dtype in (torch.float32, torch.bfloat16, torch.float16):
        # one kernel: a wave per token recomputes the softmax and applies both Jacobians
        dw = dw.contiguous()
        dlogits = torch.empty_like(logits)
        rc = _lib.lib().mfl_route_softmax_topk_bwd(_lib.ptr(logits), _lib.dtype_code(logits.dtype), T, E, k,
                                                   int(bool(renorm)), _lib.ptr(idx), _lib.ptr(w32), _lib.ptr(dw),
                                                   _lib.dtype_code(dw.dtype), _lib.ptr(dlogits), _lib.stream())
        _lib.check(rc, "mfl_route_softmax_topk_bwd")
        return dlogits
    dw = dw.float()
    p = torch.softmax(logits.float(), dim=-1)
    if renorm:
        # w = p_sel / s  ->  dp_sel = (dw - sum(dw * w)) / s, with s = sum(p_sel)
        s = p.gather(1, idx).sum(dim=-1, keepdim=True)
        dw = (dw - (dw * w32).sum(dim=-1, keepdim=True)) / s
    dp = torch.zeros_like(p).scatter_(1, idx, dw)
    dlogits = p * (dp - (dp * p).sum(dim=-1, keepdim=True))
    return dlogits.to(logits.dtype)


_ROUTE_WS_BYTES = {}  # (T, E, k) -> bytes of scratch mfl_route_sort asks for


def _round256(n: int) -> int:
    return (n + 255) // 256 * 256


def _route_and_sort_raw(logits: torch.Tensor, k: int, renorm: bool, out_dtype: Optional[torch.dtype]):
    """One library call (``mfl_route_sort``: one launch up to 64 tokens, two above) and ONE allocation, of which
    the outputs and the call's scratch are views.  Returns (w32, weights, idx, m_sizes, sort_idx, inv_sort_idx)."""
    assert logits.is_cuda and logits.ndim == 2 and logits.is_contiguous()
    T, E = logits.shape
    out_dtype = logits.dtype if out_dtype is None else out_dtype
    R = T * k
    key = (T, E, k)
    ws_bytes = _ROUTE_WS_BYTES.get(key)
    if ws_bytes is None:
        ws_bytes = _ROUTE_WS_BYTES[key] = int(_lib.lib().mfl_route_sort_workspace(T, E, k))
    # 256-byte aligned pieces of one block: idx int64, w32 fp32, sort_idx / inv / m_sizes int32, weights, scratch
    o_w32 = _round256(R * 8)
    o_sort = o_w32 + _round256(R * 4)
    o_inv = o_sort + _round256(R * 4)
    o_ms = o_inv + _round256(R * 4)
    o_wc = o_ms + _round256(E * 4)
    o_ws = o_wc + _round256(R * out_dtype.itemsize)
    buf = torch.empty(o_ws + ws_bytes, device=logits.device, dtype=torch.uint8)
    # one typed alias of the block per element type, then one strided view per output (every piece starts on a
    # multiple of 256 bytes, the block's size is a multiple of 256)
    i32 = buf.view(torch.int32)
    idx = torch.as_strided(buf.view(torch.int64), (T, k), (k, 1), 0)
    w32 = torch.as_strided(buf.view(torch.float32), (T, k), (k, 1), o_w32 // 4)
    sort_idx = torch.as_strided(i32, (R,), (1,), o_sort // 4)
    inv = torch.as_strided(i32, (R,), (1,), o_inv // 4)
    m_sizes = torch.as_strided(i32, (E,), (1,), o_ms // 4)
    wc = torch.as_strided(buf.view(out_dtype), (T, k), (k, 1), o_wc // out_dtype.itemsize)
    base = buf.data_ptr()
    rc = _lib.lib().mfl_route_sort(logits.data_ptr(), _lib.dtype_code(logits.dtype), T, E, k, int(bool(renorm)),
                                   base + o_w32, base + o_wc, _lib.dtype_code(out_dtype), base, base + o_ms,
                                   base + o_sort, base + o_inv, base + o_ws, ws_bytes, _lib.stream())
    _lib.check(rc, "mfl_route_sort")
    return w32, wc, idx, m_sizes, sort_idx, inv


class _RouteAndSort(torch.autograd.Function):
    """softmax + top-k and the stable expert sort of its selections, differentiable in the logits.  Returns
    (routing weights (T,k), expert ids (T,k) int64, m_sizes (E,), sort_idx, inv_sort_idx)."""

    @staticmethod
    def forward(ctx, logits, k, renorm, out_dtype, num_experts):
        assert logits.shape[1] == num_experts
        w32, wc, idx, m_sizes, sort_idx, inv = _route_and_sort_raw(logits, k, renorm, out_dtype)
        ctx.save_for_backward(logits, idx, w32)
        ctx.renorm = renorm
        ctx.mark_non_differentiable(idx, m_sizes, sort_idx, inv)
        return wc, idx, m_sizes, sort_idx, inv

    @staticmethod
    def backward(ctx, dw, *_unused):
        logits, idx, w32 = ctx.saved_tensors
        return _softmax_topk_backward(logits, idx, w32, ctx.renorm, dw), None, None, None, None


def route_and_sort(logits: torch.Tensor, k: int, renorm: bool, out_dtype: Optional[torch.dtype],
                   num_experts: int):
    """(routing_weights (T,k) in ``out_dtype``, selected_experts (T,k) int64, m_sizes, sort_idx,
    inv_sort_idx): ``softmax_topk`` followed by ``get_expert_counts_and_idx`` on its selections
    (modular_qwen3_moe_fused.py:87-93,102)."""
    if not (torch.is_grad_enabled() and logits.requires_grad):
        # nothing to differentiate (inference, frozen router): skip the autograd function, whose bookkeeping
        # costs as much host time as the call itself
        assert logits.shape[1] == num_experts
        return _route_and_sort_raw(logits, k, renorm, out_dtype)[1:]
    return _RouteAndSort.apply(logits, k, renorm, out_dtype, num_experts)


def softmax_topk(logits: torch.Tensor, k: int, renorm: bool,
                 out_dtype: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(routing_weights (T,k) in ``out_dtype``, selected_experts (T,k) int64)."""
    return _SoftmaxTopk.apply(logits, k, renorm, out_dtype)


def _gather(src: torch.Tensor, idx: torch.Tensor, div: int, row_scale: Optional[torch.Tensor]) -> torch.Tensor:
    assert src.is_cuda and src.ndim == 2 and src.is_contiguous()
    assert idx.dtype == torch.int32 and idx.is_contiguous()
    out = torch.empty((idx.numel(), src.shape[1]), device=src.device, dtype=src.dtype)
    if row_scale is not None:
        assert row_scale.dtype == src.dtype and row_scale.is_contiguous()
    rc = _lib.lib().mfl_gather_rows(_lib.ptr(src), _lib.ptr(idx), div, _lib.ptr(row_scale), _lib.ptr(out), idx.numel(),
                                    src.shape[1], _lib.dtype_code(src.dtype), _lib.stream())
    _lib.check(rc, "mfl_gather_rows")
    return out


def _scatter(src: torch.Tensor, pos: torch.Tensor, k: int, row_scale: Optional[torch.Tensor]) -> torch.Tensor:
    """out[pos[r * k + j]] = src[r] (* row_scale[r * k + j]): ``_gather`` with idx the inverse of ``pos``, every
    source row read once."""
    assert src.is_cuda and src.ndim == 2 and src.is_contiguous()
    assert pos.dtype == torch.int32 and pos.is_contiguous() and pos.numel() == src.shape[0] * k
    out = torch.empty((pos.numel(), src.shape[1]), device=src.device, dtype=src.dtype)
    if row_scale is not None:
        assert row_scale.dtype == src.dtype and row_scale.is_contiguous() and row_scale.numel() == pos.numel()
    rc = _lib.lib().mfl_scatter_rows(_lib.ptr(src), _lib.ptr(pos), k, _lib.ptr(row_scale), _lib.ptr(out), src.shape[0],
                                     src.shape[1], _lib.dtype_code(src.dtype), _lib.stream())
    _lib.check(rc, "mfl_scatter_rows")
    return out


def _combine(src: torch.Tensor, pos: torch.Tensor, weights: Optional[torch.Tensor], T: int, k: int) -> torch.Tensor:
    assert src.is_cuda and src.ndim == 2 and src.is_contiguous()
    assert pos.dtype == torch.int32 and pos.is_contiguous() and pos.numel() == T * k
    if weights is not None:
        assert weights.dtype == src.dtype and weights.is_contiguous() and weights.numel() == T * k
    out = torch.empty((T, src.shape[1]), device=src.device, dtype=src.dtype)
    rc = _lib.lib().mfl_combine_rows(_lib.ptr(src), _lib.ptr(pos), _lib.ptr(weights), _lib.ptr(out), T, k, src.shape[1],
                                     _lib.dtype_code(src.dtype), _lib.stream())
    _lib.check(rc, "mfl_combine_rows")
    return out


class _GatherRows(torch.autograd.Function):
    """out[j] = src[idx[j] // div]; ``inv`` is the inverse permutation of ``idx``
    (row r of the un-divided source order sits at out[inv[r]])."""

    @staticmethod
    def forward(ctx, src, idx, div, inv):
        ctx.save_for_backward(inv)
        ctx.div = div
        ctx.n_src = src.shape[0]
        if div > 1 and inv.numel() == src.shape[0] * div:
            return _scatter(src, inv, div, None)  # every source row read once, not div times
        return _gather(src, idx, div, None)

    @staticmethod
    def backward(ctx, dout):
        (inv,) = ctx.saved_tensors
        # d src[t] = sum_{j<div} dout[inv[t*div + j]]
        return _combine(dout.contiguous(), inv, None, ctx.n_src, ctx.div), None, None, None


def gather_rows(src: torch.Tensor, idx: torch.Tensor, div: int, inv: torch.Tensor) -> torch.Tensor:
    """Replicate every row of ``src`` ``div`` times and permute by ``idx`` in one pass
    (modular_qwen3_moe_fused.py:95-103 with idx = sort_idx, div = num_selected)."""
    return _GatherRows.apply(src, idx, div, inv)


class _CombineRows(torch.autograd.Function):
    """out[t] = sum_j y[pos[t*k+j]] * w[t, j]  (modular_qwen3_moe_fused.py:112-115)."""

    @staticmethod
    def forward(ctx, y, pos, w, sort_idx):
        T, k = w.shape
        wc = w.contiguous()
        ctx.save_for_backward(y, pos, wc, sort_idx)
        return _combine(y, pos, wc.view(-1), T, k)

    @staticmethod
    def backward(ctx, dout):
        y, pos, w, sort_idx = ctx.saved_tensors
        T, k = w.shape
        dout = dout.contiguous()
        dy = dw = None
        if ctx.needs_input_grad[0]:
            # dy[i] = dout[sort_idx[i] // k] * w.flat[sort_idx[i]]
            dy = _scatter(dout, pos, k, w.view(-1)) if k > 1 else _gather(dout, sort_idx, k, w.view(-1))
        if ctx.needs_input_grad[2]:
            dw = torch.empty_like(w)
            rc = _lib.lib().mfl_rows_dot(_lib.ptr(dout), _lib.ptr(y), _lib.ptr(pos), _lib.ptr(dw), T, k, y.shape[1],
                                         _lib.dtype_code(y.dtype), _lib.stream())
            _lib.check(rc, "mfl_rows_dot")
        return dy, None, dw, None


def combine_rows(y: torch.Tensor, inv_sort_idx: torch.Tensor, weights: torch.Tensor,
                 sort_idx: torch.Tensor) -> torch.Tensor:
    """Un-sort the expert outputs and sum each token's k rows with its routing weights."""
    return _CombineRows.apply(y, inv_sort_idx, weights, sort_idx)
