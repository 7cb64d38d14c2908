"""Expert histogram and stable expert sort (reference: qwen3_moe_fused/kernels/indexing.py).

The reference builds an (E, M) compare matrix under ``torch.compile``; here one library call
(``mfl_expert_sort``: wave ballots + LDS histograms, no atomics) yields the same int32 outputs.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _lib


def _sort(s: torch.Tensor, E: int, want_idx: bool) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    assert s.is_cuda, "expert ids must live on the GPU"
    assert s.ndim == 1
    s = _lib.as_index_tensor(s).contiguous()
    R = s.numel()
    ws_bytes = _lib.lib().mfl_expert_sort_workspace(R, E)
    # one allocation for all int32 outputs and the scratch table (fewer allocator calls per layer)
    n_out = E + (2 * R if want_idx else 0)
    buf = torch.empty(n_out + (ws_bytes + 3) // 4 + 64, device=s.device, dtype=torch.int32)
    counts = buf[:E]
    sort_idx = inv_sort_idx = None
    if want_idx:
        sort_idx, inv_sort_idx = buf[E:E + R], buf[E + R:E + 2 * R]
    ws = buf[(n_out + 63) // 64 * 64:]                      # 256-byte aligned offset into a 256-byte aligned block
    rc = _lib.lib().mfl_expert_sort(_lib.ptr(s), _lib.itype_code(s.dtype), R, E, _lib.ptr(counts), _lib.ptr(sort_idx),
                                    _lib.ptr(inv_sort_idx), _lib.ptr(ws), ws_bytes, _lib.stream())
    _lib.check(rc, "mfl_expert_sort")
    return counts, sort_idx, inv_sort_idx


@torch.no_grad()
def get_expert_counts(s: torch.Tensor, E: int) -> torch.Tensor:
    """counts[e] = number of rows routed to expert e (int32).  indexing.py:18-23."""
    return _sort(s, E, False)[0]


@torch.no_grad()
def get_expert_counts_and_idx(s: torch.Tensor, E: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(m_sizes, sort_idx, inv_sort_idx)``, all int32: ``x[sort_idx]`` groups rows by
    expert in a stable order, ``y[inv_sort_idx]`` undoes it.  indexing.py:48-65 (whose locals
    call the last two ``inv_idx`` and ``idx``)."""
    counts, sort_idx, inv_sort_idx = _sort(s, E, True)
    return counts, sort_idx, inv_sort_idx


@torch.no_grad()
def sort_experts(s: torch.Tensor, E: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(s_sorted, sort_idx, inv_sort_idx)`` with ``s_sorted`` int32.  indexing.py:27-45."""
    counts, sort_idx, inv_sort_idx = _sort(s, E, True)
    experts = torch.arange(E, device=s.device, dtype=torch.int32)
    s_sorted = torch.repeat_interleave(experts, counts.to(torch.int64), output_size=s.numel())
    return s_sorted, sort_idx, inv_sort_idx


@torch.no_grad()
def get_batch_begins_ends(s: torch.Tensor, E: int) -> torch.Tensor:
    """For ``s`` sorted ascending: (E, 2) int32 of [begin, end) row ranges per expert.
    indexing.py:7-14."""
    counts = _sort(s, E, False)[0]
    ends = torch.cumsum(counts, dim=0, dtype=torch.int32)
    return torch.stack([ends - counts, ends], dim=1)
