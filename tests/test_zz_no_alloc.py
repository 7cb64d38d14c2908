"""The entry point that allocates nothing (mfl_expert_sort_static) against mfl_expert_sort, through
the C ABI: same counts, sort_idx and inv_sort_idx bit for bit, on two calls in a row, the second
with a smaller input (the library's fixed table array keeps the first call's contents), and on a
call after other work has used the GPU.  "Allocates nothing" is read from the driver (free device memory
before and after a call, once the first call on the device has looked up the array's address and set the
kernels' attributes) as well as from torch's allocator, which would not see a hipMalloc inside the library."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

from qwen3_moe_fused import _lib  # noqa: E402

DEV = "cuda"


def _sort_with_workspace(sel, E):
    R = sel.numel()
    lib = _lib.lib()
    counts = torch.empty(E, dtype=torch.int32, device=DEV)
    sort_idx = torch.empty(R, dtype=torch.int32, device=DEV)
    inv = torch.empty(R, dtype=torch.int32, device=DEV)
    ws_bytes = lib.mfl_expert_sort_workspace(R, E)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=DEV)
    rc = lib.mfl_expert_sort(_lib.ptr(sel), _lib.itype_code(sel.dtype), R, E, _lib.ptr(counts), _lib.ptr(sort_idx),
                             _lib.ptr(inv), _lib.ptr(ws), ws_bytes, _lib.stream())
    assert rc == 0, rc
    return counts, sort_idx, inv


def _sort_static(sel, E, outputs=None):
    R = sel.numel()
    if outputs is None:
        outputs = (torch.empty(E, dtype=torch.int32, device=DEV), torch.empty(R, dtype=torch.int32, device=DEV),
                   torch.empty(R, dtype=torch.int32, device=DEV))
    counts, sort_idx, inv = outputs
    rc = _lib.lib().mfl_expert_sort_static(_lib.ptr(sel), _lib.itype_code(sel.dtype), R, E, _lib.ptr(counts),
                                           _lib.ptr(sort_idx), _lib.ptr(inv), _lib.stream())
    assert rc == 0, rc
    return counts, sort_idx, inv


def _keys(R, E, seed, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, E, (R,), generator=g).to(dtype).to(DEV)


def test_static_sort_matches_workspace_sort_on_two_calls_in_a_row():
    cases = [(131072, 128, 1, torch.int64), (1000, 16, 2, torch.int32)]   # the second call is the smaller one
    for R, E, seed, dtype in cases:
        sel = _keys(R, E, seed, dtype)
        # outputs are allocated before the call; between here and the comparison the static call allocates nothing
        outs = (torch.empty(E, dtype=torch.int32, device=DEV), torch.empty(R, dtype=torch.int32, device=DEV),
                torch.empty(R, dtype=torch.int32, device=DEV))
        _sort_static(sel, E, outs)          # the first call on a device does the one-time set-up
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        got = _sort_static(sel, E, outs)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated during the call"
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "torch allocated during the call"
        ref = _sort_with_workspace(sel, E)
        for a, b, name in zip(got, ref, ("counts", "sort_idx", "inv_sort_idx")):
            assert torch.equal(a, b), f"{name} differs at R={R}, E={E}"
        c_ref, s_ref, i_ref = oracle.expert_counts_and_idx(sel.cpu().numpy(), E)
        assert np.array_equal(got[0].cpu().numpy(), c_ref) and np.array_equal(got[1].cpu().numpy(), s_ref)
        assert np.array_equal(got[2].cpu().numpy(), i_ref)


def test_static_sort_edges_and_limit():
    lib = _lib.lib()
    # counts only, empty input, the largest table (E = 512, more rows than the wave cap covers one to one)
    sel = _keys(300000, 512, 3)
    got = _sort_static(sel, 512)
    ref = _sort_with_workspace(sel, 512)
    assert all(torch.equal(a, b) for a, b in zip(got, ref))
    counts = torch.full((8,), -1, dtype=torch.int32, device=DEV)
    rc = lib.mfl_expert_sort_static(None, _lib.I64, 0, 8, _lib.ptr(counts), None, None, _lib.stream())
    assert rc == 0 and torch.count_nonzero(counts).item() == 0
    sel = _keys(5000, 8, 4)
    rc = lib.mfl_expert_sort_static(_lib.ptr(sel), _lib.I64, 5000, 8, _lib.ptr(counts), None, None, _lib.stream())
    assert rc == 0 and torch.equal(counts.cpu(), torch.bincount(sel.cpu(), minlength=8).int())
    # beyond the maximum: a clear error, nothing enqueued
    sel = _keys(100, 513, 5)
    c513 = torch.empty(513, dtype=torch.int32, device=DEV)
    rc = lib.mfl_expert_sort_static(_lib.ptr(sel), _lib.I64, 100, 513, _lib.ptr(c513), None, None, _lib.stream())
    assert rc == -7 and b"maximum" in lib.mfl_strerror(rc)
