"""benchmark configuration 1 against the committed fixture tests/golden/config1.npz (made by
tests/golden/make_golden.py from float64 library routines): the oracle on the CPU, and the
HIP path on the GPU."""
import os

import numpy as np
import pytest
import torch

import oracle

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz"))
E, K, N, T, TOPK = 8, 64, 128, 256, 2


def _rows():
    x = np.repeat(FIX["hidden"], TOPK, axis=0)
    sel = FIX["selected_experts"].reshape(-1)
    return x, sel


def test_oracle_reproduces_config1():
    x, sel = _rows()
    w, idx = oracle.softmax_topk(FIX["logits"], TOPK, False)
    np.testing.assert_array_equal(idx, FIX["selected_experts"])
    np.testing.assert_allclose(w, FIX["routing_weights"], rtol=1e-6)
    c, s, i = oracle.expert_counts_and_idx(sel, E)
    np.testing.assert_array_equal(c, FIX["m_sizes"])
    np.testing.assert_array_equal(s, FIX["sort_idx"])
    np.testing.assert_array_equal(i, FIX["inv_sort_idx"])
    np.testing.assert_allclose(oracle.linear_fwd(x, FIX["weight"], sel), FIX["out"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.linear_bwd_input(FIX["grad_out"], FIX["weight"], sel), FIX["grad_input"],
                               rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.linear_bwd_weight(FIX["grad_out"], x, sel, E), FIX["grad_weight"],
                               rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_hip_path_reproduces_config1():
    from qwen3_moe_fused.functional import moe_fused_linear, moe_fused_linear_unsorted
    from qwen3_moe_fused.kernels.indexing import get_expert_counts_and_idx
    from qwen3_moe_fused.kernels.routing import gather_rows, softmax_topk_raw

    dev = "cuda"
    w32, _, idx = softmax_topk_raw(torch.from_numpy(FIX["logits"]).to(dev), TOPK, False, torch.float32)
    assert np.array_equal(idx.cpu().numpy(), FIX["selected_experts"])
    np.testing.assert_allclose(w32.cpu().numpy(), FIX["routing_weights"], rtol=2e-6)
    m_sizes, sort_idx, inv = get_expert_counts_and_idx(idx.view(-1), E)
    assert np.array_equal(m_sizes.cpu().numpy(), FIX["m_sizes"])
    assert np.array_equal(sort_idx.cpu().numpy(), FIX["sort_idx"])
    assert np.array_equal(inv.cpu().numpy(), FIX["inv_sort_idx"])

    hidden = torch.from_numpy(FIX["hidden"]).to(dev)
    weight = torch.from_numpy(FIX["weight"]).to(dev).requires_grad_()
    x = gather_rows(hidden, sort_idx, TOPK, inv).requires_grad_()
    y = moe_fused_linear(x, weight, m_sizes)                 # fp32 path, sorted rows
    dy_sorted = torch.from_numpy(FIX["grad_out"]).to(dev)[sort_idx.long()]
    y.backward(dy_sorted)
    s = FIX["sort_idx"].astype(np.int64)
    np.testing.assert_allclose(y.detach().cpu().numpy(), FIX["out"][s], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(x.grad.cpu().numpy(), FIX["grad_input"][s], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(weight.grad.cpu().numpy(), FIX["grad_weight"], rtol=1e-4, atol=1e-5)
    # the selected_experts form of the call (north-star signature): no pre-sorting by the caller
    rows = torch.from_numpy(np.repeat(FIX["hidden"], TOPK, axis=0)).to(dev)
    out = moe_fused_linear_unsorted(rows, weight.detach(), idx.view(-1))
    np.testing.assert_allclose(out.cpu().numpy(), FIX["out"], rtol=1e-4, atol=1e-5)
