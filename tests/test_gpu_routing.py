"""GPU parity of softmax-top-k routing, the stable expert sort and the gather / combine
kernels.  Index outputs are compared bit for bit with the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, randn, to_np32, zipf_bias

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.kernels.indexing import (get_batch_begins_ends, get_expert_counts,  # noqa: E402
                                              get_expert_counts_and_idx, sort_experts)
from qwen3_moe_fused.kernels.routing import combine_rows, gather_rows, softmax_topk, softmax_topk_raw  # noqa: E402

DEV = "cuda"


def _tie_free_rows(logits: np.ndarray, k: int) -> np.ndarray:
    """Rows whose top k+1 probabilities are separated by a relative gap that no ulp-level
    difference in exp() can bridge; only there is the top-k order independent of the exp()
    implementation."""
    p = torch.softmax(torch.from_numpy(logits).double(), -1).numpy()
    top = -np.sort(-p, axis=1)[:, : k + 1]
    gap = (top[:, :-1] - top[:, 1:]) / top[:, :-1]
    return (gap > 1e-5).all(axis=1)


def _check_near_tie_rows(logits: np.ndarray, idx: np.ndarray, idx_ref: np.ndarray, rows, E: int, gap=1e-5):
    """Rows that hold a near-tie among their top k+1 probabilities: an ulp of difference between two
    exp() implementations may order the tied experts either way.  Everything else is still fixed:
    ids in range and distinct, and wherever the two answers differ at a position the two experts
    named there have probabilities within `gap` (relative) of each other."""
    p = torch.softmax(torch.from_numpy(logits).double(), -1).numpy()
    for r in rows:
        got, ref = idx[r], idx_ref[r]
        assert got.min() >= 0 and got.max() < E and len(set(got.tolist())) == len(got), f"row {r}: {got}"
        for a, b in zip(got, ref):
            if a != b:
                assert abs(p[r, a] - p[r, b]) <= gap * p[r, b], f"row {r}: experts {a} and {b} are not near-tied"


def test_softmax_topk_near_ties_are_checked_too():
    """A fixture in which every row has a near-tie inside its top k and one across the k / k+1
    boundary (logits that differ by one fp32 ulp): ids stay in range and distinct, differ from the
    oracle only inside a near-tied pair, and the routing weights agree on every row."""
    T, E, k = 512, 128, 8
    logits = randn((T, E), gen(77), 1.0).numpy()
    order = np.argsort(-logits, axis=1)
    rows = np.arange(T)
    for hi, lo in ((2, 3), (k - 1, k)):                 # ranks tied inside the top k / across its edge
        logits[rows, order[:, lo]] = np.nextafter(logits[rows, order[:, hi]], np.float32(-np.inf))
    clear = _tie_free_rows(logits, k)
    assert not clear.any()
    w_ref, idx_ref = oracle.softmax_topk(logits, k, True)
    w32, _, idx = softmax_topk_raw(torch.from_numpy(logits).to(DEV), k, True, torch.float32)
    _check_near_tie_rows(logits, idx.cpu().numpy(), idx_ref, rows, E)
    np.testing.assert_allclose(w32.cpu().numpy(), w_ref, rtol=2e-5, atol=1e-9)


@pytest.mark.parametrize("T,E,k,renorm", [(256, 8, 2, False), (4096, 128, 8, True), (4096, 128, 8, False),
                                          (37, 11, 3, True), (100, 60, 4, True), (64, 256, 8, True),
                                          (16, 1000, 6, True)])
def test_softmax_topk_matches_oracle(T, E, k, renorm):
    logits = randn((T, E), gen(100 + T + E), 1.0)
    lnp = logits.numpy()
    clear = _tie_free_rows(lnp, min(k, E - 1))
    assert clear.mean() > 0.99
    w_ref, idx_ref = oracle.softmax_topk(lnp, k, renorm)
    w32, wc, idx = softmax_topk_raw(logits.to(DEV), k, renorm, torch.bfloat16)
    assert idx.dtype == torch.int64
    idx_np = idx.cpu().numpy()
    assert np.array_equal(idx_np[clear], idx_ref[clear]), "expert ids must match bit for bit"
    _check_near_tie_rows(lnp, idx_np, idx_ref, np.nonzero(~clear)[0], E)
    np.testing.assert_allclose(w32.cpu().numpy(), w_ref, rtol=2e-6, atol=1e-9)
    assert torch.equal(wc, w32.to(torch.bfloat16))


def test_softmax_topk_tie_rule_and_bf16_logits():
    # exact duplicates: the lower expert id comes first
    logits = torch.tensor([[1.0, 3.0, 3.0, 0.5, 3.0, -1.0, 2.0, 2.0]] * 5)
    _, _, idx = softmax_topk_raw(logits.to(DEV), 5, True, torch.float32)
    assert idx[0].tolist() == [1, 2, 4, 6, 7]
    w_ref, idx_ref = oracle.softmax_topk(logits.numpy(), 5, True)
    assert np.array_equal(idx.cpu().numpy(), idx_ref)
    # bf16 logits (what a bf16 gate produces) are widened to fp32 first
    lg = randn((512, 128), gen(9), 1.0, torch.bfloat16)
    w_ref, idx_ref = oracle.softmax_topk(to_np32(lg), 8, True)
    _, _, idx = softmax_topk_raw(lg.to(DEV), 8, True)
    # bf16 logits have many exact ties; with the declared rule the ids still agree except
    # where two different logits round to the same probability in one implementation only
    agree = (idx.cpu().numpy() == idx_ref).mean()
    assert agree > 0.999


@pytest.mark.parametrize("R,E,dtype", [(512, 8, torch.int64), (32768, 128, torch.int64), (32768, 128, torch.int32),
                                       (131072, 128, torch.int64), (1, 4, torch.int64), (0, 4, torch.int64),
                                       (1001, 11, torch.int64), (70000, 60, torch.int64), (5000, 1000, torch.int32),
                                       (300000, 16, torch.int64)])
def test_expert_sort_bit_exact(R, E, dtype):
    g = gen(R + E)
    if R >= 32768 and E == 128:
        # real routing: top-8 of softmax over Zipf-skewed logits, flattened
        T = R // 8
        logits = torch.randn((T, E), generator=g) + zipf_bias(E, 1.2, g)
        s = torch.topk(torch.softmax(logits, -1), 8, -1).indices.reshape(-1)
    else:
        s = torch.randint(0, E, (R,), generator=g)
    c_ref, sort_ref, inv_ref = oracle.expert_counts_and_idx(s.numpy(), E)
    c, sort_idx, inv = get_expert_counts_and_idx(s.to(dtype).to(DEV), E)
    assert c.dtype == sort_idx.dtype == inv.dtype == torch.int32
    assert np.array_equal(c.cpu().numpy(), c_ref)
    assert np.array_equal(sort_idx.cpu().numpy(), sort_ref)
    assert np.array_equal(inv.cpu().numpy(), inv_ref)
    assert np.array_equal(get_expert_counts(s.to(dtype).to(DEV), E).cpu().numpy(), c_ref)


def test_sort_helpers():
    s = torch.randint(0, 7, (500,), generator=gen(1))
    s_sorted, sort_idx, inv = sort_experts(s.to(DEV), 7)
    assert s_sorted.dtype == torch.int32
    assert torch.equal(s_sorted.cpu().long(), torch.sort(s, stable=True).values)
    assert torch.equal(sort_idx.cpu().long(), torch.sort(s, stable=True).indices)
    be = get_batch_begins_ends(s_sorted.to(DEV), 7).cpu()
    counts = torch.bincount(s, minlength=7)
    assert torch.equal(be[:, 1] - be[:, 0], counts.int())
    assert be[0, 0] == 0 and be[-1, 1] == 500


@pytest.mark.parametrize("T,k,H,dtype", [(256, 2, 64, torch.float32), (4096, 8, 2048, torch.bfloat16),
                                         (91, 3, 16, torch.float32), (50, 4, 36, torch.bfloat16)])
def test_gather_and_combine(T, k, H, dtype):
    g = gen(T + H)
    E = 16
    hidden = randn((T, H), g, 1.0, dtype)
    sel = torch.randint(0, E, (T * k,), generator=g)
    rw = torch.rand((T, k), generator=g).to(dtype)
    _, sort_ref, inv_ref = oracle.expert_counts_and_idx(sel.numpy(), E)
    sort_idx, inv = torch.from_numpy(sort_ref).to(DEV), torch.from_numpy(inv_ref).to(DEV)

    x = gather_rows(hidden.to(DEV), sort_idx, k, inv)
    exp = hidden.repeat_interleave(k, dim=0)[torch.from_numpy(sort_ref).long()]   # modular...:95-103
    assert torch.equal(x.cpu(), exp), "gather is a pure copy: bit exact"

    y = randn((T * k, H), g, 1.0, dtype)
    out = combine_rows(y.to(DEV), inv, rw.to(DEV), sort_idx)
    ref = np.einsum("beo,be->bo", to_np32(y)[inv_ref].reshape(T, k, H).astype(np.float64), to_np32(rw).astype(np.float64))
    check_close(out, ref, 1e-2 if dtype == torch.bfloat16 else 1e-5, 1e-2 if dtype == torch.bfloat16 else 1e-5,
                "combine")


@pytest.mark.parametrize("T,k,H,dtype,scaled", [(300, 8, 2048, torch.bfloat16, False), (300, 8, 2048, torch.bfloat16, True),
                                                  (41, 3, 100, torch.float32, True), (64, 2, 36, torch.float16, False),
                                                  (5, 1, 8, torch.float32, True)])
def test_scatter_form_of_the_row_copy_equals_the_gather_form(T, k, H, dtype, scaled):
    from qwen3_moe_fused.kernels.routing import _gather, _scatter

    g = gen(T + H)
    src = randn((T, H), g, 1.0, dtype).to(DEV)
    sort_idx = torch.randperm(T * k, generator=g).to(torch.int32)
    inv = torch.empty_like(sort_idx)
    inv[sort_idx.long()] = torch.arange(T * k, dtype=torch.int32)
    scale = randn((T * k,), g, 1.0, dtype).to(DEV) if scaled else None
    a = _gather(src, sort_idx.to(DEV), k, scale)
    b = _scatter(src, inv.to(DEV), k, scale)
    assert torch.equal(a, b)
    exp = src.cpu()[(sort_idx.long() // k)]
    if scaled:
        exp = (exp.float() * scale.cpu().float()[sort_idx.long()][:, None]).to(dtype)
    assert torch.equal(a.cpu(), exp)


def test_gather_combine_autograd_fp32():
    """Gradients of gather / combine / softmax-top-k against torch autograd of the reference's
    formulation (modular_qwen3_moe_fused.py:87-115)."""
    T, k, H, E = 40, 3, 24, 6
    g = gen(5)
    hidden = randn((T, H), g).to(DEV).requires_grad_()
    logits = randn((T, E), g).to(DEV).requires_grad_()
    wts = randn((T * k, H), g).to(DEV)

    rw, sel = softmax_topk(logits, k, True, torch.float32)
    c, sort_idx, inv = get_expert_counts_and_idx(sel.view(-1), E)
    x = gather_rows(hidden, sort_idx, k, inv)
    y = x * wts            # any row-wise differentiable op between gather and combine
    out = combine_rows(y, inv, rw, sort_idx)
    loss_w = randn((T, H), g).to(DEV)
    (out * loss_w).sum().backward()

    h2 = hidden.detach().clone().requires_grad_()
    l2 = logits.detach().clone().requires_grad_()
    p = torch.softmax(l2, dim=1, dtype=torch.float32)
    rw2, sel2 = torch.topk(p, k, dim=-1)
    rw2 = rw2 / rw2.sum(dim=-1, keepdim=True)
    assert torch.equal(sel2, sel)
    x2 = h2.unsqueeze(1).expand(T, k, H).reshape(T * k, H)[sort_idx.long()]
    y2 = (x2 * wts)[inv.long()].view(T, k, H)
    out2 = torch.einsum("beo,be->bo", y2, rw2)
    (out2 * loss_w).sum().backward()
    torch.testing.assert_close(out, out2, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(hidden.grad, h2.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(logits.grad, l2.grad, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("T,k,H,dtype", [(300, 8, 2048, torch.bfloat16), (50, 3, 40, torch.bfloat16),
                                         (50, 5, 36, torch.bfloat16), (33, 2, 4104, torch.bfloat16),
                                         (64, 8, 64, torch.float32)])
def test_rows_dot_against_numpy(T, k, H, dtype):
    """dots[t, j] = <a[t], b[pos[t*k+j]]> (gradient of the combine with respect to the routing
    weights): vector path, scalar path (row length not a multiple of 16 bytes), rows longer than
    one pass of the wave, k not a multiple of the rows in flight."""
    from qwen3_moe_fused import _lib

    g = gen(T + H)
    a = randn((T, H), g, 1.0, dtype)
    b = randn((T * k, H), g, 1.0, dtype)
    pos = torch.randperm(T * k, generator=g).to(torch.int32)
    dots = torch.empty((T, k), dtype=dtype, device=DEV)
    ad, bd, pd = a.to(DEV), b.to(DEV), pos.to(DEV)
    rc = _lib.lib().mfl_rows_dot(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(pd), _lib.ptr(dots), T, k, H,
                                 _lib.dtype_code(dtype), _lib.stream())
    _lib.check(rc, "mfl_rows_dot")
    ref = np.einsum("th,tjh->tj", to_np32(a).astype(np.float64),
                    to_np32(b)[pos.numpy().astype(np.int64)].reshape(T, k, H).astype(np.float64))
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-5
    check_close(dots, ref, tol, tol, "rows_dot")


def _check_route_outputs(logits, k, E, w, sel, m_sizes, sort_idx, inv):
    _, w_ref, sel_ref = softmax_topk_raw(logits, k, True, torch.bfloat16)
    c_ref, s_ref, i_ref = get_expert_counts_and_idx(sel_ref.view(-1), E)
    assert torch.equal(sel, sel_ref) and torch.equal(w, w_ref)
    assert torch.equal(m_sizes, c_ref) and torch.equal(sort_idx, s_ref) and torch.equal(inv, i_ref)
    # and against the oracle
    c_o, s_o, i_o = oracle.expert_counts_and_idx(sel.view(-1).cpu().numpy(), E)
    assert np.array_equal(m_sizes.cpu().numpy(), c_o) and np.array_equal(sort_idx.cpu().numpy(), s_o)
    assert np.array_equal(inv.cpu().numpy(), i_o)


# one launch up to 64 tokens; two launches (top-k that counts, scatter) above; three where the two-launch form
# does not apply: more than 512 experts, more than 1024 segments of 256 selections
@pytest.mark.parametrize("T,E,k,dtype", [(16, 128, 8, torch.float32), (1, 128, 8, torch.bfloat16), (64, 128, 8, torch.bfloat16),
                                         (7, 11, 3, torch.float32), (60, 512, 6, torch.float32), (33, 60, 1, torch.float32),
                                         (65, 128, 8, torch.float32), (129, 128, 8, torch.float32),
                                         (4096, 128, 8, torch.bfloat16), (777, 60, 3, torch.float32),
                                         (5000, 512, 6, torch.float32), (300, 600, 4, torch.float32),
                                         (33000, 128, 8, torch.bfloat16), (2049, 64, 64, torch.float32)])
def test_route_and_sort_equals_the_separate_calls(T, E, k, dtype):
    from qwen3_moe_fused.kernels.routing import route_and_sort

    logits = randn((T, E), gen(T + E), 2.0, dtype).to(DEV)
    w, sel, m_sizes, sort_idx, inv = route_and_sort(logits, k, True, torch.bfloat16, E)
    _check_route_outputs(logits, k, E, w, sel, m_sizes, sort_idx, inv)


@pytest.mark.parametrize("T", [200, 4096])
def test_route_and_sort_with_a_row_of_nan(T):
    """A token whose logits are all NaN selects no expert (no probability compares greater than another): its
    k selections are left out of the counts and of the sort, and every other token is routed as without it.
    The histogram pass of the two-launch form must not count the row's "no expert" id."""
    from qwen3_moe_fused.kernels.routing import route_and_sort

    E, k, bad = 128, 8, T // 3
    clean = randn((T, E), gen(T), 2.0, torch.float32)
    logits = clean.clone()
    logits[bad] = float("nan")
    w, sel, m_sizes, sort_idx, inv = route_and_sort(logits.to(DEV), k, True, torch.float32, E)
    torch.cuda.synchronize()
    keep = np.ones(T, bool)
    keep[bad] = False
    _, sel_ref = oracle.softmax_topk(clean.numpy()[keep], k, True)
    assert np.array_equal(sel.cpu().numpy()[keep], sel_ref), "the other tokens are routed as without the row"
    counts_ref = oracle.expert_counts(sel_ref.reshape(-1), E)
    assert np.array_equal(m_sizes.cpu().numpy(), counts_ref) and int(m_sizes.sum()) == (T - 1) * k
    # the sorted positions of the other tokens' selections are those of the stable sort without the row
    flat_keep = np.repeat(keep, k)
    _, s_ref, _ = oracle.expert_counts_and_idx(sel_ref.reshape(-1), E)
    orig = np.nonzero(flat_keep)[0]
    assert np.array_equal(sort_idx.cpu().numpy()[: (T - 1) * k], orig[s_ref])


@pytest.mark.parametrize("T,E,k", [(128, 128, 8), (100, 512, 6), (65, 40, 5)])
def test_one_launch_entry_point_up_to_its_own_limit(T, E, k):
    # mfl_route_sort uses the one-workgroup form up to 64 tokens; the entry point itself takes up to 128
    from qwen3_moe_fused import _lib

    logits = randn((T, E), gen(T), 2.0).to(DEV)
    w = torch.empty((T, k), device=DEV, dtype=torch.bfloat16)
    sel = torch.empty((T, k), device=DEV, dtype=torch.int64)
    m_sizes = torch.empty(E, device=DEV, dtype=torch.int32)
    sort_idx = torch.empty(T * k, device=DEV, dtype=torch.int32)
    inv = torch.empty(T * k, device=DEV, dtype=torch.int32)
    rc = _lib.lib().mfl_route_sort_small(_lib.ptr(logits), _lib.dtype_code(logits.dtype), T, E, k, 1, None, _lib.ptr(w),
                                         _lib.dtype_code(w.dtype), _lib.ptr(sel), _lib.ptr(m_sizes), _lib.ptr(sort_idx),
                                         _lib.ptr(inv), _lib.stream())
    _lib.check(rc, "mfl_route_sort_small")
    _check_route_outputs(logits, k, E, w, sel, m_sizes, sort_idx, inv)


@pytest.mark.parametrize("dw_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("renorm", [True, False])
@pytest.mark.parametrize("T,E,k", [(37, 8, 2), (4096, 128, 8), (5, 1000, 64), (64, 130, 3), (1, 64, 1)])
def test_routing_weight_gradient_matches_autograd_in_fp64(T, E, k, renorm, dw_dtype):
    """d logits of the routing weights (one kernel) against autograd of the textbook composition
    softmax -> topk -> renormalise (modular_qwen3_moe_fused.py:87-93) in fp64."""
    g = gen(T + E + k)
    logits = randn((T, E), g)
    dw = randn((T, k), g).to(dw_dtype)
    ld = logits.to(DEV).requires_grad_()
    w, idx = softmax_topk(ld, k, renorm, torch.float32)
    (w * dw.to(DEV).float()).sum().backward()
    l64 = logits.double().requires_grad_()
    p = torch.softmax(l64, dim=-1)
    w64 = p.gather(1, idx.cpu())              # the same selections: the gradient of the weights, not of the choice
    if renorm:
        w64 = w64 / w64.sum(dim=-1, keepdim=True)
    (w64 * dw.double()).sum().backward()
    ref = l64.grad.numpy()
    check_close(ld.grad, ref, rtol=1e-4, atol=1e-6 * max(1.0, float(np.abs(ref).max())), what="d logits")
    assert ld.grad.dtype == torch.float32


def test_routing_weight_gradient_bf16_logits_through_route_and_sort():
    from qwen3_moe_fused.kernels.routing import route_and_sort
    g = gen(91)
    T, E, k = 300, 128, 8
    logits = randn((T, E), g).bfloat16()
    dw = randn((T, k), g).bfloat16()
    ld = logits.to(DEV).requires_grad_()
    w, idx, *_ = route_and_sort(ld, k, True, torch.bfloat16, E)
    (w.float() * dw.to(DEV).float()).sum().backward()
    l64 = logits.double().requires_grad_()
    p = torch.softmax(l64, dim=-1)
    w64 = p.gather(1, idx.cpu())
    w64 = w64 / w64.sum(dim=-1, keepdim=True)
    (w64 * dw.double()).sum().backward()
    assert ld.grad.dtype == torch.bfloat16
    check_close(ld.grad, l64.grad.numpy(), rtol=1e-2, atol=1e-2 * float(l64.grad.abs().max()), what="d logits (bf16)")
