"""Pins the CPU oracle (oracle/moe_oracle.c) with checks that do not retype its formulas:
library routines that the math reduces to, autograd, brute force on tiny inputs, invariants.
The reference ships no golden vectors or fixtures for this path (its test scripts draw
unseeded CUDA inputs and print), so these checks -- plus tests/golden -- are what the parity
claims rest on.  A plausible slip (transposed operand, dropped term, wrong sign, off-by-one
index, unstable sort) fails at least one of them."""
import itertools

import numpy as np
import pytest
import torch
from scipy.stats import norm

import oracle


def _rand(seed, *shape, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale)


# ------------------------------------------------------------------ linear trio

@pytest.mark.parametrize("B,N,K,E", [(512, 128, 64, 8), (37, 3, 16, 11), (1, 5, 7, 2), (64, 16, 16, 1)])
def test_linear_fwd_is_batched_matvec(B, N, K, E):
    x, w = _rand(1, B, K), _rand(2, E, N, K, scale=0.05)
    sel = torch.randint(0, E, (B,), generator=torch.Generator().manual_seed(3))
    got = oracle.linear_fwd(x.numpy(), w.numpy(), sel.numpy())
    ref = torch.einsum("bnk,bk->bn", w[sel].double(), x.double())          # library routine
    np.testing.assert_allclose(got, ref.numpy(), rtol=1e-6, atol=1e-7)
    if E == 1:
        np.testing.assert_allclose(got, torch.nn.functional.linear(x, w[0]).numpy(), rtol=1e-5, atol=1e-6)


def test_linear_fwd_brute_force_and_special_cases():
    B, N, K, E = 6, 4, 5, 3
    x, w = _rand(4, B, K).numpy(), _rand(5, E, N, K).numpy()
    sel = np.array([2, 0, 1, 1, 2, 0])
    got = oracle.linear_fwd(x, w, sel)
    for b, o in itertools.product(range(B), range(N)):
        assert abs(got[b, o] - sum(float(w[sel[b], o, i]) * float(x[b, i]) for i in range(K))) < 1e-6
    # one-hot rows read out weight columns (catches a transposed weight)
    onehot = np.eye(K, dtype=np.float32)[[1, 3, 0, 4, 2, 1]]
    got = oracle.linear_fwd(onehot, w, sel)
    for b, col in enumerate([1, 3, 0, 4, 2, 1]):
        np.testing.assert_array_equal(got[b], w[sel[b], :, col])
    # row-permutation equivariance
    perm = np.array([3, 1, 5, 0, 2, 4])
    np.testing.assert_array_equal(oracle.linear_fwd(x[perm], w, sel[perm]), oracle.linear_fwd(x, w, sel)[perm])


@pytest.mark.parametrize("B,N,K,E", [(200, 24, 40, 6), (37, 3, 16, 11), (50, 16, 3, 11)])
def test_linear_backward_is_autograd_of_forward(B, N, K, E):
    """What the reference's own script does (test_moe_fused_linear_bwd.py:49-54)."""
    x = _rand(6, B, K).double().requires_grad_()
    w = _rand(7, E, N, K, scale=0.1).double().requires_grad_()
    dy = _rand(8, B, N)
    sel = torch.randint(0, E, (B,), generator=torch.Generator().manual_seed(9))
    sel[sel == E - 1] = 0                                                  # leave one expert empty
    torch.einsum("bnk,bk->bn", w[sel], x).backward(dy.double())
    dx = oracle.linear_bwd_input(dy.numpy(), w.detach().float().numpy(), sel.numpy())
    dw = oracle.linear_bwd_weight(dy.numpy(), x.detach().float().numpy(), sel.numpy(), E)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dw, w.grad.numpy(), rtol=1e-5, atol=1e-6)
    assert not dw[E - 1].any(), "an expert without rows gets exact zeros (backward_dw.py:110)"
    # sum over experts of dW equals the ungrouped dy^T x
    np.testing.assert_allclose(dw.sum(0), (dy.double().t() @ x.detach()).numpy(), rtol=1e-5, atol=1e-5)


def test_sel_from_m_sizes():
    np.testing.assert_array_equal(oracle.sel_from_m_sizes([2, 0, 3]), [0, 0, 2, 2, 2])


# ------------------------------------------------------------------ sort

@pytest.mark.parametrize("R,E", [(0, 4), (1, 1), (512, 8), (5000, 128), (333, 11), (4096, 1000)])
def test_expert_sort_is_stable_argsort(R, E):
    s = torch.randint(0, E, (R,), generator=torch.Generator().manual_seed(R + E))
    counts, sort_idx, inv = oracle.expert_counts_and_idx(s.numpy(), E)
    assert counts.dtype == sort_idx.dtype == inv.dtype == np.int32
    np.testing.assert_array_equal(counts, torch.bincount(s, minlength=E).numpy())
    np.testing.assert_array_equal(sort_idx, torch.argsort(s, stable=True).numpy())
    np.testing.assert_array_equal(sort_idx[inv], np.arange(R))
    np.testing.assert_array_equal(inv[sort_idx], np.arange(R))
    sorted_s = s.numpy()[sort_idx]
    assert (np.diff(sorted_s) >= 0).all()
    same = np.diff(sorted_s) == 0
    assert (np.diff(sort_idx)[same] > 0).all(), "ties keep their original order"
    assert counts.sum() == R
    np.testing.assert_array_equal(oracle.expert_counts(s.numpy(), E), counts)


def test_expert_sort_matches_the_compare_matrix_definition():
    """Literal evaluation of the reference's O(E*M) formulation (kernels/indexing.py:50-62)
    on a small input, in stock torch ops."""
    E = 5
    s = torch.tensor([3, 1, 3, 0, 1, 1, 4, 3, 0])
    compare = torch.arange(E)[:, None] == s[None, :]
    counts = compare.sum(1)
    ranks = compare.cumsum(1)[s, torch.arange(s.numel())]
    offsets = counts.cumsum(0) - counts
    idx = ranks + offsets[s] - 1
    inv_idx = torch.empty_like(idx)
    inv_idx[idx] = torch.arange(s.numel())
    c, sort_idx, inv_sort_idx = oracle.expert_counts_and_idx(s.numpy(), E)
    np.testing.assert_array_equal(c, counts.numpy())
    np.testing.assert_array_equal(sort_idx, inv_idx.numpy())       # returned 2nd, used as sort_idx
    np.testing.assert_array_equal(inv_sort_idx, idx.numpy())       # returned 3rd, used as inv_sort_idx


def test_expert_sort_rejects_out_of_range():
    with pytest.raises(ValueError):
        oracle.expert_counts_and_idx(np.array([0, 4]), 4)


# ------------------------------------------------------------------ routing

@pytest.mark.parametrize("T,E,k,renorm", [(256, 8, 2, False), (512, 128, 8, True), (33, 11, 3, True)])
def test_softmax_topk_is_library_softmax_topk(T, E, k, renorm):
    logits = _rand(T + E, T, E)
    w, idx = oracle.softmax_topk(logits.numpy(), k, renorm)
    p = torch.softmax(logits, dim=1, dtype=torch.float32)
    tw, ti = torch.topk(p, k, dim=-1)
    gap = (tw[:, :-1] - tw[:, 1:]).min()
    assert gap > 0, "fixture must be tie-free"
    if renorm:
        tw = tw / tw.sum(dim=-1, keepdim=True)
    np.testing.assert_array_equal(idx, ti.numpy())
    np.testing.assert_allclose(w, tw.numpy(), rtol=1e-6, atol=1e-9)
    assert (np.diff(w, axis=1) <= 0).all(), "descending"
    if renorm:
        np.testing.assert_allclose(w.sum(1), 1.0, rtol=1e-6)


def test_softmax_topk_tie_rule():
    w, idx = oracle.softmax_topk(np.array([[1.0, 3.0, 3.0, 0.5, 3.0, -1.0, 2.0, 2.0]], np.float32), 5, True)
    assert idx[0].tolist() == [1, 2, 4, 6, 7]
    assert w[0, 0] == w[0, 1] == w[0, 2] and w[0, 3] == w[0, 4]


def test_softmax_topk_matches_installed_hf_router():
    """Second, independent pin: transformers' Qwen3MoeTopKRouter does the same arithmetic."""
    mod = pytest.importorskip("transformers.models.qwen3_moe.modeling_qwen3_moe")
    if not hasattr(mod, "Qwen3MoeTopKRouter"):
        pytest.skip("installed transformers has no Qwen3MoeTopKRouter")
    from types import SimpleNamespace

    cfg = SimpleNamespace(num_experts_per_tok=4, num_experts=16, norm_topk_prob=True, hidden_size=32)
    router = mod.Qwen3MoeTopKRouter(cfg)
    with torch.no_grad():
        router.weight.copy_(_rand(1, 16, 32, scale=0.3))
    hidden = _rand(2, 50, 32)
    out = router(hidden)
    logits = torch.nn.functional.linear(hidden, router.weight)
    w, idx = oracle.softmax_topk(logits.detach().numpy(), 4, True)
    hf_w, hf_idx = out[-2], out[-1]
    np.testing.assert_array_equal(idx, hf_idx.numpy())
    np.testing.assert_allclose(w, hf_w.detach().float().numpy(), rtol=1e-5, atol=1e-7)


# ------------------------------------------------------------------ SiLU-mul

def test_silu_mul_bf16_rounding_chain_is_library_silu():
    e = _rand(1, 4096, scale=3.0).bfloat16()
    g = _rand(2, 4096, scale=3.0).bfloat16()
    got = oracle.from_bf16_bits(oracle.silu_mul_fwd_bf16(oracle.to_bf16_bits(e.float().numpy()),
                                                         oracle.to_bf16_bits(g.float().numpy())))
    ref = (torch.nn.functional.silu(e.float()).to(torch.bfloat16) * g).float().numpy()   # silu_mul.py:34-39
    mism = got != ref
    # libm expf vs torch's vectorised exp can differ by an ulp: at most one bf16 step, and rare
    assert mism.mean() < 2e-3
    np.testing.assert_allclose(got, ref, rtol=2 ** -7, atol=1e-30)


def test_silu_mul_backward_is_autograd_fp64():
    e, g, dh = (_rand(s, 2000, scale=2.0) for s in (3, 4, 5))
    e64, g64 = e.double().requires_grad_(), g.double().requires_grad_()
    (torch.nn.functional.silu(e64) * g64).backward(dh.double())
    h, de, dg = oracle.silu_mul_bwd_f32(dh.numpy(), e.numpy(), g.numpy())
    np.testing.assert_allclose(de, e64.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dg, g64.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(h, (torch.nn.functional.silu(e) * g).numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.silu_mul_fwd_f32(e.numpy(), g.numpy()), h, rtol=0, atol=0)
    # bf16 chain stays within bf16 resolution of the exact gradients
    bits = [oracle.to_bf16_bits(t.numpy()) for t in (dh, e, g)]
    eb, gb, dhb = (torch.from_numpy(oracle.from_bf16_bits(b)).double().requires_grad_() for b in (bits[1], bits[2], bits[0]))
    (torch.nn.functional.silu(eb) * gb).backward(dhb.detach())
    hb, deb, dgb = (oracle.from_bf16_bits(t) for t in oracle.silu_mul_bwd_bf16(*bits))
    np.testing.assert_allclose(deb, eb.grad.numpy(), rtol=2e-2, atol=1e-3)
    np.testing.assert_allclose(dgb, gb.grad.numpy(), rtol=2e-2, atol=1e-3)


# ------------------------------------------------------------------ bf16 helpers

def test_bf16_round_trip_matches_torch():
    x = torch.cat([_rand(1, 10000, scale=10.0), torch.tensor([0.0, -0.0, 1.0, 65504.0, 1e-40, 3.3895314e38])])
    bits = oracle.to_bf16_bits(x.numpy())
    np.testing.assert_array_equal(bits, x.bfloat16().view(torch.int16).numpy().view(np.uint16))
    np.testing.assert_array_equal(oracle.from_bf16_bits(bits), x.bfloat16().float().numpy())


# ------------------------------------------------------------------ NF4 (parity vs bitsandbytes unpinned)

def test_nf4_code_table_closed_form():
    """The table is bitsandbytes' hard-coded one; structurally it is the published construction:
    8 positive and 7 negative normal quantiles plus an exact zero, normalised to [-1, 1]."""
    code = oracle.nf4_code()
    assert code.dtype == np.float32 and code.shape == (16,)
    assert code[0] == -1.0 and code[7] == 0.0 and code[15] == 1.0 and (np.diff(code) > 0).all()
    offset = 0.9677083
    pos = norm.ppf(np.linspace(offset, 0.5, 9)[:-1])
    neg = -norm.ppf(np.linspace(offset, 0.5, 8)[:-1])
    closed = np.sort(np.concatenate([pos, [0.0], neg]))
    closed /= np.abs(closed).max()
    assert np.abs(closed - code).max() < 1.5e-7


def test_nf4_dequant_layout_and_arithmetic():
    """Nibble order and block indexing as the reference's kernel states them
    (forward_4bit.py:99-104): high nibble first, absmax per `blocksize` consecutive elements."""
    code = oracle.nf4_code()
    q = np.array([0x0F, 0x71, 0xA3, 0xFF], np.uint8)                      # 8 elements, blocksize 4
    absmax = np.array([2.0, 0.5], np.float32)
    got = oracle.nf4_dequant(q, absmax, 4)
    nibbles = [0x0, 0xF, 0x7, 0x1, 0xA, 0x3, 0xF, 0xF]
    ref = np.array([code[n] for n in nibbles], np.float32) * np.repeat(absmax, 4)
    np.testing.assert_array_equal(got, ref)
    # bf16 output = one round-to-nearest-even of the fp32 product
    got16 = oracle.nf4_dequant(q, absmax, 4, bf16=True)
    np.testing.assert_array_equal(got16, torch.from_numpy(ref).bfloat16().view(torch.int16).numpy().view(np.uint16))


def test_nf4_quant_round_trip_and_nearest():
    w = _rand(11, 64 * 40, scale=0.02).numpy()
    q, absmax = oracle.nf4_quant(w, 64)
    np.testing.assert_array_equal(absmax, np.abs(w.reshape(-1, 64)).max(1))
    deq = oracle.nf4_dequant(q, absmax, 64)
    q2, absmax2 = oracle.nf4_quant(deq, 64)
    np.testing.assert_array_equal(q2, q)                                   # quant(dequant(q)) == q
    # brute force: no other code entry is closer
    code = oracle.nf4_code().astype(np.float64)
    scaled = (w.reshape(-1, 64) * (np.float32(1.0) / absmax)[:, None]).reshape(-1).astype(np.float64)
    best = np.abs(scaled[:, None] - code[None, :]).argmin(1)
    nib = np.stack([q >> 4, q & 15], 1).reshape(-1)
    assert (nib == best).mean() > 0.9999                                   # differ only at fp32 midpoints
    assert np.abs(deq - w).max() <= 0.16 * absmax.max()


def test_dequant_blockwise_u8():
    code = np.linspace(-1, 1, 256).astype(np.float32)
    v = np.array([0, 255, 128, 7, 9, 200], np.uint8)
    absmax2 = np.array([2.0, 4.0], np.float32)
    got = oracle.dequant_blockwise_u8(v, code, absmax2, 4, 0.5)
    ref = (code[v] * np.array([2, 2, 2, 2, 4, 4], np.float32)) + np.float32(0.5)
    np.testing.assert_array_equal(got, ref)


# ------------------------------------------------------------------ compositions

def test_block_composition_matches_installed_hf_block():
    """The oracle's block (router -> sort -> experts -> combine) against transformers' eager
    Qwen3MoeSparseMoeBlock with the same weights: same math, different summation order."""
    mod = pytest.importorskip("transformers.models.qwen3_moe.modeling_qwen3_moe")
    from transformers import Qwen3MoeConfig

    cfg = Qwen3MoeConfig(hidden_size=16, moe_intermediate_size=12, num_experts=6, num_experts_per_tok=2,
                         norm_topk_prob=True, num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=2,
                         intermediate_size=24, vocab_size=32)
    try:
        blk = mod.Qwen3MoeSparseMoeBlock(cfg)
        gate_up = blk.experts.gate_up_proj            # (E, 2I, H)
        down = blk.experts.down_proj                  # (E, H, I)
        router_w = blk.gate.weight
    except AttributeError:
        pytest.skip("installed transformers lays the experts out differently")
    with torch.no_grad():
        for i, p in enumerate(blk.parameters()):
            p.copy_(_rand(20 + i, *p.shape, scale=0.2))
    hidden = _rand(3, 2, 9, 16)
    with torch.no_grad():
        out = blk(hidden)
    out = out[0] if isinstance(out, tuple) else out
    I = 12
    got, _ = oracle.moe_block_fwd(hidden.reshape(-1, 16).numpy(), router_w.detach().numpy(),
                                  gate_up[:, :I].detach().numpy(), gate_up[:, I:].detach().numpy(),
                                  down.detach().numpy(), 2, True)
    np.testing.assert_allclose(got, out.reshape(-1, 16).numpy(), rtol=1e-4, atol=1e-5)


def test_lora_composition_equals_merged_weight():
    B, N, K, E, r, s = 80, 12, 20, 4, 3, 0.7
    x, w = _rand(1, B, K).numpy(), _rand(2, E, N, K, scale=0.1).numpy()
    a, b = _rand(3, E, r, K, scale=0.1).numpy(), _rand(4, E, N, r, scale=0.1).numpy()
    sel = torch.randint(0, E, (B,), generator=torch.Generator().manual_seed(5)).numpy()
    merged = w + s * np.einsum("enr,erk->enk", b, a)
    np.testing.assert_allclose(oracle.lora_linear_fwd(x, w, a, b, s, sel), oracle.linear_fwd(x, merged, sel),
                               rtol=1e-4, atol=1e-6)


def test_lora_mlp_composition_matches_autograd_of_merged_weights():
    """oracle.lora_mlp_fwd_bwd (the expert MLP with LoRA on its three projections and all its
    gradients) against fp64 autograd of the same network written with merged weights
    P' = P + S B A (kernels/fast_lora.py:13-19): the forward formula is not retyped with LoRA
    terms, and no gradient formula is retyped at all."""
    B, H, M, E, r = 90, 20, 12, 4, 3
    Sg, Su, Sw = 0.7, 1.3, 0.5
    g = lambda i, *s, scale=0.2: _rand(100 + i, *s, scale=scale)
    x, dy = g(0, B, H, scale=1.0), g(1, B, H, scale=1.0)
    G, U, W = g(2, E, M, H), g(3, E, M, H), g(4, E, H, M)
    Ag, Bg, Au, Bu = g(5, E, r, H), g(6, E, M, r), g(7, E, r, H), g(8, E, M, r)
    Aw, Bw = g(9, E, r, M), g(10, E, H, r)
    sel = torch.randint(0, E, (B,), generator=torch.Generator().manual_seed(11))
    sel = torch.sort(sel).values
    got = oracle.lora_mlp_fwd_bwd(*(t.numpy() for t in (x, G, Ag, Bg)), Sg, *(t.numpy() for t in (U, Au, Bu)), Su,
                                  *(t.numpy() for t in (W, Aw, Bw)), Sw, sel.numpy(), dy.numpy())
    leaves = {n: t.double().requires_grad_() for n, t in dict(x=x, Ag=Ag, Bg=Bg, Au=Au, Bu=Bu, Aw=Aw, Bw=Bw).items()}
    merged = lambda P, A, Bm, S: P.double() + S * torch.einsum("eor,eri->eoi", Bm, A)
    mv = lambda Wm, v: torch.einsum("boi,bi->bo", Wm[sel], v)
    e = mv(merged(G, leaves["Ag"], leaves["Bg"], Sg), leaves["x"])
    gg = mv(merged(U, leaves["Au"], leaves["Bu"], Su), leaves["x"])
    h = torch.nn.functional.silu(e) * gg
    y = mv(merged(W, leaves["Aw"], leaves["Bw"], Sw), h)
    y.backward(dy.double())
    np.testing.assert_allclose(got["y"], y.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(got["h"], h.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(got["dx"], leaves["x"].grad.numpy(), rtol=1e-4, atol=1e-5)
    for n in ("Ag", "Bg", "Au", "Bu", "Aw", "Bw"):
        np.testing.assert_allclose(got["d" + n], leaves[n].grad.numpy(), rtol=1e-4, atol=1e-5, err_msg=n)
