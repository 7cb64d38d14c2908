"""Forward products fused with their neighbours (gathered rows; gate/up/SiLU in one kernel)
against the oracle, and bit for bit against the separate kernels they stand in for."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, m_sizes_uniform, randn, to_np32, unit_scale_atol

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_4bit  # noqa: E402
from qwen3_moe_fused.grouped_gemm.fused import (grouped_gemm_forward_4bit_gathered,  # noqa: E402
                                                grouped_gemm_forward_gathered, grouped_glu_forward,
                                                grouped_glu_forward_4bit)
from qwen3_moe_fused.kernels.silu_mul import silu_mul_forward  # noqa: E402
from qwen3_moe_fused.quantize.nf4 import Nf4QuantState, nf4_code  # noqa: E402

DEV = "cuda"


def _routing(T, E, k, seed):
    """k distinct experts per token; returns (m_sizes int32, sort_idx int32) of the stable sort."""
    g = gen(seed)
    sel = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).reshape(-1)
    counts, sort_idx, _ = oracle.expert_counts_and_idx(sel.numpy(), E)
    return torch.from_numpy(counts.astype(np.int32)), torch.from_numpy(sort_idx.astype(np.int32)), sel.numpy()


def _quantised(E, N, K, blocksize, seed):
    w = randn((E, N, K), gen(seed), 0.05)
    q, absmax = oracle.nf4_quant(w.numpy(), blocksize)
    w_deq = oracle.round_bf16(oracle.nf4_dequant(q, absmax, blocksize)).reshape(E, N, K)
    state = Nf4QuantState(absmax=torch.from_numpy(absmax).to(DEV), shape=(E, N, K), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=torch.bfloat16)
    return torch.from_numpy(q).view(-1, 1).to(DEV), state, w_deq


def _nf4_atol(ref, K, *blocksizes, rows=None, experts=None):
    """The decode-size kernels that scale partial sums (see unit_scale_atol) take K % 128 == 0 with blocks of at
    least 64 weights, and, with at most two rows per expert (one up to K = 1024), 256 < K <= 2048 with any block size that
    divides K:
    two percent of the output scale there, one percent of unit scale elsewhere."""
    streaming = K % 128 == 0 and min(blocksizes) >= 64
    matrix_vector = (rows is not None and rows <= (2 if K > 1024 else 1) * experts and 256 < K <= 2048
                     and all(K % b == 0 for b in blocksizes))
    if streaming or matrix_vector:
        return unit_scale_atol(ref, 2e-2)
    return 1e-2


def _oracle_glu(xg, wg, wu, sel_sorted):
    """e, g rounded to bf16, then the SiLU-mul with the reference's rounding chain."""
    e = oracle.round_bf16(oracle.linear_fwd(xg, wg, sel_sorted))
    g = oracle.round_bf16(oracle.linear_fwd(xg, wu, sel_sorted))
    h = oracle.from_bf16_bits(oracle.silu_mul_fwd_bf16(oracle.to_bf16_bits(e), oracle.to_bf16_bits(g)))
    return h, e, g


# (tokens, experts, selected, N, K): tile-sized, ragged, decode-sized, one expert, many rows per expert
GATHER_CASES = [(512, 16, 4, 192, 256), (300, 5, 2, 72, 136), (8, 32, 4, 256, 128), (700, 1, 1, 64, 64),
                (2048, 4, 2, 392, 192), (64, 128, 8, 768, 2048)]


@pytest.mark.parametrize("T,E,k,N,K", GATHER_CASES)
def test_gathered_forward_matches_oracle_and_explicit_gather(T, E, k, N, K):
    ms, sort_idx, sel = _routing(T, E, k, T + N)
    x = randn((T, K), gen(T), 1.0, torch.bfloat16)
    w = randn((E, N, K), gen(N), 0.05, torch.bfloat16)
    rows = sort_idx.numpy() // k
    y = grouped_gemm_forward_gathered(x.to(DEV), sort_idx.to(DEV), k, w.to(DEV), ms.to(DEV))
    check_close(y, oracle.linear_fwd(to_np32(x)[rows], to_np32(w), np.sort(sel, kind="stable")), what="gathered fwd")
    y2 = grouped_gemm_forward(x[rows.astype(np.int64)].contiguous().to(DEV), w.to(DEV), ms.to(DEV))
    assert torch.equal(y, y2), "gather folded into the operand load must not change a bit"


@pytest.mark.parametrize("T,E,k,N,K,blocksize", [(512, 16, 4, 192, 256, 64), (40, 20, 2, 136, 128, 16),
                                                 (1024, 4, 2, 264, 192, 32), (16, 128, 8, 768, 2048, 64),
                                                 (24, 6, 2, 136, 384, 128),    # streaming kernel, ragged edges
                                                 (9, 12, 2, 96, 1280, 128)])   # matrix-vector kernel, lanes past K
def test_gathered_nf4_forward(T, E, k, N, K, blocksize):
    ms, sort_idx, sel = _routing(T, E, k, T + N)
    x = randn((T, K), gen(T), 1.0, torch.bfloat16)
    packed, state, w_deq = _quantised(E, N, K, blocksize, N + K)
    rows = sort_idx.numpy() // k
    y = grouped_gemm_forward_4bit_gathered(x.to(DEV), sort_idx.to(DEV), k, packed, state, ms.to(DEV))
    ref = oracle.linear_fwd(to_np32(x)[rows], w_deq, np.sort(sel, kind="stable"))
    check_close(y, ref, atol=_nf4_atol(ref, K, blocksize, rows=T * k, experts=E), what="gathered nf4 fwd")
    y2 = grouped_gemm_forward_4bit(x[rows.astype(np.int64)].contiguous().to(DEV), packed, state, ms.to(DEV))
    assert torch.equal(y, y2)


@pytest.mark.parametrize("gathered", [False, True])
@pytest.mark.parametrize("T,E,k,N,K", GATHER_CASES)
def test_glu_forward(T, E, k, N, K, gathered):
    ms, sort_idx, sel = _routing(T, E, k, T + N + 1)
    x = randn((T, K), gen(T), 1.0, torch.bfloat16)
    wg = randn((E, N, K), gen(N), 0.05, torch.bfloat16)
    wu = randn((E, N, K), gen(N + 1), 0.05, torch.bfloat16)
    rows = (sort_idx.numpy() // k).astype(np.int64)
    xg = x[rows].contiguous()
    if gathered:
        h, e, g = grouped_glu_forward(x.to(DEV), wg.to(DEV), wu.to(DEV), ms.to(DEV), sort_idx.to(DEV), k,
                                      return_products=True)
    else:
        h, e, g = grouped_glu_forward(xg.to(DEV), wg.to(DEV), wu.to(DEV), ms.to(DEV), return_products=True)
    h_ref, e_ref, g_ref = _oracle_glu(to_np32(xg), to_np32(wg), to_np32(wu), np.sort(sel, kind="stable"))
    check_close(e, e_ref, what="gate product")
    check_close(g, g_ref, what="up product")
    # the oracle's e and g may differ from the kernel's by a bf16 ulp, and silu(e) * g carries that on
    check_close(h, h_ref, 2e-2, 2e-2, what="glu")
    # bit for bit: the separate kernels
    e2 = grouped_gemm_forward(xg.to(DEV), wg.to(DEV), ms.to(DEV))
    g2 = grouped_gemm_forward(xg.to(DEV), wu.to(DEV), ms.to(DEV))
    assert torch.equal(e, e2) and torch.equal(g, g2)
    assert torch.equal(h, silu_mul_forward(e2, g2))
    # without the products
    h3 = grouped_glu_forward(xg.to(DEV), wg.to(DEV), wu.to(DEV), ms.to(DEV))
    assert torch.equal(h, h3)


@pytest.mark.parametrize("T,E,k,N,K,bs_g,bs_u", [(512, 16, 4, 192, 256, 64, 64), (40, 20, 2, 136, 128, 16, 32),
                                                 (1024, 4, 2, 264, 192, 32, 8), (16, 128, 8, 768, 2048, 64, 64),
                                                 (256, 128, 8, 768, 2048, 64, 64),
                                                 (24, 6, 2, 136, 384, 64, 128),    # streaming kernel, ragged edges
                                                 (160, 6, 2, 136, 384, 64, 128),   # the same with 64-row tiles
                                                 (640, 128, 8, 768, 2048, 64, 64),
                                                 (9, 12, 2, 96, 1280, 128, 256),   # matrix-vector kernel
                                                 (3, 5, 3, 32, 2048, 2048, 8),
                                                 (4, 9, 2, 64, 768, 64, 256)])    # 32 lanes to a column
def test_glu_nf4_forward(T, E, k, N, K, bs_g, bs_u):
    ms, sort_idx, sel = _routing(T, E, k, T + N + 2)
    x = randn((T, K), gen(T), 1.0, torch.bfloat16)
    pg, sg, wg_deq = _quantised(E, N, K, bs_g, N + K)
    pu, su, wu_deq = _quantised(E, N, K, bs_u, N + K + 1)
    rows = (sort_idx.numpy() // k).astype(np.int64)
    xg = x[rows].contiguous()
    h, e, g = grouped_glu_forward_4bit(x.to(DEV), pg, sg, pu, su, ms.to(DEV), sort_idx.to(DEV), k,
                                       return_products=True)
    h_ref, e_ref, g_ref = _oracle_glu(to_np32(xg), wg_deq, wu_deq, np.sort(sel, kind="stable"))
    check_close(e, e_ref, atol=_nf4_atol(e_ref, K, bs_g, bs_u, rows=T * k, experts=E), what="gate product")
    check_close(g, g_ref, atol=_nf4_atol(g_ref, K, bs_g, bs_u, rows=T * k, experts=E), what="up product")
    # the oracle's e and g differ from the kernel's by a few bf16 ulps, and silu(e) * g carries that on, times
    # the size of the other factor: h is checked against the oracle's SiLU-mul of the kernel's own e and g
    # (one ulp), and against the oracle's h by its largest error relative to the largest value
    h_own = oracle.from_bf16_bits(oracle.silu_mul_fwd_bf16(oracle.to_bf16_bits(to_np32(e)), oracle.to_bf16_bits(to_np32(g))))
    check_close(h, h_own, 2e-2, 2e-2, what="glu of the kernel's own products")
    assert np.abs(to_np32(h) - h_ref).max() <= 1e-2 * np.abs(h_ref).max(), "glu against the oracle's"
    e2 = grouped_gemm_forward_4bit(xg.to(DEV), pg, sg, ms.to(DEV))
    g2 = grouped_gemm_forward_4bit(xg.to(DEV), pu, su, ms.to(DEV))
    assert torch.equal(e, e2) and torch.equal(g, g2)
    assert torch.equal(h, silu_mul_forward(e2, g2))
    h3 = grouped_glu_forward_4bit(xg.to(DEV), pg, sg, pu, su, ms.to(DEV))
    assert torch.equal(h, h3)


@pytest.mark.parametrize("T", [256, 16])   # the streaming kernel; the matrix-vector kernel
def test_decode_size_nf4_product_is_as_accurate_as_the_reference_rounding(T):
    # The decode-size kernels compute sum over blocks of absmax * (x . bf16(code)), the reference x . bf16(code * absmax).
    # Against the product with the unrounded weights code * absmax, in float64, neither is better: same rms
    # error, same largest error, within the scatter of such figures.
    E, k, N, K, blocksize = 128, 8, 768, 2048, 64
    ms, sort_idx, sel = _routing(T, E, k, 11)
    x = randn((T, K), gen(3), 1.0, torch.bfloat16)
    w = randn((E, N, K), gen(4), 0.05)
    q, absmax = oracle.nf4_quant(w.numpy(), blocksize)
    w_exact = oracle.nf4_dequant(q, absmax, blocksize).reshape(E, N, K)
    state = Nf4QuantState(absmax=torch.from_numpy(absmax).to(DEV), shape=(E, N, K), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=torch.bfloat16)
    rows = (sort_idx.numpy() // k).astype(np.int64)
    xg = to_np32(x)[rows]
    sel_sorted = np.sort(sel, kind="stable")
    y = to_np32(grouped_gemm_forward_4bit(x[rows].contiguous().to(DEV), torch.from_numpy(q).view(-1, 1).to(DEV), state,
                                          ms.to(DEV))).astype(np.float64)
    exact = oracle.linear_fwd(xg, w_exact, sel_sorted).astype(np.float64)
    reference = oracle.round_bf16(oracle.linear_fwd(xg, oracle.round_bf16(w_exact), sel_sorted)).astype(np.float64)
    err_k, err_r = y - exact, reference - exact
    rms_k, rms_r = np.sqrt((err_k ** 2).mean()), np.sqrt((err_r ** 2).mean())
    assert rms_k <= 1.1 * rms_r, (rms_k, rms_r)
    assert np.abs(err_k).max() <= 1.5 * np.abs(err_r).max(), (np.abs(err_k).max(), np.abs(err_r).max())


def test_unsupported_requests_fall_back_to_the_separate_kernels():
    # fp32 and a width that is not a multiple of 8: no fused kernel, same results
    T, E, k, N, K = 64, 3, 2, 12, 20
    ms, sort_idx, sel = _routing(T, E, k, 5)
    x = randn((T, K), gen(1), 1.0)
    wg, wu = randn((E, N, K), gen(2), 0.1), randn((E, N, K), gen(3), 0.1)
    rows = (sort_idx.numpy() // k).astype(np.int64)
    y = grouped_gemm_forward_gathered(x.to(DEV), sort_idx.to(DEV), k, wg.to(DEV), ms.to(DEV))
    ref = oracle.linear_fwd(to_np32(x)[rows], to_np32(wg), np.sort(sel, kind="stable"))
    check_close(y, ref, 1e-4, 1e-4, "fp32 gathered fwd")
    h = grouped_glu_forward(x.to(DEV), wg.to(DEV), wu.to(DEV), ms.to(DEV), sort_idx.to(DEV), k)
    e = oracle.linear_fwd(to_np32(x)[rows], to_np32(wg), np.sort(sel, kind="stable"))
    g = oracle.linear_fwd(to_np32(x)[rows], to_np32(wu), np.sort(sel, kind="stable"))
    check_close(h, oracle.silu_mul_fwd_f32(e, g), 1e-4, 1e-4, "fp32 glu")


def _random_fused_case(seed):
    """Arbitrary per-expert row counts (empty experts, tile-edge sizes, one hot expert) and an
    arbitrary row index (any source row may appear any number of times)."""
    rng = np.random.default_rng(1000 + seed)
    E = int(rng.choice([1, 2, 5, 9, 24]))
    N = int(rng.choice([8, 40, 96, 104, 192, 200, 328]))
    K = int(rng.choice([8, 24, 64, 72, 128, 264]))
    kind = seed % 4
    if kind == 0:
        m = rng.integers(0, 12, size=E)
    elif kind == 1:
        m = rng.integers(0, 400, size=E)
    elif kind == 2:
        m = rng.integers(0, 20, size=E)
        m[int(rng.integers(0, E))] += int(rng.integers(500, 1500))
    else:
        m = rng.choice([0, 1, 31, 32, 33, 319, 320, 321, 640, 641], size=E)
    if m.sum() == 0:
        m[0] = 3
    R = int(m.sum())
    div = int(rng.choice([1, 2, 8]))
    T = max(1, R // div + int(rng.integers(0, 5)))
    row_idx = rng.integers(0, T * div, size=R).astype(np.int32)
    return E, N, K, torch.from_numpy(m.astype(np.int32)), T, div, torch.from_numpy(row_idx)


@pytest.mark.parametrize("seed", range(16))
def test_random_shapes_gathered_and_glu(seed):
    E, N, K, ms, T, div, row_idx = _random_fused_case(seed)
    R = int(ms.sum())
    what = f"seed {seed}: E={E} N={N} K={K} T={T} div={div} m_sizes={ms.tolist()}"
    x = randn((T, K), gen(seed), 1.0, torch.bfloat16)
    wg = randn((E, N, K), gen(seed + 1), 0.1, torch.bfloat16)
    wu = randn((E, N, K), gen(seed + 2), 0.1, torch.bfloat16)
    rows = (row_idx.numpy() // div).astype(np.int64)
    xg = x[rows].contiguous()
    sel = oracle.sel_from_m_sizes(ms.numpy())
    y = grouped_gemm_forward_gathered(x.to(DEV), row_idx.to(DEV), div, wg.to(DEV), ms.to(DEV))
    check_close(y, oracle.linear_fwd(to_np32(xg), to_np32(wg), sel), what=what + " gathered")
    assert torch.equal(y, grouped_gemm_forward(xg.to(DEV), wg.to(DEV), ms.to(DEV))), what
    h, e, g = grouped_glu_forward(x.to(DEV), wg.to(DEV), wu.to(DEV), ms.to(DEV), row_idx.to(DEV), div,
                                  return_products=True)
    assert torch.equal(e, y), what
    g2 = grouped_gemm_forward(xg.to(DEV), wu.to(DEV), ms.to(DEV))
    assert torch.equal(g, g2), what
    assert torch.equal(h, silu_mul_forward(y, g2)), what
    h_ref, _, _ = _oracle_glu(to_np32(xg), to_np32(wg), to_np32(wu), sel)
    check_close(h, h_ref, 2e-2, 2e-2, what=what + " glu")


from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed  # noqa: E402
from qwen3_moe_fused.grouped_gemm.fused import grouped_gemm_forward_transposed_dual  # noqa: E402


# dx (R, N) = dy1 (R, K) @ w1[e] + dy2 (R, K) @ w2[e], w (E, K, N)
@pytest.mark.parametrize("R,N,K,E", [(2048, 2048, 768, 8), (700, 200, 64, 5), (300, 72, 128, 3), (33, 8, 192, 40),
                                     (5000, 392, 64, 2), (1000, 1024, 128, 8),   # 192 x 256 tiles
                                     (64, 24, 72, 4)])   # the last: K % 64 != 0, two plain products
def test_two_term_input_gradient(R, N, K, E):
    g = gen(R + N)
    dy1, dy2 = randn((R, K), g, 1.0, torch.bfloat16), randn((R, K), g, 1.0, torch.bfloat16)
    w1, w2 = randn((E, K, N), g, 0.05, torch.bfloat16), randn((E, K, N), g, 0.05, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    dx = grouped_gemm_forward_transposed_dual(dy1.to(DEV), w1.to(DEV), dy2.to(DEV), w2.to(DEV), ms.to(DEV))
    ref = (oracle.linear_bwd_input(to_np32(dy1), to_np32(w1), sel).astype(np.float64)
           + oracle.linear_bwd_input(to_np32(dy2), to_np32(w2), sel))
    check_close(dx, ref, what="two-term dx vs oracle")
    # closed form: one product over the concatenated reduction
    dx_cat = grouped_gemm_forward_transposed(torch.cat([dy1, dy2], 1).contiguous().to(DEV),
                                             torch.cat([w1, w2], 1).contiguous().to(DEV), ms.to(DEV))
    if K % 64 == 0:
        assert torch.equal(dx, dx_cat), "the same reduction in the same order"
    else:
        check_close(dx, to_np32(dx_cat), what="two-term dx vs concatenated product")


from qwen3_moe_fused.grouped_gemm.fused import grouped_gemm_forward_transposed_silu_bwd  # noqa: E402
from qwen3_moe_fused.kernels.silu_mul import silu_mul_backward  # noqa: E402


# (de, dg[, h]) = silu_mul_backward(dy (R, K) @ w[e] (K, N), e, g): the product's epilogue against the two kernels, bit
# for bit (the product is rounded to bf16 before it meets e and g, as when it is stored), and against the oracle.
# Shapes: the down projection's (several tiles per expert, experts without rows), a width that leaves the last
# column tile partly empty, one reduction step, more experts than rows; the last two have no pipelined kernel
# (N % 8 != 0; fp32) and run as two launches.
@pytest.mark.parametrize("R,N,K,E,dtype", [(3000, 768, 2048, 8, torch.bfloat16), (700, 200, 64, 5, torch.bfloat16),
                                           (33, 8, 192, 40, torch.bfloat16), (5000, 392, 128, 2, torch.bfloat16),
                                           (9000, 768, 256, 4, torch.bfloat16),   # 256 x 256 tiles
                                           (64, 20, 72, 4, torch.bfloat16), (50, 24, 64, 3, torch.float32)])
def test_input_gradient_with_silu_mul_backward_in_the_epilogue(R, N, K, E, dtype):
    gn = gen(R + N)
    dy = randn((R, K), gn, 1.0, dtype).to(DEV)
    w = randn((E, K, N), gn, 0.05, dtype).to(DEV)
    e, g = randn((R, N), gn, 2.0, dtype).to(DEV), randn((R, N), gn, 1.0, dtype).to(DEV)
    ms = m_sizes_uniform(R, E, gn)
    if E >= 4:
        ms[1] += ms[2]
        ms[2] = 0                                # an expert without rows
    msd = ms.to(DEV)
    dh = grouped_gemm_forward_transposed(dy, w, msd)
    de_ref, dg_ref = silu_mul_backward(dh, e, g)
    de, dg, h = grouped_gemm_forward_transposed_silu_bwd(dy, w, e, g, msd, return_h=True)
    assert torch.equal(de, de_ref) and torch.equal(dg, dg_ref), "the same bits as product, then silu_mul_backward"
    assert torch.equal(h, silu_mul_forward(e, g))
    de2, dg2 = grouped_gemm_forward_transposed_silu_bwd(dy, w, e, g, msd)
    assert torch.equal(de2, de_ref) and torch.equal(dg2, dg_ref)
    if dtype == torch.bfloat16:
        sel = oracle.sel_from_m_sizes(ms.numpy())
        dh_o = oracle.round_bf16(oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel))
        _, de_o, dg_o = oracle.silu_mul_bwd_f32(dh_o, to_np32(e), to_np32(g))
        check_close(de, de_o, 3e-2, 3e-2 * float(np.abs(de_o).max()), "de vs oracle")
        check_close(dg, dg_o, 3e-2, 3e-2 * float(np.abs(dg_o).max()), "dg vs oracle")


def test_input_gradient_with_silu_mul_backward_in_place():
    """de may be e and dg may be g: every piece is read before it is written, by the lane that writes it."""
    from qwen3_moe_fused import _lib
    R, N, K, E = 1500, 392, 256, 6
    gn = gen(7)
    dy = randn((R, K), gn, 1.0, torch.bfloat16).to(DEV)
    w = randn((E, K, N), gn, 0.05, torch.bfloat16).to(DEV)
    e, g = randn((R, N), gn, 2.0, torch.bfloat16).to(DEV), randn((R, N), gn, 1.0, torch.bfloat16).to(DEV)
    ms = m_sizes_uniform(R, E, gn).to(DEV)
    de_ref, dg_ref, h_ref = grouped_gemm_forward_transposed_silu_bwd(dy, w, e, g, ms, return_h=True)
    e2, g2, h2 = e.clone(), g.clone(), torch.empty_like(e)
    rc = _lib.lib().mfl_gemm_dx_silu_bwd(_lib.ptr(dy), _lib.ptr(w), _lib.ptr(e2), _lib.ptr(g2), _lib.ptr(ms),
                                         _lib.itype_code(ms.dtype), _lib.ptr(e2), _lib.ptr(g2), _lib.ptr(h2), R, N, K, E,
                                         _lib.dtype_code(torch.bfloat16), _lib.stream())
    _lib.check(rc, "mfl_gemm_dx_silu_bwd")
    assert torch.equal(e2, de_ref) and torch.equal(g2, dg_ref) and torch.equal(h2, h_ref)


from qwen3_moe_fused.grouped_gemm.fused import (grouped_gemm_forward_lora,  # noqa: E402
                                                grouped_gemm_forward_transposed_lora)

# R, N, K, E, rank.  The rank-r term of a LoRA adapter in the reduction of the base product
# (qwen3_moe_fused/lora.py:134): y = x w^T + xt wt^T.
LORA_CASES = [(4096, 768, 2048, 16, 16),     # the 320 x 192 tiles of the expert shapes
              (9000, 512, 256, 4, 32),       # more than 512 rows per expert: 256 x 256 tiles
              (700, 200, 64, 5, 8),
              (300, 72, 128, 3, 24),         # rank not a multiple of 16
              (600, 136, 192, 6, 72),        # rank beyond one reduction step
              (33, 8, 192, 40, 16),          # a row or none per expert: the flat decode tiles
              (500, 40, 256, 3, 16),         # thin output: 128 x 64 tiles
              (64, 24, 72, 4, 16)]           # K % 64 != 0: a partial last step before the thin term


@pytest.mark.parametrize("R,N,K,E,r", LORA_CASES)
def test_forward_with_lora_term(R, N, K, E, r):
    g = gen(R + N + r)
    x, xt = randn((R, K), g, 1.0, torch.bfloat16), randn((R, r), g, 1.0, torch.bfloat16)
    w, wt = randn((E, N, K), g, 0.05, torch.bfloat16), randn((E, N, r), g, 0.2, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    y = grouped_gemm_forward_lora(x.to(DEV), w.to(DEV), xt.to(DEV), wt.to(DEV), ms.to(DEV))
    ref = (oracle.linear_fwd(to_np32(x), to_np32(w), sel).astype(np.float64)
           + oracle.linear_fwd(to_np32(xt), to_np32(wt), sel))
    check_close(y, ref, what="forward with a rank-r term vs oracle")
    # closed form: one product over the concatenated reduction
    y_cat = grouped_gemm_forward(torch.cat([x, xt], 1).contiguous().to(DEV), torch.cat([w, wt], 2).contiguous().to(DEV),
                                 ms.to(DEV))
    if K % 64 == 0:
        assert torch.equal(y, y_cat), "the same reduction in the same order"
    else:
        check_close(y, to_np32(y_cat), what="forward with a rank-r term vs concatenated product")


@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("R,N,K,E,r", LORA_CASES)
def test_input_gradient_with_lora_term(R, N, K, E, r, dual):
    # dx (R, N) = dy (R, K) @ w[e] (+ dy2 @ w2[e]) + xt (R, r) @ wt[e],  w (E, K, N), wt (E, r, N)
    g = gen(R + N + r + 1)
    dy, dy2 = randn((R, K), g, 1.0, torch.bfloat16), randn((R, K), g, 1.0, torch.bfloat16)
    xt = randn((R, r), g, 1.0, torch.bfloat16)
    w, w2 = randn((E, K, N), g, 0.05, torch.bfloat16), randn((E, K, N), g, 0.05, torch.bfloat16)
    wt = randn((E, r, N), g, 0.2, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    kw = dict(dy2=dy2.to(DEV), w2=w2.to(DEV)) if dual else {}
    dx = grouped_gemm_forward_transposed_lora(dy.to(DEV), w.to(DEV), xt.to(DEV), wt.to(DEV), ms.to(DEV), **kw)
    ref = (oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel).astype(np.float64)
           + oracle.linear_bwd_input(to_np32(xt), to_np32(wt), sel))
    if dual:
        ref = ref + oracle.linear_bwd_input(to_np32(dy2), to_np32(w2), sel)
    check_close(dx, ref, what="input gradient with a rank-r term vs oracle")
    terms_a = [dy] + ([dy2] if dual else []) + [xt]
    terms_w = [w] + ([w2] if dual else []) + [wt]
    dx_cat = grouped_gemm_forward_transposed(torch.cat(terms_a, 1).contiguous().to(DEV),
                                             torch.cat(terms_w, 1).contiguous().to(DEV), ms.to(DEV))
    if K % 64 == 0:
        assert torch.equal(dx, dx_cat), "the same reduction in the same order"
    else:
        check_close(dx, to_np32(dx_cat), what="input gradient with a rank-r term vs concatenated product")


def test_lora_term_of_other_element_types_runs_as_two_products():
    g = gen(77)
    R, N, K, E, r = 90, 12, 20, 3, 4                     # fp32, odd sizes: no fused kernel
    x, xt = randn((R, K), g), randn((R, r), g)
    w, wt = randn((E, N, K), g, 0.1), randn((E, N, r), g, 0.1)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    y = grouped_gemm_forward_lora(x.to(DEV), w.to(DEV), xt.to(DEV), wt.to(DEV), ms.to(DEV))
    ref = oracle.linear_fwd(to_np32(x), to_np32(w), sel).astype(np.float64) + oracle.linear_fwd(to_np32(xt), to_np32(wt), sel)
    check_close(y, ref, rtol=1e-4, atol=1e-4, what="fp32 forward with a rank-r term")
    dy = randn((R, N), g)
    wa = randn((E, r, K), g, 0.1)
    dx = grouped_gemm_forward_transposed_lora(dy.to(DEV), w.to(DEV), xt.to(DEV), wa.to(DEV), ms.to(DEV))
    ref = (oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel).astype(np.float64)
           + oracle.linear_bwd_input(to_np32(xt), to_np32(wa), sel))
    check_close(dx, ref, rtol=1e-4, atol=1e-4, what="fp32 input gradient with a rank-r term")


@pytest.mark.parametrize("seed", range(16))
def test_lora_term_random_shapes(seed):
    g = gen(4000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))  # noqa: E731
    E, R = ri(1, 48), ri(1, 3000)
    N, K, r = 8 * ri(1, 100), 8 * ri(1, 64), 8 * ri(1, 12)
    x, xt = randn((R, K), g, 1.0, torch.bfloat16), randn((R, r), g, 1.0, torch.bfloat16)
    w, wt = randn((E, N, K), g, 0.05, torch.bfloat16), randn((E, N, r), g, 0.2, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    print(f"lora term seed {seed}: E={E} R={R} N={N} K={K} r={r}", flush=True)
    y = grouped_gemm_forward_lora(x.to(DEV), w.to(DEV), xt.to(DEV), wt.to(DEV), ms.to(DEV))
    ref = (oracle.linear_fwd(to_np32(x), to_np32(w), sel).astype(np.float64)
           + oracle.linear_fwd(to_np32(xt), to_np32(wt), sel))
    check_close(y, ref, what="forward with a rank-r term vs oracle")
    # the input gradient of the same layer: dx (R, K) = dy (R, N) @ w[e] + tt (R, r) @ a[e], a (E, r, K)
    dy, tt = randn((R, N), g, 1.0, torch.bfloat16), randn((R, r), g, 1.0, torch.bfloat16)
    a = randn((E, r, K), g, 0.2, torch.bfloat16)
    dx = grouped_gemm_forward_transposed_lora(dy.to(DEV), w.to(DEV), tt.to(DEV), a.to(DEV), ms.to(DEV))
    ref = (oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel).astype(np.float64)
           + oracle.linear_bwd_input(to_np32(tt), to_np32(a), sel))
    check_close(dx, ref, what="input gradient with a rank-r term vs oracle")


from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_transposed_4bit  # noqa: E402
from qwen3_moe_fused.grouped_gemm.fused import (grouped_gemm_forward_4bit_lora,  # noqa: E402
                                                grouped_gemm_forward_transposed_4bit_lora)
from qwen3_moe_fused.quantize.nf4 import quantize_nf4  # noqa: E402


# R, N, K, E, rank, blocksize: the rank-r term in the reduction of a product over packed NF4 weights
@pytest.mark.parametrize("R,N,K,E,r,bs", [(4096, 768, 2048, 16, 16, 64), (9000, 512, 256, 4, 32, 64),
                                          (700, 224, 64, 5, 8, 16), (600, 160, 192, 6, 72, 32),
                                          (300, 72, 128, 3, 24, 64),      # dx: N % 32 != 0 -> two products
                                          (40, 64, 128, 20, 16, 64)])     # a row or two per expert
def test_nf4_products_with_lora_term(R, N, K, E, r, bs):
    g = gen(R + N + r + 7)
    w = randn((E, N, K), g, 0.05, torch.bfloat16).to(DEV)
    packed, state = quantize_nf4(w, bs)
    x, xt = randn((R, K), g, 1.0, torch.bfloat16).to(DEV), randn((R, r), g, 1.0, torch.bfloat16).to(DEV)
    wt = randn((E, N, r), g, 0.2, torch.bfloat16).to(DEV)
    ms = m_sizes_uniform(R, E, g).to(DEV)
    # forward: against the fused NF4 product followed by the accumulated thin product (two roundings instead of
    # one: a bf16 ulp of the sum apart at most), and against the oracle on the dequantised weights
    y = grouped_gemm_forward_4bit_lora(x, packed, state, xt, wt, ms)
    y2 = grouped_gemm_forward_4bit(x, packed, state, ms)
    grouped_gemm_forward(xt, wt, ms, out=y2, accumulate=True)
    sel = oracle.sel_from_m_sizes(ms.cpu().numpy())
    from qwen3_moe_fused.quantize.nf4 import dequantize_nf4
    wd = to_np32(dequantize_nf4(packed, state, torch.bfloat16))
    ref = oracle.linear_fwd(to_np32(x), wd, sel).astype(np.float64) + oracle.linear_fwd(to_np32(xt), to_np32(wt), sel)
    check_close(y, ref, what="NF4 forward with a rank-r term vs oracle")
    # (two bf16 roundings against one: up to two ulps of the output apart)
    check_close(y, to_np32(y2), atol=unit_scale_atol(to_np32(y2), 2e-2), what="NF4 forward with a rank-r term vs two products")
    # input gradient of the same layer: dx (R, K) = dy (R, N) @ W[e] + tt (R, r) @ a[e]
    dy, tt = randn((R, N), g, 1.0, torch.bfloat16).to(DEV), randn((R, r), g, 1.0, torch.bfloat16).to(DEV)
    a = randn((E, r, K), g, 0.2, torch.bfloat16).to(DEV)
    dx = grouped_gemm_forward_transposed_4bit_lora(dy, packed, state, tt, a, ms)
    ref = (oracle.linear_bwd_input(to_np32(dy), wd, sel).astype(np.float64)
           + oracle.linear_bwd_input(to_np32(tt), to_np32(a), sel))
    check_close(dx, ref, what="NF4 input gradient with a rank-r term vs oracle")
    dx2 = grouped_gemm_forward_transposed_4bit(dy, packed, state, ms)
    grouped_gemm_forward_transposed(tt, a, ms, out=dx2, accumulate=True)
    check_close(dx, to_np32(dx2), atol=unit_scale_atol(to_np32(dx2), 2e-2),
                what="NF4 input gradient with a rank-r term vs two products")


from qwen3_moe_fused.grouped_gemm.fused import grouped_glu_forward_lora  # noqa: E402


@pytest.mark.parametrize("R,N,K,E,r", [(4096, 768, 2048, 16, 16), (9000, 512, 256, 4, 32), (700, 208, 64, 5, 8),
                                       (33, 64, 192, 40, 16), (300, 72, 128, 3, 24)])
def test_glu_with_lora_terms_equals_the_separate_products(R, N, K, E, r):
    """Gate and up projections with their adapters' rank-r terms and the SiLU-mul in one launch: the two
    products bit for bit those of the product with one thin term (the other adapter's columns meet zeros), h
    the SiLU-mul kernel's on them."""
    g = gen(R + N + r + 3)
    x = randn((R, K), g, 1.0, torch.bfloat16).to(DEV)
    wg, wu = randn((E, N, K), g, 0.05, torch.bfloat16).to(DEV), randn((E, N, K), g, 0.05, torch.bfloat16).to(DEV)
    ug, uu = randn((R, r), g, 1.0, torch.bfloat16).to(DEV), randn((R, r), g, 1.0, torch.bfloat16).to(DEV)
    bg, bu = randn((E, N, r), g, 0.2, torch.bfloat16).to(DEV), randn((E, N, r), g, 0.2, torch.bfloat16).to(DEV)
    ms = m_sizes_uniform(R, E, g).to(DEV)
    xt = torch.cat([ug, uu], 1).contiguous()
    zeros = torch.zeros_like(bg)
    wt_g, wt_u = torch.cat([bg, zeros], 2).contiguous(), torch.cat([zeros, bu], 2).contiguous()
    h, e, gg = grouped_glu_forward_lora(x, wg, wu, xt, wt_g, wt_u, ms)
    e_ref = grouped_gemm_forward_lora(x, wg, ug, bg, ms)
    g_ref = grouped_gemm_forward_lora(x, wu, uu, bu, ms)
    sel = oracle.sel_from_m_sizes(ms.cpu().numpy())
    ref = (oracle.linear_fwd(to_np32(x), to_np32(wg), sel).astype(np.float64)
           + oracle.linear_fwd(to_np32(ug), to_np32(bg), sel))
    check_close(e, ref, what="gate product with its rank-r term vs oracle")
    if K % 64 == 0:
        assert torch.equal(e, e_ref) and torch.equal(gg, g_ref), "the same reductions in the same order"
        assert torch.equal(h, silu_mul_forward(e_ref, g_ref))
    else:
        check_close(e, to_np32(e_ref), what="gate product")
        check_close(gg, to_np32(g_ref), what="up product")
        assert torch.equal(h, silu_mul_forward(e, gg))
