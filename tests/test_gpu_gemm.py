"""GPU parity of the grouped GEMM (fwd / dX / dW) against the CPU oracle, through the C ABI
(the Python wrappers are thin ctypes calls).  Shapes follow the reference's own scripts
(test_moe_fused_linear.py:19-23: 1024 x 2048 -> 768, 128 experts; the tiny model's odd sizes
3 / 16 / 11 experts from test_model.py:29-40) plus the benchmark configurations 1-3."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, m_sizes_uniform, randn, to_np32, topk_routing

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.functional import moe_fused_linear  # noqa: E402
from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed  # noqa: E402

DEV = "cuda"


def _case(seed, R, N, K, E, dtype, m_sizes=None):
    g = gen(seed)
    x = randn((R, K), g, 1.0, dtype)
    w = randn((E, N, K), g, 0.02 if dtype != torch.float32 else 0.1, dtype)
    dy = randn((R, N), g, 1.0, dtype)
    ms = m_sizes_uniform(R, E, g) if m_sizes is None else m_sizes
    sel = oracle.sel_from_m_sizes(ms.numpy())
    return x, w, dy, ms, sel


def _tol(dtype):
    return (1e-2, 1e-2) if dtype != torch.float32 else (1e-4, 1e-4)  # the reference's fp32 figures (test_moe_fused_linear.py:30-32)


SHAPES = [
    # R, N, K, E
    (512, 128, 64, 8),       # benchmark configuration 1 sizes
    (1024, 768, 2048, 128),  # the reference's test shape
    (91, 3, 16, 11),         # tiny model: gate/up (moe_intermediate 3, hidden 16, 11 experts)
    (91, 16, 3, 11),         # tiny model: down
    (300, 40, 72, 5),        # multiples of 8 only
    (257, 136, 264, 3),      # one row past a tile edge
    (64, 16, 2048, 128),     # LoRA A shape, most experts empty
    (64, 768, 16, 128),      # LoRA B shape
    (2000, 200, 256, 3),     # experts of several row tiles each
    (700, 64, 128, 600),     # more experts than the pipelined kernel's LDS tables hold
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("R,N,K,E", SHAPES)
def test_forward_dx_dw_match_oracle(R, N, K, E, dtype):
    x, w, dy, ms, sel = _case(1234 + R + N, R, N, K, E, dtype)
    rtol, atol = _tol(dtype)
    xd, wd, dyd, msd = x.to(DEV), w.to(DEV), dy.to(DEV), ms.to(DEV)

    y = grouped_gemm_forward(xd, wd, msd)
    assert y.dtype == dtype and y.shape == (R, N)
    check_close(y, oracle.linear_fwd(to_np32(x), to_np32(w), sel), rtol, atol, "fwd")

    dx = grouped_gemm_forward_transposed(dyd, wd, msd)
    check_close(dx, oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel), rtol, atol, "dx")

    dw = grouped_gemm_backward_dw(xd, dyd, msd, dtype)
    exp_dw = oracle.linear_bwd_weight(to_np32(dy), to_np32(x), sel, E)
    # dW sums up to R/E products of N(0,1) values: scale the absolute tolerance with its size
    check_close(dw, exp_dw, rtol, atol * max(1.0, np.abs(exp_dw).max()), "dw")
    empty = (ms == 0).nonzero().flatten().tolist()
    for e in empty:
        assert torch.count_nonzero(dw[e]).item() == 0, "experts without rows must get exact zeros"


def test_autograd_matches_oracle_bf16():
    """moe_fused_linear(...).backward, the reference's test_moe_fused_linear_bwd.py:67-78."""
    R, N, K, E = 1024, 768, 2048, 128
    x, w, dy, ms, sel = _case(7, R, N, K, E, torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    wd = w.to(DEV).requires_grad_()
    out = moe_fused_linear(xd, wd, ms.to(DEV))
    out.backward(dy.to(DEV))
    check_close(out, oracle.linear_fwd(to_np32(x), to_np32(w), sel), what="fwd")
    check_close(xd.grad, oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel), what="dx")
    exp_dw = oracle.linear_bwd_weight(to_np32(dy), to_np32(x), sel, E)
    check_close(wd.grad, exp_dw, 1e-2, 1e-2 * max(1.0, np.abs(exp_dw).max()), "dw")
    # grads are gated on requires_grad (interface.py:18-26)
    x2 = x.to(DEV).requires_grad_()
    moe_fused_linear(x2, w.to(DEV), ms.to(DEV)).backward(dy.to(DEV))
    assert x2.grad is not None


@pytest.mark.parametrize("ms_dtype", [torch.int32, torch.int64, torch.int16])
def test_m_sizes_integer_types(ms_dtype):
    x, w, dy, ms, sel = _case(11, 256, 64, 64, 4, torch.bfloat16)
    y = grouped_gemm_forward(x.to(DEV), w.to(DEV), ms.to(ms_dtype).to(DEV))
    check_close(y, oracle.linear_fwd(to_np32(x), to_np32(w), sel), what="fwd")


def test_edge_cases_empty_and_single_expert():
    # no rows at all
    w = randn((4, 32, 64), gen(0), 0.02, torch.bfloat16).to(DEV)
    ms0 = torch.zeros(4, dtype=torch.int32, device=DEV)
    y = grouped_gemm_forward(torch.empty((0, 64), dtype=torch.bfloat16, device=DEV), w, ms0)
    assert y.shape == (0, 32)
    dw = grouped_gemm_backward_dw(torch.empty((0, 64), dtype=torch.bfloat16, device=DEV),
                                  torch.empty((0, 32), dtype=torch.bfloat16, device=DEV), ms0, torch.bfloat16)
    assert dw.shape == (4, 32, 64) and torch.count_nonzero(dw).item() == 0
    # E = 1 is an ordinary linear layer
    x, w1, dy, ms, sel = _case(3, 200, 48, 96, 1, torch.bfloat16, m_sizes=torch.tensor([200], dtype=torch.int32))
    y = grouped_gemm_forward(x.to(DEV), w1.to(DEV), ms.to(DEV))
    ref = torch.nn.functional.linear(x.float(), w1[0].float())
    check_close(y, ref.numpy(), what="E=1 vs F.linear")
    # all rows on the last expert, the rest empty
    ms_last = torch.tensor([0, 0, 0, 130], dtype=torch.int32)
    x, w4, dy, _, _ = _case(4, 130, 32, 64, 4, torch.bfloat16, m_sizes=ms_last)
    sel = oracle.sel_from_m_sizes(ms_last.numpy())
    y = grouped_gemm_forward(x.to(DEV), w4.to(DEV), ms_last.to(DEV))
    check_close(y, oracle.linear_fwd(to_np32(x), to_np32(w4), sel), what="last expert only")


@pytest.mark.parametrize("R,N,K,E,dtype", [(600, 192, 128, 4, torch.bfloat16),   # pipelined kernel
                                           (90, 24, 40, 3, torch.bfloat16),      # register-staged kernel
                                           (90, 3, 16, 3, torch.float32)])       # generic kernel
def test_rows_past_the_sum_of_m_sizes_stay_unwritten(R, N, K, E, dtype):
    """sum(m_sizes) < R: the products cover the first sum(m_sizes) rows only; the reference's
    wrappers leave the rest of the freshly allocated output as it is (forward.py:136)."""
    x, w, dy, _, _ = _case(21, R, N, K, E, dtype)
    ms = torch.full((E,), (R - 37) // E, dtype=torch.int32)
    used = int(ms.sum())
    assert used < R
    sel = oracle.sel_from_m_sizes(ms.numpy())
    rtol, atol = _tol(dtype)
    sentinel = 12345.0
    out = torch.full((R, N), sentinel, dtype=dtype, device=DEV)
    grouped_gemm_forward(x.to(DEV), w.to(DEV), ms.to(DEV), out=out)
    check_close(out[:used], oracle.linear_fwd(to_np32(x[:used]), to_np32(w), sel), rtol, atol, "fwd, used rows")
    assert (out[used:] == sentinel).all(), "forward wrote past sum(m_sizes)"
    dx = torch.full((R, K), sentinel, dtype=dtype, device=DEV)
    grouped_gemm_forward_transposed(dy.to(DEV), w.to(DEV), ms.to(DEV), out=dx)
    check_close(dx[:used], oracle.linear_bwd_input(to_np32(dy[:used]), to_np32(w), sel), rtol, atol, "dx, used rows")
    assert (dx[used:] == sentinel).all(), "input gradient wrote past sum(m_sizes)"
    dw = grouped_gemm_backward_dw(x.to(DEV), dy.to(DEV), ms.to(DEV), dtype)
    exp_dw = oracle.linear_bwd_weight(to_np32(dy[:used]), to_np32(x[:used]), sel, E)
    check_close(dw, exp_dw, rtol, atol * max(1.0, np.abs(exp_dw).max()), "dw ignores the trailing rows")


def test_alpha_and_accumulate():
    x, w, dy, ms, sel = _case(5, 300, 64, 128, 6, torch.bfloat16)
    base = randn((300, 64), gen(6), 1.0, torch.bfloat16)
    out = base.clone().to(DEV)
    grouped_gemm_forward(x.to(DEV), w.to(DEV), ms.to(DEV), out=out, alpha=0.5, accumulate=True)
    ref = to_np32(base) + 0.5 * oracle.linear_fwd(to_np32(x), to_np32(w), sel)
    check_close(out, ref, what="y += alpha * x w^T")


def test_wrapper_asserts_like_the_reference():
    w = torch.zeros((2, 8, 8), dtype=torch.bfloat16, device=DEV)
    ms = torch.tensor([1, 1], dtype=torch.int32, device=DEV)
    with pytest.raises(AssertionError):
        grouped_gemm_forward(torch.zeros((2, 8), dtype=torch.bfloat16), w, ms)           # CPU input
    with pytest.raises(AssertionError):
        grouped_gemm_forward(torch.zeros((2, 16), dtype=torch.bfloat16, device=DEV), w, ms)  # K mismatch
    with pytest.raises(AssertionError):
        grouped_gemm_forward(torch.zeros((2, 8), dtype=torch.bfloat16, device=DEV), w, ms.float())


# ---- benchmark configurations 2 and 3 at full size: oracle on a sample + size-independent properties

def _config23(seed):
    g = gen(seed)
    E, H, I, T, k = 128, 2048, 768, 4096, 8
    sel, ms = topk_routing(T, E, k, g)
    return g, E, H, I, T * k, ms


def test_config2_gate_proj_forward_full_size():
    g, E, H, I, R, ms = _config23(2)
    x = randn((R, H), g, 1.0, torch.bfloat16)
    w = randn((E, I, H), g, 0.02, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    xd, wd, msd = x.to(DEV), w.to(DEV), ms.to(DEV)
    y = grouped_gemm_forward(xd, wd, msd)
    rows = np.sort(np.random.default_rng(0).choice(R, 1024, replace=False))
    # include the first and last row of some experts (tile edges)
    ends = np.cumsum(ms.numpy())
    rows = np.unique(np.concatenate([rows, ends[:16] - 1, ends[:16] % R]))
    exp = oracle.linear_fwd(to_np32(x[rows]), to_np32(w), sel[rows])
    check_close(y[rows], exp, what="config 2 sampled rows")
    # linearity in x: f(2x) == 2 f(x) exactly in bf16 (power-of-two scaling)
    y2 = grouped_gemm_forward(xd * 2, wd, msd)
    assert torch.equal(y2, y * 2)
    # run-to-run determinism
    assert torch.equal(grouped_gemm_forward(xd, wd, msd), y)


def test_config3_down_proj_backward_full_size():
    g, E, H, I, R, ms = _config23(3)
    x = randn((R, I), g, 1.0, torch.bfloat16)
    dy = randn((R, H), g, 1.0, torch.bfloat16)
    w = randn((E, H, I), g, 0.02, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    xd, dyd, wd, msd = x.to(DEV), dy.to(DEV), w.to(DEV), ms.to(DEV)
    dx = grouped_gemm_forward_transposed(dyd, wd, msd)
    rows = np.sort(np.random.default_rng(1).choice(R, 1024, replace=False))
    check_close(dx[rows], oracle.linear_bwd_input(to_np32(dy[rows]), to_np32(w), sel[rows]), what="config 3 dX")
    dw = grouped_gemm_backward_dw(xd, dyd, msd, torch.bfloat16)
    # per-expert dW depends only on that expert's rows: oracle on a few experts
    starts = np.concatenate([[0], np.cumsum(ms.numpy())])
    for e in (0, 63, 127):
        sl = slice(starts[e], starts[e + 1])
        exp = oracle.linear_bwd_weight(to_np32(dy[sl]), to_np32(x[sl]), np.zeros(sl.stop - sl.start, np.int64), 1)[0]
        check_close(dw[e], exp, 1e-2, 1e-2 * np.abs(exp).max(), f"config 3 dW expert {e}")
    # checksum identity: sum_e dW[e] == dy^T x  (fp32 accumulation of bf16-rounded tiles)
    total = dw.float().sum(dim=0)
    ref = dyd.float().t() @ xd.float()
    check_close(total, to_np32(ref), 2e-2, 2e-2 * float(ref.abs().max()), "sum_e dW == dy^T x")
    assert torch.equal(grouped_gemm_backward_dw(xd, dyd, msd, torch.bfloat16), dw)


# ---- randomised shapes: every tile configuration and edge path of the bf16 kernels
def _random_case(seed):
    rng = np.random.default_rng(seed)
    E = int(rng.choice([1, 2, 3, 5, 8, 17, 40]))
    N = int(rng.choice([8, 16, 24, 64, 72, 136, 200, 256, 384, 520]))
    K = int(rng.choice([8, 16, 64, 72, 128, 192, 264, 512]))
    kind = int(rng.integers(0, 4))
    if kind == 0:      # a few rows per expert (decode-sized), many experts empty
        m = rng.integers(0, 6, size=E) * (rng.random(E) < 0.6)
    elif kind == 1:    # a few hundred rows per expert
        m = rng.integers(100, 400, size=E)
    elif kind == 2:    # skewed: one expert holds most rows, several tiles of it
        m = rng.integers(0, 40, size=E)
        m[int(rng.integers(0, E))] += int(rng.integers(700, 1500))
    else:              # tile edges
        m = rng.choice([0, 1, 31, 32, 33, 255, 256, 257, 319, 320, 321], size=E)
    m = np.minimum(m, max(1, 6000 // E)).astype(np.int64)
    return E, N, K, torch.from_numpy(m)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_match_oracle_bf16(seed):
    E, N, K, ms = _random_case(seed)
    R = int(ms.sum())
    x, w, dy, _, _ = _case(9000 + seed, R, N, K, E, torch.bfloat16, m_sizes=ms)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    xd, wd, dyd, msd = x.to(DEV), w.to(DEV), dy.to(DEV), ms.to(DEV)
    what = f"seed {seed}: E={E} N={N} K={K} m_sizes={ms.tolist()}"

    y = grouped_gemm_forward(xd, wd, msd)
    exp_y = oracle.linear_fwd(to_np32(x), to_np32(w), sel)
    check_close(y, exp_y, 1e-2, 1e-2, "fwd " + what)
    # y2 = 0.5 * product + y, rounded once
    y2 = y.clone()
    grouped_gemm_forward(xd, wd, msd, out=y2, alpha=0.5, accumulate=True)
    check_close(y2, 0.5 * exp_y + to_np32(y), 1e-2, 1e-2, "fwd accumulate " + what)

    dx = grouped_gemm_forward_transposed(dyd, wd, msd)
    check_close(dx, oracle.linear_bwd_input(to_np32(dy), to_np32(w), sel), 1e-2, 1e-2, "dx " + what)

    dw = grouped_gemm_backward_dw(xd, dyd, msd, torch.bfloat16)
    exp_dw = oracle.linear_bwd_weight(to_np32(dy), to_np32(x), sel, E)
    check_close(dw, exp_dw, 1e-2, 1e-2 * max(1.0, np.abs(exp_dw).max()), "dw " + what)
    for e in (ms == 0).nonzero().flatten().tolist():
        assert torch.count_nonzero(dw[e]).item() == 0, "experts without rows must get exact zeros"


# ---- the four-wave kernel (128 x 128 wave tiles): whole 256 x 256 tiles along the weight dimensions and at least
# 64 rows per expert on average.  Row counts that end inside a 32-row step, inside its first half, on a step edge;
# experts without rows (exact zeros, written between two experts with rows); one expert that holds most rows; rows
# past sum(m_sizes); int64 sizes; more experts than a wave has lanes.
WIDE_DW_CASES = [
    # N, K, m_sizes
    (256, 256, [64]),
    (256, 512, [1, 0, 300, 31, 32, 33, 0, 700]),
    (512, 256, [0, 0, 517, 0, 15, 16, 17, 480, 0]),
    (768, 256, [96] * 7 + [0] + [1000]),
    (256, 768, [70 + (3 * e) % 11 for e in range(130)]),
]


@pytest.mark.parametrize("N,K,sizes", WIDE_DW_CASES)
@pytest.mark.parametrize("ms_dtype", [torch.int32, torch.int64])
def test_dw_four_wave_kernel_matches_oracle(N, K, sizes, ms_dtype):
    ms = torch.tensor(sizes, dtype=ms_dtype)
    E, rows = ms.numel(), int(ms.sum())
    extra = 37                                   # rows that belong to no expert
    R = max(rows + extra, 64 * E)                # enough rows for the dispatcher to take this kernel
    g = gen(N + K + E)
    x = randn((R, K), g, 1.0, torch.bfloat16)
    dy = randn((R, N), g, 1.0, torch.bfloat16)
    x[rows:] = float("nan")
    dy[rows:] = float("inf")
    sel = oracle.sel_from_m_sizes(ms.numpy())
    xd, dyd, msd = x.to(DEV), dy.to(DEV), ms.to(DEV)
    print(f"four-wave dW N={N} K={K} E={E} R={R}", flush=True)
    dw = grouped_gemm_backward_dw(xd, dyd, msd, torch.bfloat16)
    exp = oracle.linear_bwd_weight(to_np32(dy[:rows]), to_np32(x[:rows]), sel, E)
    check_close(dw, exp, 1e-2, 1e-2 * max(1.0, np.abs(exp).max()), "four-wave dW")
    for e in (ms == 0).nonzero().flatten().tolist():
        assert torch.count_nonzero(dw[e]).item() == 0, "experts without rows must get exact zeros"
    assert torch.equal(grouped_gemm_backward_dw(xd, dyd, msd, torch.bfloat16), dw), "same bits from run to run"


# the same kernel in the row-grouped products (forward and input gradient with more than 64 output columns, from 48
# rows per expert on average): tiles of 320 x 192 up to 512 rows per expert, so N = 200, 520 and 2048 end in a partial
# column tile; experts of 0, 1, 319, 320, 321 and 700 rows (no tile, one block, a full tile, a tile and one row,
# several tiles); a reduction longer than the output is wide; 256 x 256 tiles from 512 rows per expert on (N = 520:
# two tiles and eight columns).
WIDE_ROW_CASES = [
    # N, K, m_sizes
    (200, 64, [300, 0, 1, 319, 320, 321, 700, 95]),
    (520, 128, [257] * 5 + [0, 64, 512]),
    (2048, 768, [250 + 7 * (e % 5) for e in range(16)]),
    (384, 192, [100 + e for e in range(70)]),
    (768, 2048, [48, 60, 0, 130, 50, 49]),
    (520, 128, [1000, 0, 700]),
    (768, 256, [513, 2047, 256, 1300]),
    # 192 x 256 tiles (outputs a multiple of 256 columns and at least 1024 wide, at most 152 rows per expert on
    # average): experts of 0, 1, 191, 192 and 193 rows, one of two tiles, a reduction of one step
    (2048, 768, [100 + 13 * (e % 7) for e in range(16)]),
    (1024, 128, [0, 193, 60, 192, 1, 150, 191, 120]),
    (1280, 64, [64] * 3 + [400, 48, 0, 97, 129]),
    # the same widths between 152 and 232 rows per expert: 256 x 256 tiles (experts of 255, 256, 257 and 520 rows)
    (1024, 192, [255, 256, 257, 0, 190, 520, 100, 180]),
]


@pytest.mark.parametrize("N,K,sizes", WIDE_ROW_CASES)
def test_row_grouped_products_on_the_four_wave_kernel_match_oracle(N, K, sizes):
    ms = torch.tensor(sizes, dtype=torch.int32)
    E, R = ms.numel(), int(ms.sum())
    assert 48 * E <= R and N > 64 and K % 64 == 0
    x, w, _, _, sel = _case(N + K + E, R, N, K, E, torch.bfloat16, m_sizes=ms)
    xd, wd, msd = x.to(DEV), w.to(DEV), ms.to(DEV)
    print(f"four-wave fwd/dX N={N} K={K} E={E} R={R}", flush=True)
    y = grouped_gemm_forward(xd, wd, msd)
    check_close(y, oracle.linear_fwd(to_np32(x), to_np32(w), sel), 1e-2, 1e-2, "four-wave fwd")
    assert torch.equal(grouped_gemm_forward(xd, wd, msd), y)
    # input gradient with the roles the kernel sees: dy (R, K) against w2 (E, K, N) -> (R, N)
    g = gen(7 + N)
    dy = randn((R, K), g, 1.0, torch.bfloat16)
    w2 = randn((E, K, N), g, 0.02, torch.bfloat16)
    dx = grouped_gemm_forward_transposed(dy.to(DEV), w2.to(DEV), msd)
    exp = oracle.linear_bwd_input(to_np32(dy), to_np32(w2), sel)
    check_close(dx, exp, 1e-2, 1e-2, "four-wave dX")
