"""Fused NF4-dequant grouped GEMM against the oracle (oracle dequant -> oracle linear), the way
the reference checks its 4-bit kernel against the naive forward on dequantised weights
(test_moe_fused_linear.py:39-58), plus fused == dequant-then-GEMM within bf16 tolerance."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, m_sizes_uniform, randn, to_np32, unit_scale_atol

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_4bit  # noqa: E402
from qwen3_moe_fused.quantize.nf4 import Nf4QuantState, dequantize_nf4, nf4_code  # noqa: E402

DEV = "cuda"


def _quantised(E, N, K, blocksize, seed):
    w = randn((E, N, K), gen(seed), 0.02)
    q, absmax = oracle.nf4_quant(w.numpy(), blocksize)
    w_deq = oracle.round_bf16(oracle.nf4_dequant(q, absmax, blocksize)).reshape(E, N, K)
    state = Nf4QuantState(absmax=torch.from_numpy(absmax).to(DEV), shape=(E, N, K), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=torch.bfloat16)
    return torch.from_numpy(q).view(-1, 1).to(DEV), state, w_deq


@pytest.mark.parametrize("R,N,K,E,blocksize", [(1024, 768, 2048, 128, 256), (1024, 768, 2048, 128, 64),
                                               (128, 768, 2048, 128, 64), (300, 40, 72, 5, 8), (513, 136, 64, 3, 64),
                                               # >= 32 rows per expert: the pipelined kernel, several row tiles
                                               # per expert and many reduction steps
                                               (8192, 768, 2048, 16, 64), (4096, 200, 512, 4, 128),
                                               # an output of 1024 columns at 200 rows per expert: 256 x 256 tiles
                                               (1600, 1024, 128, 8, 64),
                                               # small quantisation blocks on the pipelined kernel
                                               (2048, 64, 128, 2, 16), (1500, 72, 192, 3, 8),
                                               # decode-sized batches (register-decode kernel), small blocks, a
                                               # column count that is not a multiple of 32
                                               (60, 64, 128, 3, 16), (90, 72, 256, 5, 8), (200, 200, 192, 9, 32),
                                               # at most two rows per expert: the decode kernel loads the
                                               # rows a lane per row, without its LDS stage
                                               (10, 64, 128, 8, 16), (12, 72, 256, 6, 64)])
def test_fused_nf4_forward(R, N, K, E, blocksize):
    packed, state, w_deq = _quantised(E, N, K, blocksize, R + N)
    g = gen(R)
    x = randn((R, K), g, 1.0, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    y = grouped_gemm_forward_4bit(x.to(DEV), packed, state, ms.to(DEV))
    assert y.dtype == torch.bfloat16 and y.shape == (R, N)
    check_close(y, oracle.linear_fwd(to_np32(x), w_deq, sel), what="fused nf4 vs oracle")
    # the unfused route (dequantise, then bf16 GEMM) sees the same bf16 weights
    y2 = grouped_gemm_forward(x.to(DEV), dequantize_nf4(packed, state, torch.bfloat16), ms.to(DEV))
    check_close(y, to_np32(y2), 1e-2, 1e-2, "fused vs dequant-then-GEMM")


def _random_nf4_case(seed):
    rng = np.random.default_rng(seed)
    E = int(rng.choice([1, 3, 6, 20]))
    N = int(rng.choice([8, 40, 64, 136, 256, 392]))
    K = int(rng.choice([64, 72, 128, 192, 512]))
    blocksize = int(rng.choice([8, 16, 32, 64, 128]))
    while (N * K) % blocksize:  # a quantisation block must not straddle two experts
        blocksize //= 2
    kind = int(rng.integers(0, 3))
    if kind == 0:      # decode-sized
        m = rng.integers(0, 20, size=E)
    elif kind == 1:    # a few hundred rows per expert
        m = rng.integers(60, 400, size=E)
    else:              # one large expert
        m = rng.integers(0, 30, size=E)
        m[int(rng.integers(0, E))] += int(rng.integers(600, 1200))
    return E, N, K, blocksize, torch.from_numpy(m.astype(np.int64))


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_fused_nf4(seed):
    E, N, K, blocksize, ms = _random_nf4_case(seed)
    R = int(ms.sum())
    packed, state, w_deq = _quantised(E, N, K, blocksize, 700 + seed)
    x = randn((R, K), gen(800 + seed), 1.0, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    y = grouped_gemm_forward_4bit(x.to(DEV), packed, state, ms.to(DEV))
    check_close(y, oracle.linear_fwd(to_np32(x), w_deq, sel),
                what=f"seed {seed}: E={E} N={N} K={K} blocksize={blocksize} m_sizes={ms.tolist()}")


# The streaming decode-size kernel (K % 128 == 0, blocks of at least 64 weights, at most 32 rows per expert on
# average): one stage, an odd number of stages, column counts that leave a wave or a workgroup partly or wholly
# empty, experts of two and three row tiles, more than 64 experts, empty experts, large quantisation blocks,
# 64-bit row counts, fp32 output, rows past sum(m_sizes).
@pytest.mark.parametrize("m_sizes,N,K,blocksize,ms_dtype,out_dtype", [
    ([3, 0, 1, 7], 8, 128, 64, torch.int32, torch.bfloat16),
    ([5, 2], 136, 384, 64, torch.int64, torch.bfloat16),
    ([33, 0, 70, 1, 0, 12], 200, 256, 128, torch.int32, torch.float32),
    ([1] * 70 + [0] * 5 + [40], 64, 128, 64, torch.int32, torch.bfloat16),
    ([9, 31, 32, 2], 264, 640, 512, torch.int64, torch.bfloat16),
    ([0, 0, 6, 0], 768, 2048, 256, torch.int32, torch.bfloat16),
])
def test_streaming_decode_kernel_edges(m_sizes, N, K, blocksize, ms_dtype, out_dtype):
    E = len(m_sizes)
    ms = torch.tensor(m_sizes, dtype=ms_dtype)
    R = int(ms.sum()) + 3                      # three rows past the last expert: not written
    assert R <= 32 * E and K % 128 == 0 and blocksize >= 64 and (N * K) % blocksize == 0
    packed, state, w_deq = _quantised(E, N, K, blocksize, N + K)
    x = randn((R, K), gen(K), 1.0, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(np.asarray(m_sizes))
    y = torch.full((R, N), 7.0, device=DEV, dtype=out_dtype)
    from qwen3_moe_fused import _lib
    xd, msd = x.to(DEV), ms.to(DEV)
    rc = _lib.lib().mfl_gemm_fwd_nf4(_lib.ptr(xd), _lib.ptr(packed), _lib.ptr(state.code), _lib.ptr(state.absmax), blocksize,
                                     _lib.ptr(msd), _lib.itype_code(ms_dtype), _lib.ptr(y), R, N, K, E,
                                     _lib.dtype_code(torch.bfloat16), _lib.dtype_code(out_dtype), _lib.stream())
    _lib.check(rc, "mfl_gemm_fwd_nf4")
    ref = oracle.linear_fwd(to_np32(x)[:R - 3], w_deq, sel)
    check_close(y[:R - 3], ref, what=f"streaming kernel m_sizes={m_sizes} N={N} K={K} blocksize={blocksize}")
    assert torch.all(y[R - 3:] == 7.0), "rows past sum(m_sizes) stay as they were"
    # through the wrapper, and again: the same bits
    y2 = grouped_gemm_forward_4bit(xd, packed, state, msd, out_dtype)
    assert torch.equal(y2[:R - 3], y[:R - 3])


# The same kernel with 64-row tiles, which the plain product takes from 20 up to 128 rows per expert on average:
# experts that end inside the first or the second 32-row block of a tile, experts of two and three tiles, empty
# experts, a last column tile that is partly empty, fp32 output, rows past sum(m_sizes); with and without the
# tile-ordered scales (the same bits).
@pytest.mark.parametrize("m_sizes,N,K,blocksize,ms_dtype,out_dtype", [
    ([65, 0, 40, 128, 33, 1, 64, 97], 200, 256, 128, torch.int32, torch.bfloat16),
    ([70, 70, 0, 150, 31], 136, 384, 64, torch.int64, torch.float32),
    ([100] * 3 + [0] + [96] * 2, 768, 2048, 64, torch.int32, torch.bfloat16),
])
def test_streaming_kernel_64_row_tiles(m_sizes, N, K, blocksize, ms_dtype, out_dtype):
    E = len(m_sizes)
    ms = torch.tensor(m_sizes, dtype=ms_dtype)
    R = int(ms.sum()) + 3
    assert 20 * E < R <= 128 * E and K % 128 == 0 and blocksize >= 64
    packed, state, w_deq = _quantised(E, N, K, blocksize, N + K + 1)
    x = randn((R, K), gen(K + 1), 1.0, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(np.asarray(m_sizes))
    y = torch.full((R, N), 7.0, device=DEV, dtype=out_dtype)
    from qwen3_moe_fused import _lib
    xd, msd = x.to(DEV), ms.to(DEV)
    rc = _lib.lib().mfl_gemm_fwd_nf4(_lib.ptr(xd), _lib.ptr(packed), _lib.ptr(state.code), _lib.ptr(state.absmax), blocksize,
                                     _lib.ptr(msd), _lib.itype_code(ms_dtype), _lib.ptr(y), R, N, K, E,
                                     _lib.dtype_code(torch.bfloat16), _lib.dtype_code(out_dtype), _lib.stream())
    _lib.check(rc, "mfl_gemm_fwd_nf4")
    ref = oracle.linear_fwd(to_np32(x)[:R - 3], w_deq, sel)
    check_close(y[:R - 3], ref, what=f"streaming kernel, 64-row tiles, m_sizes={m_sizes} N={N} K={K}")
    assert torch.all(y[R - 3:] == 7.0), "rows past sum(m_sizes) stay as they were"
    # through the wrapper (which brings the tile-ordered scales): the same bits
    y2 = grouped_gemm_forward_4bit(xd, packed, state, msd, out_dtype)
    assert torch.equal(y2[:R - 3], y[:R - 3])


def _tile_ordered(absmax, E, N, K, blocksize):
    """The scales in the order the streaming kernel's waves consume them: [expert][32-column tile][128-wide
    stage][column of the tile][half of the stage], columns past N repeating the last one."""
    a = np.asarray(absmax, dtype=np.float32).reshape(-1)
    tiles, stages = -(-N // 32), K // 128
    e, t, s, l = np.meshgrid(np.arange(E), np.arange(tiles), np.arange(stages), np.arange(64), indexing="ij")
    col = np.minimum(32 * t + l // 2, N - 1)
    first_weight = (e.astype(np.int64) * N + col) * K + 128 * s + 64 * (l % 2)
    return a[first_weight // blocksize].reshape(-1)


# Scales handed over in the order of consumption: the copy is the permutation it is documented to be, and the plain,
# the gathered and the gated product return the same bits with it as without (column counts that are and are not
# multiples of 32 and 128, blocks of 64 to 512 weights, several row tiles per expert, empty experts).
@pytest.mark.parametrize("m_sizes,N,K,blocksize", [([3, 0, 1, 7], 8, 128, 64), ([33, 0, 70, 1, 0, 12], 200, 256, 128),
                                                   ([9, 31, 32, 2], 264, 640, 512), ([5, 17, 0, 2], 768, 2048, 64)])
def test_tile_ordered_scales(m_sizes, N, K, blocksize):
    from qwen3_moe_fused import _lib
    from qwen3_moe_fused.grouped_gemm.fused import grouped_glu_forward_4bit
    E, k_sel = len(m_sizes), 2
    ms = torch.tensor(m_sizes, dtype=torch.int32).to(DEV)
    R = int(sum(m_sizes))
    packed, state, _ = _quantised(E, N, K, blocksize, N + K + 1)
    packed_u, state_u, _ = _quantised(E, N, K, blocksize, N + K + 2)
    count = int(_lib.lib().mfl_nf4_tiled_absmax_floats(blocksize, N, K, E))
    assert count == E * -(-N // 32) * (K // 128) * 64
    tiled = torch.full((count,), -1.0, device=DEV)
    _lib.check(_lib.lib().mfl_nf4_tile_absmax(_lib.ptr(state.absmax), blocksize, N, K, E, _lib.ptr(tiled),
                                              _lib.stream()), "mfl_nf4_tile_absmax")
    assert np.array_equal(tiled.cpu().numpy(), _tile_ordered(state.absmax.cpu().numpy(), E, N, K, blocksize))
    tiled_u = torch.empty_like(tiled)
    _lib.check(_lib.lib().mfl_nf4_tile_absmax(_lib.ptr(state_u.absmax), blocksize, N, K, E, _lib.ptr(tiled_u),
                                              _lib.stream()), "mfl_nf4_tile_absmax")
    g = gen(N)
    src = randn((-(-R // k_sel), K), g, 1.0, torch.bfloat16).to(DEV)
    row_idx = torch.randperm(src.shape[0] * k_sel, generator=g)[:R].to(torch.int32).to(DEV)
    x = src[(row_idx // k_sel).long()].contiguous()
    bf, i32 = _lib.dtype_code(torch.bfloat16), _lib.itype_code(torch.int32)

    def fwd(rows, idx, t):
        y = torch.zeros((R, N), device=DEV, dtype=torch.bfloat16)
        rc = _lib.lib().mfl_gemm_fwd_nf4_tiled(_lib.ptr(rows), rows.shape[0], _lib.ptr(idx), k_sel, _lib.ptr(packed),
                                               _lib.ptr(state.code), _lib.ptr(state.absmax), _lib.ptr(t), blocksize,
                                               _lib.ptr(ms), i32, _lib.ptr(y), R, N, K, E, bf, bf, _lib.stream())
        _lib.check(rc, "mfl_gemm_fwd_nf4_tiled")
        return y

    def glu(tg, tu):
        out = [torch.zeros((R, N), device=DEV, dtype=torch.bfloat16) for _ in range(3)]
        rc = _lib.lib().mfl_glu_fwd_nf4_tiled(_lib.ptr(src), src.shape[0], _lib.ptr(row_idx), k_sel, _lib.ptr(packed),
                                              _lib.ptr(state.code), _lib.ptr(state.absmax), _lib.ptr(tg), blocksize,
                                              _lib.ptr(packed_u), _lib.ptr(state_u.code), _lib.ptr(state_u.absmax),
                                              _lib.ptr(tu), blocksize, _lib.ptr(ms), i32, _lib.ptr(out[0]),
                                              _lib.ptr(out[1]), _lib.ptr(out[2]), R, N, K, E, bf, _lib.stream())
        _lib.check(rc, "mfl_glu_fwd_nf4_tiled")
        return out

    plain = fwd(x, None, None)
    assert torch.equal(fwd(x, None, tiled), plain), "plain product"
    assert torch.equal(fwd(src, row_idx, None), plain) and torch.equal(fwd(src, row_idx, tiled), plain), "gathered rows"
    for a, b in zip(glu(tiled, tiled_u), glu(None, None)):
        assert torch.equal(a, b), "gated product"
    for a, b in zip(glu(tiled, None), glu(None, None)):  # one copy alone is not used
        assert torch.equal(a, b)
    # the wrappers build the copy once per state and take the same route
    assert torch.equal(grouped_gemm_forward_4bit(x, packed, state, ms), plain)
    first = state._mfl_absmax_tiled[3]
    grouped_gemm_forward_4bit(x, packed, state, ms)
    assert state._mfl_absmax_tiled[3] is first and torch.equal(first, tiled)
    h = grouped_glu_forward_4bit(src, packed, state, packed_u, state_u, ms, row_idx, k_sel)
    assert torch.equal(h, glu(None, None)[0])


def test_tile_ordered_scales_shapes_without_a_copy():
    from qwen3_moe_fused import _lib
    assert _lib.lib().mfl_nf4_tiled_absmax_floats(32, 64, 128, 2) == 0    # blocks under 64 weights
    assert _lib.lib().mfl_nf4_tiled_absmax_floats(64, 64, 192, 2) == 0    # K not a multiple of 128
    a = torch.ones(2 * 64 * 192 // 64, device=DEV)
    out = torch.zeros(16, device=DEV)
    assert _lib.lib().mfl_nf4_tile_absmax(_lib.ptr(a), 64, 64, 192, 2, _lib.ptr(out), _lib.stream()) == -6
    # a product over such a shape takes the pointer and ignores it
    packed, state, w_deq = _quantised(2, 64, 192, 64, 5)
    x = randn((6, 192), gen(3), 1.0, torch.bfloat16)
    ms = torch.tensor([4, 2], dtype=torch.int32)
    y = torch.zeros((6, 64), device=DEV, dtype=torch.bfloat16)
    xd, msd = x.to(DEV), ms.to(DEV)
    bf = _lib.dtype_code(torch.bfloat16)
    rc = _lib.lib().mfl_gemm_fwd_nf4_tiled(_lib.ptr(xd), 6, None, 1, _lib.ptr(packed), _lib.ptr(state.code),
                                           _lib.ptr(state.absmax), _lib.ptr(out), 64, _lib.ptr(msd),
                                           _lib.itype_code(torch.int32), _lib.ptr(y), 6, 64, 192, 2, bf, bf, _lib.stream())
    _lib.check(rc, "mfl_gemm_fwd_nf4_tiled")
    check_close(y, oracle.linear_fwd(to_np32(x), w_deq, oracle.sel_from_m_sizes(ms.numpy())), what="ignored copy")


# The matrix-vector kernel (at most two rows per expert on average, 256 < K <= 2048, K a multiple of the block
# size, N a multiple of 32; up to K = 1024 with 32 lanes to a column): lanes past the end of a row (K not a multiple of 512), experts of one to five rows
# (up to three row groups), empty experts, more than 64 experts, more units than workgroups and fewer, one
# block per row, 64-bit counts, fp32 output, rows past sum(m_sizes).
@pytest.mark.parametrize("m_sizes,N,K,blocksize,ms_dtype,out_dtype", [
    ([1, 0, 2, 1], 32, 2048, 64, torch.int32, torch.bfloat16),
    ([5, 0, 0, 0, 1, 0, 0, 0], 96, 1280, 128, torch.int64, torch.bfloat16),
    ([0] * 70 + [2] * 3 + [1] * 57, 32, 2048, 2048, torch.int32, torch.float32),
    ([2, 1, 0, 1, 0, 0], 288, 1536, 512, torch.int32, torch.bfloat16),
    ([1, 2, 0, 1, 3, 0, 0, 1], 768, 2048, 64, torch.int64, torch.bfloat16),
    ([1, 1], 32, 1088, 64, torch.int32, torch.bfloat16),
    ([0, 0, 0, 4], 64, 1032, 8, torch.int32, torch.float32),
    # 32 lanes to a column (K <= 1024, at most a row per expert on average) from here on
    ([1, 2, 0, 1, 0, 0, 0, 1], 2048, 768, 64, torch.int32, torch.bfloat16),
    ([2, 0, 0], 32, 1024, 128, torch.int64, torch.float32),
    ([1, 0, 1, 0, 0, 0, 3], 96, 264, 8, torch.int32, torch.bfloat16),
    ([0] * 66 + [1, 2], 64, 520, 8, torch.int32, torch.bfloat16),
])
def test_matrix_vector_decode_kernel_edges(m_sizes, N, K, blocksize, ms_dtype, out_dtype):
    E = len(m_sizes)
    ms = torch.tensor(m_sizes, dtype=ms_dtype)
    pad = min(3, (2 * E if K > 1024 else E) - int(ms.sum()))   # rows past the last expert: not written
    R = int(ms.sum()) + pad
    assert R <= (2 * E if K > 1024 else E) and 256 < K <= 2048 and K % blocksize == 0 and N % 32 == 0
    packed, state, w_deq = _quantised(E, N, K, blocksize, N + K)
    x = randn((R, K), gen(K), 1.0, torch.bfloat16)
    sel = oracle.sel_from_m_sizes(np.asarray(m_sizes))
    y = torch.full((R, N), 7.0, device=DEV, dtype=out_dtype)
    from qwen3_moe_fused import _lib
    xd, msd = x.to(DEV), ms.to(DEV)
    rc = _lib.lib().mfl_gemm_fwd_nf4(_lib.ptr(xd), _lib.ptr(packed), _lib.ptr(state.code), _lib.ptr(state.absmax), blocksize,
                                     _lib.ptr(msd), _lib.itype_code(ms_dtype), _lib.ptr(y), R, N, K, E,
                                     _lib.dtype_code(torch.bfloat16), _lib.dtype_code(out_dtype), _lib.stream())
    _lib.check(rc, "mfl_gemm_fwd_nf4")
    ref = oracle.linear_fwd(to_np32(x)[:R - pad], w_deq, sel)
    check_close(y[:R - pad], ref, atol=unit_scale_atol(ref),
                what=f"matrix-vector kernel m_sizes={m_sizes} N={N} K={K} blocksize={blocksize}")
    assert torch.all(y[R - pad:] == 7.0), "rows past sum(m_sizes) stay as they were"
    y2 = grouped_gemm_forward_4bit(xd, packed, state, msd, out_dtype)
    assert torch.equal(y2[:R - pad], y[:R - pad])
    # counts that run past the rows given: the rows that exist are computed, nothing past them is touched
    R_short = int(ms.sum()) - 1
    if R_short >= 1:
        y3 = torch.full((R_short + 1, N), 7.0, device=DEV, dtype=out_dtype)
        rc = _lib.lib().mfl_gemm_fwd_nf4(_lib.ptr(xd), _lib.ptr(packed), _lib.ptr(state.code), _lib.ptr(state.absmax),
                                         blocksize, _lib.ptr(msd), _lib.itype_code(ms_dtype), _lib.ptr(y3), R_short, N, K,
                                         E, _lib.dtype_code(torch.bfloat16), _lib.dtype_code(out_dtype), _lib.stream())
        _lib.check(rc, "mfl_gemm_fwd_nf4")
        assert torch.equal(y3[:R_short], y[:R_short]) and torch.all(y3[R_short] == 7.0)


from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_transposed_4bit  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed  # noqa: E402


# weight (E, K = out_features, N = in_features); dx (R, N) = dy (R, K) @ w[e]
@pytest.mark.parametrize("R,N,K,E,blocksize", [(1024, 2048, 768, 128, 64), (4096, 768, 2048, 16, 64),
                                               (300, 64, 64, 5, 8), (513, 160, 128, 3, 32), (2000, 96, 192, 2, 16),
                                               (40, 32, 64, 7, 128), (5000, 416, 128, 3, 256),
                                               (1600, 1024, 128, 8, 64)])   # 256 x 256 tiles at 200 rows per expert
def test_fused_nf4_input_gradient(R, N, K, E, blocksize):
    packed, state, w_deq = _quantised(E, K, N, blocksize, R + N)
    g = gen(R + 1)
    dy = randn((R, K), g, 1.0, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    sel = oracle.sel_from_m_sizes(ms.numpy())
    ref = oracle.linear_bwd_input(to_np32(dy), w_deq, sel)
    dx = grouped_gemm_forward_transposed_4bit(dy.to(DEV), packed, state, ms.to(DEV))
    assert dx.dtype == torch.bfloat16 and dx.shape == (R, N)
    check_close(dx, ref, what="fused nf4 dx vs oracle")
    # the same bf16 weights through the dequantise-then-GEMM route: same products, same order
    dx2 = grouped_gemm_forward_transposed(dy.to(DEV), dequantize_nf4(packed, state, torch.bfloat16), ms.to(DEV))
    check_close(dx, to_np32(dx2), 1e-2, 1e-2, "fused vs dequant-then-GEMM")
    # accumulate into an existing output with a scale: out = out0 + 0.5 * dx, one rounding
    out0 = randn((R, N), g, 1.0, torch.bfloat16)
    out = out0.to(DEV).clone()
    grouped_gemm_forward_transposed_4bit(dy.to(DEV), packed, state, ms.to(DEV), out=out, alpha=0.5, accumulate=True)
    check_close(out, to_np32(out0) + 0.5 * ref, what="fused nf4 dx, accumulate")


def test_nf4_input_gradient_falls_back_for_odd_widths():
    # N not a multiple of 32: no fused kernel; the wrapper dequantises and runs the plain product
    R, N, K, E, blocksize = 200, 72, 64, 4, 16
    packed, state, w_deq = _quantised(E, K, N, blocksize, 9)
    g = gen(10)
    dy = randn((R, K), g, 1.0, torch.bfloat16)
    ms = m_sizes_uniform(R, E, g)
    dx = grouped_gemm_forward_transposed_4bit(dy.to(DEV), packed, state, ms.to(DEV))
    check_close(dx, oracle.linear_bwd_input(to_np32(dy), w_deq, oracle.sel_from_m_sizes(ms.numpy())), what="fallback")


@pytest.mark.parametrize("R,N,K,E,blocksize,dtype", [(120, 24, 20, 3, 4, torch.bfloat16),     # K % 8 != 0, blocks under 8 weights
                                                     (90, 40, 64, 5, 64, torch.float32),      # fp32 rows
                                                     (64, 16, 36, 2, 2, torch.float16)])      # fp16 rows, K % 8 != 0
def test_nf4_forward_falls_back_for_inputs_without_a_fused_kernel(R, N, K, E, blocksize, dtype):
    # the reference's wrapper takes these (forward_4bit.py:107-160); here the wrapper dequantises and multiplies
    w = randn((E, N, K), gen(R), 0.1)
    q, absmax = oracle.nf4_quant(w.numpy(), blocksize)
    w_deq = oracle.nf4_dequant(q, absmax, blocksize).reshape(E, N, K)
    if dtype != torch.float32:
        w_deq = to_np32(torch.from_numpy(w_deq).to(dtype))
    state = Nf4QuantState(absmax=torch.from_numpy(absmax).to(DEV), shape=(E, N, K), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=dtype)
    g = gen(R + 1)
    x = randn((R, K), g, 1.0, dtype)
    ms = m_sizes_uniform(R, E, g)
    y = grouped_gemm_forward_4bit(x.to(DEV), torch.from_numpy(q).view(-1, 1).to(DEV), state, ms.to(DEV))
    assert y.dtype == dtype
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    check_close(y, oracle.linear_fwd(to_np32(x), w_deq, oracle.sel_from_m_sizes(ms.numpy())), tol, tol, "fallback forward")
