"""mfl_gemm_dw_split (dW with one side as thin as a LoRA rank, rows dealt out evenly over the workgroups)
against the CPU oracle's weight gradient (oracle.linear_bwd_weight, the restatement of
qwen3_moe_fused/functional.py:52-61; the product the reference's kernel computes is
qwen3_moe_fused/grouped_gemm/backward_dw.py:64-89), through the C ABI.  Every rank the entry takes (8, 16, 32,
64) meets the oracle on all experts, among them experts cut by a chunk border ("one": a single expert holds
every row and is cut by every border; "zipf": the hot experts span several chunks)."""
import numpy as np
import pytest
import torch

import oracle
from util import unit_scale_atol as _atol_np


def unit_scale_atol(ref, atol):
    return _atol_np(ref.detach().float().cpu().numpy(), atol)

pytestmark = pytest.mark.gpu


def _sizes(kind, E, R, gen):
    if kind == "uniform":
        idx = torch.randint(0, E, (R,), generator=gen)
    elif kind == "zipf":
        p = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.2
        p = p[torch.randperm(E, generator=gen)]
        idx = torch.multinomial(p / p.sum(), R, replacement=True, generator=gen)
    elif kind == "one":          # every row in one expert: cut by every border
        idx = torch.full((R,), E // 2)
    else:                        # "tiny": a few rows each, many experts per chunk, some empty
        idx = torch.randint(0, E, (R,), generator=gen)
        idx[idx % 3 == 0] = 1
    return torch.bincount(idx, minlength=E)


def _call(x, dy, ms, out_dtype, alpha=1.0):
    from qwen3_moe_fused import _lib
    R, K = x.shape
    N = dy.shape[1]
    E = ms.numel()
    lib = _lib.lib()
    ws_bytes = int(lib.mfl_gemm_dw_split_workspace(R, N, K, E))
    assert ws_bytes > 0
    # a dirty workspace and a dirty output: every element of dw is written, the workspace contents are ignored
    ws = torch.full((ws_bytes,), 0x7F, device=x.device, dtype=torch.uint8)
    out = torch.full((E, N, K), float("nan"), device=x.device, dtype=out_dtype)
    rc = lib.mfl_gemm_dw_split(_lib.ptr(x), _lib.ptr(dy), _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(out), R, N, K,
                               E, _lib.dtype_code(x.dtype), _lib.dtype_code(out_dtype), float(alpha), _lib.ptr(ws),
                               ws_bytes, _lib.stream())
    assert rc == 0, lib.mfl_strerror(rc)
    return out


def _closed_form(x, dy, ms, alpha):
    """alpha * dW of the CPU oracle on the same bf16-rounded inputs (rows past sum(ms) belong to no expert)."""
    counts = ms.cpu().numpy().astype(np.int64)
    rows = int(counts.sum())
    sel = oracle.sel_from_m_sizes(counts)
    ref = oracle.linear_bwd_weight(dy[:rows].float().cpu().numpy(), x[:rows].float().cpu().numpy(), sel, ms.numel())
    return torch.from_numpy(np.asarray(ref, dtype=np.float32) * np.float32(alpha)).to(x.device)


CASES = [
    # kind, E, R, N, K, m_sizes dtype, out dtype, alpha
    ("uniform", 8, 40, 16, 256, torch.int32, torch.bfloat16, 1.0),         # one chunk: nothing is cut
    ("uniform", 7, 3000, 16, 512, torch.int64, torch.bfloat16, 1.0),
    ("tiny", 130, 2500, 16, 256, torch.int32, torch.float32, 0.5),        # E not a multiple of 64
    ("zipf", 128, 20000, 16, 2048, torch.int32, torch.bfloat16, 2.0),     # dA of a rank-16 adapter
    ("zipf", 128, 20000, 768, 16, torch.int32, torch.bfloat16, 1.0),      # dB
    ("one", 5, 9000, 256, 16, torch.int32, torch.float32, 1.0),
    ("one", 3, 5000, 32, 256, torch.int32, torch.bfloat16, 1.0),          # rank 32
    ("zipf", 64, 12345, 512, 32, torch.int64, torch.bfloat16, 1.0),
    ("uniform", 512, 30000, 16, 768, torch.int32, torch.bfloat16, 1.0),    # the most experts the entry takes
    ("zipf", 48, 15000, 64, 1024, torch.int32, torch.bfloat16, 1.0),       # rank 64: two blocks of thin values
    ("tiny", 70, 6000, 512, 64, torch.int64, torch.float32, 0.25),
    ("zipf", 20, 7000, 8, 512, torch.int32, torch.bfloat16, 1.0),          # rank 8
    ("uniform", 9, 5000, 256, 8, torch.int32, torch.bfloat16, 2.0),
]


@pytest.mark.parametrize("kind,E,R,N,K,ms_dtype,out_dtype,alpha", CASES)
def test_dw_split_matches_closed_form(kind, E, R, N, K, ms_dtype, out_dtype, alpha):
    gen = torch.Generator().manual_seed(E * 1000 + R)
    ms = _sizes(kind, E, R, gen).to(ms_dtype).cuda()
    x = torch.randn(R, K, generator=gen).to(torch.bfloat16).cuda()
    dy = torch.randn(R, N, generator=gen).to(torch.bfloat16).cuda()
    print(f"dw_split {kind} E={E} R={R} N={N} K={K}", flush=True)
    got = _call(x, dy, ms, out_dtype, alpha)
    again = _call(x, dy, ms, out_dtype, alpha)
    torch.cuda.synchronize()
    assert torch.equal(got, again), "same bits from run to run"
    ref = _closed_form(x, dy, ms, alpha)
    assert not torch.isnan(got.float()).any()
    empty = (ms == 0).nonzero().flatten()
    assert (got[empty] == 0).all(), "experts without rows get exact zeros"
    # bf16 rounding of the result (2^-9 relative) on sums of R / E products of unit-scale values
    torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=unit_scale_atol(ref, 1e-2))


def test_dw_split_rows_past_the_sizes_are_ignored():
    gen = torch.Generator().manual_seed(5)
    E, R, N, K = 6, 5000, 16, 256
    ms = _sizes("uniform", E, R - 700, gen).int().cuda()       # 700 rows belong to no expert
    x = torch.randn(R, K, generator=gen).to(torch.bfloat16).cuda()
    dy = torch.randn(R, N, generator=gen).to(torch.bfloat16).cuda()
    x[R - 700:] = float("nan")
    got = _call(x, dy, ms, torch.float32)
    ref = _closed_form(x[:R - 700], dy[:R - 700], ms, 1.0)
    torch.testing.assert_close(got, ref, rtol=1e-2, atol=unit_scale_atol(ref, 1e-2))


def test_dw_split_refuses_other_shapes():
    from qwen3_moe_fused import _lib
    lib = _lib.lib()
    assert lib.mfl_gemm_dw_split_workspace(4096, 16, 2048 + 8, 8) == 0     # wide side not a multiple of 256
    assert lib.mfl_gemm_dw_split_workspace(4096, 16, 16, 8) == 0           # no wide side
    assert lib.mfl_gemm_dw_split_workspace(4096, 768, 2048, 8) == 0        # no thin side
    assert lib.mfl_gemm_dw_split_workspace(4096, 16, 2048, 513) == 0       # more experts than the tables hold
    x = torch.zeros(64, 264, dtype=torch.bfloat16, device="cuda")
    dy = torch.zeros(64, 16, dtype=torch.bfloat16, device="cuda")
    ms = torch.tensor([64], dtype=torch.int32, device="cuda")
    out = torch.zeros(1, 16, 264, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    rc = lib.mfl_gemm_dw_split(_lib.ptr(x), _lib.ptr(dy), _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(out), 64, 16,
                               264, 1, _lib.dtype_code(x.dtype), _lib.dtype_code(out.dtype), 1.0, _lib.ptr(ws), 1 << 20,
                               _lib.stream())
    assert rc == -6, lib.mfl_strerror(rc)   # MFL_ERR_UNSUPPORTED
    x = torch.zeros(64, 256, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(1, 16, 256, dtype=torch.bfloat16, device="cuda")
    rc = lib.mfl_gemm_dw_split(_lib.ptr(x), _lib.ptr(dy), _lib.ptr(ms), _lib.itype_code(ms.dtype), _lib.ptr(out), 64, 16,
                               256, 1, _lib.dtype_code(x.dtype), _lib.dtype_code(out.dtype), 1.0, _lib.ptr(ws), 16,
                               _lib.stream())
    assert rc == -5, lib.mfl_strerror(rc)   # MFL_ERR_WORKSPACE


def test_backward_dw_wrapper_takes_the_split_kernel_for_lora_shapes():
    from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw
    gen = torch.Generator().manual_seed(11)
    E, R = 32, 8192
    ms = _sizes("zipf", E, R, gen).int().cuda()
    x = torch.randn(R, 512, generator=gen).to(torch.bfloat16).cuda()
    t = torch.randn(R, 16, generator=gen).to(torch.bfloat16).cuda()
    got = grouped_gemm_backward_dw(x, t, ms, torch.bfloat16)
    ref = _closed_form(x, t, ms, 1.0)
    torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=unit_scale_atol(ref, 1e-2))
    # accumulate keeps the general kernel
    base = torch.ones_like(got)
    acc = grouped_gemm_backward_dw(x, t, ms, torch.bfloat16, out=base.clone(), accumulate=True)
    torch.testing.assert_close(acc.float(), ref + 1.0, rtol=2e-2, atol=unit_scale_atol(ref, 2e-2))


@pytest.mark.parametrize("seed", range(24))
def test_dw_split_random_shapes(seed):
    gen = torch.Generator().manual_seed(1000 + seed)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))  # noqa: E731
    E = ri(1, 200)
    R = ri(1, 12000)
    th = (8, 16, 32, 64)[ri(0, 3)]
    wide = 256 * ri(1, 4)
    thin_n = bool(ri(0, 1))
    N, K = (th, wide) if thin_n else (wide, th)
    kind = ("uniform", "zipf", "one", "tiny")[ri(0, 3)]
    ms = _sizes(kind, E, R, gen)
    if ri(0, 3) == 0:                      # rows at the end that belong to no expert
        ms[ri(0, E - 1)] = 0
    ms = ms.to((torch.int32, torch.int64)[ri(0, 1)]).cuda()
    out_dtype = (torch.bfloat16, torch.float32)[ri(0, 1)]
    x = torch.randn(R, K, generator=gen).to(torch.bfloat16).cuda()
    dy = torch.randn(R, N, generator=gen).to(torch.bfloat16).cuda()
    print(f"dw_split seed {seed}: {kind} E={E} R={R} N={N} K={K} {out_dtype} rows in experts {int(ms.sum())}", flush=True)
    got = _call(x, dy, ms, out_dtype, 1.0)
    ref = _closed_form(x, dy, ms, 1.0)
    assert (got[(ms == 0).nonzero().flatten()] == 0).all()
    torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=unit_scale_atol(ref, 1e-2))
