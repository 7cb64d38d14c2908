"""Shared helpers of the parity tests: seeded inputs, routing draws, error metrics."""
from __future__ import annotations

import numpy as np
import torch

import oracle

# bf16 GEMM tolerance: the reference's own criterion, allclose(rtol=1e-2, atol=1e-2)
# (test_moe_fused_linear.py:34-36,52), plus max|a-b| / max|ref| <= 1e-2.
BF16_RTOL = 1e-2
BF16_ATOL = 1e-2


def gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def randn(shape, g, scale=1.0, dtype=torch.float32):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def to_np32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def m_sizes_uniform(rows: int, E: int, g) -> torch.Tensor:
    """Per-expert counts of `rows` rows drawn uniformly over E experts (sorted batch)."""
    sel = torch.randint(0, E, (rows,), generator=g)
    return torch.bincount(sel, minlength=E).to(torch.int32)


def topk_routing(T: int, E: int, k: int, g, bias=None):
    """softmax -> top-k routing of T tokens; returns (sel (T*k,) int64, m_sizes int32)."""
    logits = torch.randn((T, E), generator=g)
    if bias is not None:
        logits = logits + bias
    sel = torch.topk(torch.softmax(logits, dim=-1), k, dim=-1).indices.reshape(-1)
    return sel, torch.bincount(sel, minlength=E).to(torch.int32)


def zipf_bias(E: int, s: float, g) -> torch.Tensor:
    """log-popularity of experts, p_e ~ rank^-s under a seeded random rank permutation."""
    ranks = torch.randperm(E, generator=g).float() + 1.0
    p = ranks.pow(-s)
    return (p / p.sum()).log()


def check_close(actual: torch.Tensor, expect: np.ndarray, rtol=BF16_RTOL, atol=BF16_ATOL, what=""):
    a = to_np32(actual).astype(np.float64)
    e = np.asarray(expect, dtype=np.float64)
    assert a.shape == e.shape, f"{what}: shape {a.shape} vs {e.shape}"
    assert np.isfinite(a).all(), f"{what}: non-finite values"
    diff = np.abs(a - e)
    scale = max(np.abs(e).max(), 1e-30) if e.size else 1.0
    norm_max = diff.max() / scale if e.size else 0.0
    ok = (diff <= atol + rtol * np.abs(e)).all()
    assert ok and norm_max <= rtol, (
        f"{what}: allclose={ok} normalised max err={norm_max:.3e} max abs err={diff.max():.3e} (ref max {scale:.3e})")
    return norm_max


def unit_scale_atol(expect: np.ndarray, atol=BF16_ATOL) -> float:
    """The absolute tolerance of the reference's tests, carried over to outputs that are not of unit scale.

    The reference draws weights with standard deviation 1 / sqrt(K) so that outputs have unit scale and
    atol = 1e-2 is one percent of it (test_moe_fused_linear.py:33-38).  For outputs of another scale the same
    one percent is atol * std(expect).  Used where the kernel does not reproduce the reference's rounded
    weights bit for bit: the decode-size NF4 kernel multiplies bf16(code) and applies absmax to a
    quantisation block's partial sum, the reference multiplies bf16(code * absmax); the two differ by
    rounding noise of a bf16 ulp per weight, which a sum over K elements turns into about 1e-3 of the
    output scale."""
    return atol * max(1.0, float(np.asarray(expect, dtype=np.float64).std()))


def oracle_rows(x: torch.Tensor, w: torch.Tensor, sel: np.ndarray, rows: np.ndarray) -> np.ndarray:
    """Oracle forward for a subset of rows (rows are independent)."""
    return oracle.linear_fwd(to_np32(x[rows]), to_np32(w), sel[rows])
