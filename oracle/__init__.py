"""CPU oracle for the moe_fused_linear hot path -- TEST INFRASTRUCTURE ONLY.

A numpy front end over ``oracle/moe_oracle.c`` (plain C, built by ``oracle/Makefile``)
plus the few compositions of the reference that are pure data flow (the sparse MoE
block, the LoRA expert MLP).  Nothing in the product package imports this module:
it is the checker used by ``tests/``, by the smoke check and by the benchmark's
``cpu_baseline`` leg.

Each function names the reference lines it restates; see the header of
``moe_oracle.c`` for which of them are pinned by independent checks and which are
"parity unpinned" (NF4 against bitsandbytes).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_i64p = ctypes.POINTER(ctypes.c_int64)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_u8p = ctypes.POINTER(ctypes.c_uint8)


def build(force: bool = False) -> str:
    """Compile moe_oracle.c with gcc (idempotent unless ``force``)."""
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.orc_num_threads.restype = ctypes.c_int
        _lib.orc_expert_counts_and_idx.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().orc_num_threads())


def _c(a: np.ndarray, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _p(a: np.ndarray, ptype):
    return a.ctypes.data_as(ptype)


# ----------------------------------------------------------------------------- bf16

def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern (uint16), round-to-nearest-even."""
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_bf16(_p(a, _f32p), _p(out, _u16p), ctypes.c_int64(a.size))
    return out


def from_bf16_bits(a: np.ndarray) -> np.ndarray:
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_bf16_to_f32(_p(a, _u16p), _p(out, _f32p), ctypes.c_int64(a.size))
    return out


def round_bf16(a: np.ndarray) -> np.ndarray:
    """fp32 values rounded to the nearest bf16, returned as fp32."""
    return from_bf16_bits(to_bf16_bits(a))


# ----------------------------------------------------------------------------- linear trio

def linear_fwd(x, w, sel) -> np.ndarray:
    """functional.py:7-33 -- out[b] = w[sel[b]] @ x[b]."""
    x, w, sel = _c(x, np.float32), _c(w, np.float32), _c(sel, np.int64)
    B, K = x.shape
    E, N, K2 = w.shape
    assert K2 == K and sel.shape == (B,)
    assert B == 0 or (sel.min() >= 0 and sel.max() < E)
    out = np.empty((B, N), np.float32)
    lib().orc_linear_fwd_f32(_p(x, _f32p), _p(w, _f32p), _p(sel, _i64p), _p(out, _f32p),
                             ctypes.c_int64(B), ctypes.c_int(N), ctypes.c_int(K))
    return out


def linear_bwd_input(dy, w, sel) -> np.ndarray:
    """functional.py:37-48 -- dx[b] = dy[b] @ w[sel[b]]."""
    dy, w, sel = _c(dy, np.float32), _c(w, np.float32), _c(sel, np.int64)
    B, N = dy.shape
    E, N2, K = w.shape
    assert N2 == N and sel.shape == (B,)
    assert B == 0 or (sel.min() >= 0 and sel.max() < E)
    dx = np.empty((B, K), np.float32)
    lib().orc_linear_bwd_input_f32(_p(dy, _f32p), _p(w, _f32p), _p(sel, _i64p), _p(dx, _f32p),
                                   ctypes.c_int64(B), ctypes.c_int(N), ctypes.c_int(K))
    return dx


def linear_bwd_weight(dy, x, sel, E: int) -> np.ndarray:
    """functional.py:52-61 -- dw[sel[b]] += outer(dy[b], x[b]), zeros elsewhere."""
    dy, x, sel = _c(dy, np.float32), _c(x, np.float32), _c(sel, np.int64)
    B, N = dy.shape
    B2, K = x.shape
    assert B2 == B and sel.shape == (B,)
    assert B == 0 or (sel.min() >= 0 and sel.max() < E)
    dw = np.empty((E, N, K), np.float32)
    lib().orc_linear_bwd_weight_f32(_p(dy, _f32p), _p(x, _f32p), _p(sel, _i64p), _p(dw, _f32p),
                                    ctypes.c_int64(B), ctypes.c_int(N), ctypes.c_int(K), ctypes.c_int(E))
    return dw


def sel_from_m_sizes(m_sizes) -> np.ndarray:
    """Rows grouped by expert ascending: the ``selected_experts`` that a sorted batch
    with these per-expert counts corresponds to (functional.py:64-79 contract)."""
    m = np.asarray(m_sizes, np.int64)
    return np.repeat(np.arange(m.size, dtype=np.int64), m)


# ----------------------------------------------------------------------------- sort

def expert_counts_and_idx(s, E: int):
    """kernels/indexing.py:48-65 -- returns (m_sizes, sort_idx, inv_sort_idx), all int32."""
    s = _c(s, np.int64)
    R = s.size
    counts = np.empty(E, np.int32)
    sort_idx = np.empty(R, np.int32)
    inv = np.empty(R, np.int32)
    rc = lib().orc_expert_counts_and_idx(_p(s, _i64p), ctypes.c_int64(R), ctypes.c_int(E),
                                         _p(counts, _i32p), _p(sort_idx, _i32p), _p(inv, _i32p))
    if rc != 0:
        raise ValueError("expert id outside [0, E)")
    return counts, sort_idx, inv


def expert_counts(s, E: int) -> np.ndarray:
    """kernels/indexing.py:18-23."""
    s = _c(s, np.int64)
    assert s.size == 0 or (s.min() >= 0 and s.max() < E)
    counts = np.empty(E, np.int32)
    lib().orc_expert_counts(_p(s, _i64p), ctypes.c_int64(s.size), ctypes.c_int(E), _p(counts, _i32p))
    return counts


# ----------------------------------------------------------------------------- routing

def softmax_topk(logits, k: int, renorm: bool):
    """modular_qwen3_moe_fused.py:87-91 -- fp32 softmax, top-k (descending, ties -> lower id),
    optional renormalisation.  Returns (weights fp32 (T,k), idx int64 (T,k))."""
    logits = _c(logits, np.float32)
    T, E = logits.shape
    assert 0 < k <= E
    w = np.empty((T, k), np.float32)
    idx = np.empty((T, k), np.int64)
    lib().orc_softmax_topk(_p(logits, _f32p), ctypes.c_int64(T), ctypes.c_int(E), ctypes.c_int(k),
                           ctypes.c_int(1 if renorm else 0), _p(w, _f32p), _p(idx, _i64p))
    return w, idx


# ----------------------------------------------------------------------------- silu-mul

def silu_mul_fwd_bf16(e_bits, g_bits) -> np.ndarray:
    """kernels/silu_mul.py:34-39 on bf16 bit patterns."""
    e, g = _c(e_bits, np.uint16), _c(g_bits, np.uint16)
    h = np.empty(e.shape, np.uint16)
    lib().orc_silu_mul_fwd_bf16(_p(e, _u16p), _p(g, _u16p), _p(h, _u16p), ctypes.c_int64(e.size))
    return h


def silu_mul_fwd_f32(e, g) -> np.ndarray:
    e, g = _c(e, np.float32), _c(g, np.float32)
    h = np.empty(e.shape, np.float32)
    lib().orc_silu_mul_fwd_f32(_p(e, _f32p), _p(g, _f32p), _p(h, _f32p), ctypes.c_int64(e.size))
    return h


def silu_mul_bwd_bf16(dh_bits, e_bits, g_bits):
    """kernels/silu_mul.py:62-73 (and :95-111 for h).  Returns (h, de, dg) bit patterns."""
    dh, e, g = _c(dh_bits, np.uint16), _c(e_bits, np.uint16), _c(g_bits, np.uint16)
    h, de, dg = (np.empty(e.shape, np.uint16) for _ in range(3))
    lib().orc_silu_mul_bwd_bf16(_p(dh, _u16p), _p(e, _u16p), _p(g, _u16p), _p(de, _u16p), _p(dg, _u16p),
                                _p(h, _u16p), ctypes.c_int64(e.size))
    return h, de, dg


def silu_mul_bwd_f32(dh, e, g):
    dh, e, g = _c(dh, np.float32), _c(e, np.float32), _c(g, np.float32)
    h, de, dg = (np.empty(e.shape, np.float32) for _ in range(3))
    lib().orc_silu_mul_bwd_f32(_p(dh, _f32p), _p(e, _f32p), _p(g, _f32p), _p(de, _f32p), _p(dg, _f32p),
                               _p(h, _f32p), ctypes.c_int64(e.size))
    return h, de, dg


# ----------------------------------------------------------------------------- NF4

def nf4_code() -> np.ndarray:
    out = np.empty(16, np.float32)
    lib().orc_nf4_code(_p(out, _f32p))
    return out


def nf4_quant(w, blocksize: int):
    """Blockwise NF4 quantiser (test-input generator).  Returns (packed uint8 (n/2,), absmax fp32)."""
    w = _c(w, np.float32).reshape(-1)
    assert w.size % blocksize == 0 and blocksize % 2 == 0
    q = np.empty(w.size // 2, np.uint8)
    absmax = np.empty(w.size // blocksize, np.float32)
    lib().orc_nf4_quant_f32(_p(w, _f32p), ctypes.c_int64(w.size), ctypes.c_int(blocksize), _p(q, _u8p),
                            _p(absmax, _f32p))
    return q, absmax


def nf4_dequant(q, absmax, blocksize: int, code=None, bf16: bool = False) -> np.ndarray:
    """grouped_gemm/forward_4bit.py:99-104.  fp32 values, or bf16 bit patterns when ``bf16``."""
    q, absmax = _c(q, np.uint8).reshape(-1), _c(absmax, np.float32).reshape(-1)
    code = nf4_code() if code is None else _c(code, np.float32)
    n = q.size * 2
    assert absmax.size * blocksize == n
    if bf16:
        out = np.empty(n, np.uint16)
        lib().orc_nf4_dequant_bf16(_p(q, _u8p), _p(code, _f32p), _p(absmax, _f32p), ctypes.c_int(blocksize),
                                   ctypes.c_int64(n), _p(out, _u16p))
    else:
        out = np.empty(n, np.float32)
        lib().orc_nf4_dequant_f32(_p(q, _u8p), _p(code, _f32p), _p(absmax, _f32p), ctypes.c_int(blocksize),
                                  ctypes.c_int64(n), _p(out, _f32p))
    return out


def dequant_blockwise_u8(v, code256, absmax2, blocksize2: int, offset: float) -> np.ndarray:
    """grouped_gemm/forward_4bit.py:149-152 (nested absmax)."""
    v, code256, absmax2 = _c(v, np.uint8).reshape(-1), _c(code256, np.float32), _c(absmax2, np.float32)
    out = np.empty(v.size, np.float32)
    lib().orc_dequant_blockwise_u8(_p(v, _u8p), _p(code256, _f32p), _p(absmax2, _f32p), ctypes.c_int(blocksize2),
                                   ctypes.c_float(offset), ctypes.c_int64(v.size), _p(out, _f32p))
    return out


# ----------------------------------------------------------------------------- compositions

def moe_block_fwd(hidden, gate_w, w_gate, w_up, w_down, k: int, renorm: bool, act_round=None):
    """modular_qwen3_moe_fused.py:79-118 -- router -> top-k -> sort -> gate/up -> SiLU*mul -> down
    -> un-sort -> weighted sum over k.  fp32 throughout; ``act_round`` (e.g. ``round_bf16``) is
    applied where the reference's bf16 run materialises a tensor.
    Returns (out (T,H), router_logits (T,E))."""
    rnd = (lambda a: a) if act_round is None else act_round
    hidden = _c(hidden, np.float32)
    T, H = hidden.shape
    E = w_gate.shape[0]
    logits = rnd(hidden.astype(np.float64) @ _c(gate_w, np.float32).astype(np.float64).T).astype(np.float32)
    rw, sel = softmax_topk(logits, k, renorm)
    rw = rnd(rw)
    sel_flat = sel.reshape(-1)
    m_sizes, sort_idx, inv_sort_idx = expert_counts_and_idx(sel_flat, E)
    xs = np.repeat(hidden, k, axis=0)[sort_idx]                 # :95-103
    sel_sorted = sel_from_m_sizes(m_sizes)
    e = rnd(linear_fwd(xs, w_gate, sel_sorted))                 # :105
    g = rnd(linear_fwd(xs, w_up, sel_sorted))                   # :106
    h = rnd(rnd(e / (1.0 + np.exp(-e.astype(np.float64))).astype(np.float32)) * g)   # :108
    y = rnd(linear_fwd(h, w_down, sel_sorted))                  # :110
    y = y[inv_sort_idx].reshape(T, k, H)                        # :112-114
    out = rnd(np.einsum("beo,be->bo", y.astype(np.float64), rw.astype(np.float64)).astype(np.float32))
    return out, logits


def lora_linear_fwd(x, w, a, b, scale: float, sel) -> np.ndarray:
    """lora.py:134 -- base(x) + lora_B(lora_A(x)) * scaling, per-row expert ``sel``."""
    return linear_fwd(x, w, sel) + np.float32(scale) * linear_fwd(linear_fwd(x, a, sel), b, sel)


def lora_mlp_fwd_bwd(x, G, Ag, Bg, Sg, U, Au, Bu, Su, W, Aw, Bw, Sw, sel, dy, act_round=None):
    """kernels/fast_lora.py:3-46 (the formulas) and :68-172 (what is materialised) -- the expert MLP
    with LoRA on its three projections, forward and every gradient the reference returns:

        e = G'x, g = U'x, h = silu(e) g, y = W'h          with P' = P + S * B A per projection
        dh = dy W',  (h, de, dg) = silu_mul_bwd(dh, e, g),  dx = de G' + dg U'
        dA = S (dOut B)^T In,  dB = S dOut^T (In A^T)     per projection (Out = P' In)

    ``act_round`` (e.g. ``round_bf16``) is applied where the reference's low-precision run
    materialises a tensor (:96-99, :133-152).  Returns a dict of fp32 arrays."""
    rnd = (lambda a: a) if act_round is None else act_round
    f = np.float32

    def proj(inp, P, A, B, S):                     # mv_lora, fast_lora.py:90-94
        u = rnd(linear_fwd(inp, A, sel))
        return rnd(rnd(linear_fwd(inp, P, sel)) + f(S) * rnd(linear_fwd(u, B, sel))), u

    def proj_t(dout, P, A, B, S):                  # vm_lora, fast_lora.py:127-131
        t = rnd(linear_bwd_input(dout, B, sel))
        return rnd(rnd(linear_bwd_input(dout, P, sel)) + f(S) * rnd(linear_bwd_input(t, A, sel))), t

    E = G.shape[0]
    e, ug = proj(x, G, Ag, Bg, Sg)
    g, uu = proj(x, U, Au, Bu, Su)
    h = rnd(silu_mul_fwd_f32(e, g)) if act_round is None else from_bf16_bits(
        silu_mul_fwd_bf16(to_bf16_bits(e), to_bf16_bits(g)))
    y, uw = proj(h, W, Aw, Bw, Sw)
    dh, tw = proj_t(dy, W, Aw, Bw, Sw)
    if act_round is None:
        h2, de, dg = silu_mul_bwd_f32(dh, e, g)
    else:
        h2, de, dg = (from_bf16_bits(a) for a in silu_mul_bwd_bf16(to_bf16_bits(dh), to_bf16_bits(e), to_bf16_bits(g)))
    tg = rnd(linear_bwd_input(de, Bg, sel))
    tu = rnd(linear_bwd_input(dg, Bu, sel))
    out = {
        "y": y, "e": e, "g": g, "h": h,
        "dAw": f(Sw) * linear_bwd_weight(tw, h2, sel, E), "dBw": f(Sw) * linear_bwd_weight(dy, uw, sel, E),
        "dAu": f(Su) * linear_bwd_weight(tu, x, sel, E), "dBu": f(Su) * linear_bwd_weight(dg, uu, sel, E),
        "dAg": f(Sg) * linear_bwd_weight(tg, x, sel, E), "dBg": f(Sg) * linear_bwd_weight(de, ug, sel, E),
    }
    dx = linear_bwd_input(de, G, sel) + f(Sg) * linear_bwd_input(tg, Ag, sel)
    dx = dx + linear_bwd_input(dg, U, sel) + f(Su) * linear_bwd_input(tu, Au, sel)
    out["dx"] = dx
    return out
