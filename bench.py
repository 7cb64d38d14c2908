#!/usr/bin/env python3
"""Benchmark of the moe_fused_linear hot path on one MI355X.

A step is one forward grouped GEMM over one synthetic batch at benchmark configuration 2
(Qwen3-30B-A3B gate_proj: 128 experts, weight (128, 768, 2048) bf16, 4096 tokens routed
top-8 -> 32768 rows sorted by expert).  Inputs are resident in HBM before the timed region.
One JSON line is printed.  The metric names forward, dX and dW: the forward product is the timed
step ("value"), dX and dW at config 3 are first-class fields beside it ("dx", "dw"), and the
bandwidth-bound neighbours are reported under "extra" from separate short timed loops.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "transformers-qwen3-moe-fused_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# HBM bytes per launch of the benchmarked kernel: not measured by this run but taken from the FETCH_SIZE /
# WRITE_SIZE counter passes summarised in profiles/gemm_fwd_gate_proj_config2_hbm_traffic.txt
# (537.6 MB read + 57.7 MB written); the JSON line names that file as the source
MEASURED_TRAFFIC_BYTES = 595.3e6
TRAFFIC_SOURCE = "profiles/gemm_fwd_gate_proj_config2_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not this run)"
# A burst of back-to-back launches starts in a transient of the board's power management (boost clocks for
# the first ten launches, a dip around launch 20, settled after about 150): every timed loop is preceded by
# at least this many untimed launches, whatever --warmup says.
MIN_WARMUP = 200

E, HIDDEN, INTER, TOKENS, TOPK = 128, 2048, 768, 4096, 8
ROWS = TOKENS * TOPK


def _event_us(fn, iters, warm, stream):
    import torch

    for i in range(warm):
        fn(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record(stream)
    for i in range(iters):
        fn(i)
    stop.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e3 / iters


def _event_us_median(fn, iters, warm, stream, blocks=5):
    """Median over `blocks` timed runs of `iters` calls each: calls that are bound by the host (a few
    microseconds of GPU work per launch) now and then hit a one-off stall of tens of milliseconds in a
    long loop, which a single mean would spread over every call."""
    runs = sorted(_event_us(fn, iters, warm if b == 0 else 0, stream) for b in range(blocks))
    return runs[len(runs) // 2]


def _per_launch_us(fn, iters, warm, stream):
    """Time of every launch of a loop by its own pair of events: (median, 20 % quantile, 80 % quantile), the
    figures the reference's benchmarks report (do_bench(quantiles=[0.5, 0.2, 0.8]),
    benchmark_moe_fused_linear.py:56-59)."""
    import torch

    for i in range(warm):
        fn(i)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(evs):
        a.record(stream)
        fn(i)
        b.record(stream)
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
    return ts[len(ts) // 2], ts[len(ts) // 5], ts[len(ts) * 4 // 5]


def _reference_sweep(dev, stream, ws, qsets):
    """The reference's own benchmark definition (benchmark_moe_fused_linear.py:27-28,43-61, _bwd_dx.py:44-60,
    _bwd_dw.py:42-58, _4bit.py:51-69): rows 1024 ... 16384 in steps of 1024, every row's expert drawn
    uniformly, in_features 2048, out_features 768, 128 experts, bf16; forward, input gradient, weight gradient
    and the 4-bit forward.  Per point: median and 20 / 80 % quantiles over per-launch event times, TFLOP/s
    (two flops per multiply-add), and the fraction of the 8 TB/s HBM peak that the algorithmic bytes of the
    point (each operand read once, the output written once) amount to at the median."""
    import torch

    from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw
    from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward
    from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_4bit
    from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed
    from qwen3_moe_fused.grouped_gemm.fused import grouped_glu_forward_4bit

    NB = len(ws)
    g = torch.Generator().manual_seed(1)
    rmax = 16384
    x = torch.randn((rmax, HIDDEN), device=dev, dtype=torch.bfloat16)
    dy = torch.randn((rmax, INTER), device=dev, dtype=torch.bfloat16)
    points = []
    wbytes = 2.0 * E * INTER * HIDDEN
    iters, warm = 60, 20
    # one long untimed burst first: the board's power management settles after about 150 launches
    ms0 = torch.bincount(torch.randint(0, E, (rmax,), generator=g), minlength=E).to(torch.int32).to(dev)
    for i in range(MIN_WARMUP):
        grouped_gemm_forward(x, ws[i % NB], ms0)
    for rows in range(1024, rmax + 1, 1024):
        ms = torch.bincount(torch.randint(0, E, (rows,), generator=g), minlength=E).to(torch.int32).to(dev)
        xr, dyr = x[:rows], dy[:rows]
        flop = 2.0 * rows * INTER * HIDDEN
        io = 2.0 * rows * (HIDDEN + INTER)
        legs = {
            "fwd": (lambda i: grouped_gemm_forward(xr, ws[i % NB], ms), io + wbytes),
            "dx": (lambda i: grouped_gemm_forward_transposed(dyr, ws[i % NB], ms), io + wbytes),
            "dw": (lambda i: grouped_gemm_backward_dw(xr, dyr, ms, torch.bfloat16), io + wbytes),
            "fwd_4bit": (lambda i: grouped_gemm_forward_4bit(xr, *qsets[i % NB], ms),
                         io + E * INTER * HIDDEN * (0.5 + 4.0 / 64)),
            # not one of the reference's benchmarks: gate and up projection with packed weights and SiLU-mul in one
            # launch, as the sparse block's front half runs them (twice the flops of the other legs)
            "glu_4bit": (lambda i: grouped_glu_forward_4bit(xr, *qsets[i % NB], *qsets[(i + 1) % NB], ms),
                         io + 2 * E * INTER * HIDDEN * (0.5 + 4.0 / 64)),
        }
        point = {"rows": rows}
        for name, (fn, nbytes) in legs.items():
            med, q20, q80 = _per_launch_us(fn, iters, warm, stream)
            fl = 2 * flop if name == "glu_4bit" else flop
            point[name] = {"us": round(med, 1), "us_q20": round(q20, 1), "us_q80": round(q80, 1),
                           "tflops": round(fl / med / 1e6, 1), "gbs": round(nbytes / med / 1e3, 1),
                           "hbm_frac": round(nbytes / med / 1e3 / PEAK_HBM_GBS, 4)}
        points.append(point)
    # largest step in achieved GB/s between neighbouring points, per product (a cliff marks a bad switch of
    # tile configurations)
    jumps = {}
    for name in ("fwd", "dx", "dw", "fwd_4bit"):
        gb = [p[name]["gbs"] for p in points]
        jumps[name] = round(max(abs(b - a) / max(a, b) for a, b in zip(gb, gb[1:])), 3)
    return {"definition": "rows 1024..16384 step 1024, uniform random experts, in 2048, out 768, 128 experts, bf16; "
                          "median / 20 % / 80 % of 60 per-launch event times after 20 warm launches; "
                          "three weight sets in rotation",
            "points": points, "largest_neighbour_step_in_gbs": jumps}


def _kernel_tour(n, dev):
    """N launches of each hot kernel at the shapes of configurations 2, 3 and 5, in a fixed order, with a line
    per kernel that states its algorithmic bytes and flops per launch.  Nothing is timed: counter passes
    (rocprofv3 --pmc) and kernel traces are taken over this."""
    import torch

    from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw
    from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward
    from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_4bit
    from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed
    from qwen3_moe_fused.grouped_gemm.fused import grouped_glu_forward, grouped_glu_forward_4bit
    from qwen3_moe_fused.kernels.indexing import get_expert_counts_and_idx
    from qwen3_moe_fused.kernels.routing import combine_rows, gather_rows, route_and_sort, softmax_topk_raw
    from qwen3_moe_fused.kernels.silu_mul import silu_mul_backward, silu_mul_forward
    from qwen3_moe_fused.quantize.nf4 import dequantize_nf4, quantize_nf4

    g = torch.Generator(device=dev).manual_seed(0)
    bf = torch.bfloat16

    def rnd(*shape, scale=1.0):
        return (torch.randn(shape, device=dev, generator=g) * scale).to(bf)

    logits = torch.randn((TOKENS, E), device=dev, generator=g)
    _, rw, sel = softmax_topk_raw(logits, TOPK, True, bf)
    m_sizes, sort_idx, inv_sort_idx = get_expert_counts_and_idx(sel.view(-1), E)
    hidden = rnd(TOKENS, HIDDEN)
    x = rnd(ROWS, HIDDEN)
    w_gate, w_up = rnd(E, INTER, HIDDEN, scale=0.02), rnd(E, INTER, HIDDEN, scale=0.02)
    w_down = rnd(E, HIDDEN, INTER, scale=0.02)
    h, h2, dh = rnd(ROWS, INTER), rnd(ROWS, INTER), rnd(ROWS, INTER)
    dy = rnd(ROWS, HIDDEN)
    # three packed weight sets in rotation: one set (113 MB) would stay in the 256 MB MALL between launches
    qsets = [quantize_nf4(w, 64) for w in (w_gate, w_up, rnd(E, INTER, HIDDEN, scale=0.02))]
    packed, qstate = qsets[0]
    gemm_b = 2.0 * (ROWS * HIDDEN + E * INTER * HIDDEN + ROWS * INTER)
    gemm_f = 2.0 * ROWS * INTER * HIDDEN
    nf4_b = E * INTER * HIDDEN * (0.5 + 4.0 / 64)
    legs = [
        ("gemm_fwd gate_proj 4096 tokens", gemm_b, gemm_f, lambda i: grouped_gemm_forward(x, w_gate, m_sizes)),
        ("gemm_dx down_proj 4096 tokens", gemm_b, gemm_f, lambda i: grouped_gemm_forward_transposed(dy, w_down, m_sizes)),
        ("gemm_dw down_proj 4096 tokens", gemm_b, gemm_f, lambda i: grouped_gemm_backward_dw(h, dy, m_sizes, bf)),
        ("gemm_fwd down_proj 4096 tokens", gemm_b, gemm_f, lambda i: grouped_gemm_forward(h, w_down, m_sizes)),
        ("glu_fwd (gather + gate + up + SiLU-mul) 4096 tokens",
         2.0 * (TOKENS * HIDDEN + 2 * E * INTER * HIDDEN + ROWS * INTER), 2 * gemm_f,
         lambda i: grouped_glu_forward(hidden, w_gate, w_up, m_sizes, sort_idx, TOPK)),
        ("silu_mul_fwd 32768 rows", 3.0 * ROWS * INTER * 2, 0.0, lambda i: silu_mul_forward(h, h2)),
        ("silu_mul_bwd 32768 rows", 5.0 * ROWS * INTER * 2, 0.0, lambda i: silu_mul_backward(dh, h, h2)),
        ("gather_rows 4096 tokens (scatter form)", 2.0 * (TOKENS + ROWS) * HIDDEN, 0.0,
         lambda i: gather_rows(hidden, sort_idx, TOPK, inv_sort_idx)),
        ("combine_rows 4096 tokens", 2.0 * (TOKENS + ROWS) * HIDDEN, 0.0,
         lambda i: combine_rows(dy, inv_sort_idx, rw, sort_idx)),
        ("softmax_topk 4096 tokens", TOKENS * E * 4.0 + TOKENS * TOPK * (4 + 2 + 8), 0.0,
         lambda i: softmax_topk_raw(logits, TOPK, True, bf)),
        ("expert_sort 32768 rows", ROWS * 8.0 + 2 * ROWS * 4 + E * 4, 0.0,
         lambda i: get_expert_counts_and_idx(sel.view(-1), E)),
        ("route_and_sort 4096 tokens (top-k that counts + scatter)",
         TOKENS * E * 4.0 + TOKENS * TOPK * (4 + 2 + 8) + 2 * ROWS * 4 + E * 4, 0.0,
         lambda i: route_and_sort(logits, TOPK, True, bf, E)),
        ("nf4_dequant gate_proj", nf4_b + 2.0 * E * INTER * HIDDEN, 0.0, lambda i: dequantize_nf4(*qsets[i % 3], bf)),
    ]
    for tokens in (16, 256, 16384):
        lgt = torch.randn((tokens, E), device=dev, generator=g)
        _, _, s5 = softmax_topk_raw(lgt, TOPK, True, bf)
        ms5, _, _ = get_expert_counts_and_idx(s5.view(-1), E)
        x5 = rnd(tokens * TOPK, HIDDEN)
        active = int((ms5 > 0).sum().item())
        legs.append((f"gemm_fwd_nf4 gate_proj {tokens} tokens ({active} experts hit)",
                     active * nf4_b / E + 2.0 * tokens * TOPK * (HIDDEN + INTER), 2.0 * tokens * TOPK * INTER * HIDDEN,
                     lambda i, x5=x5, ms5=ms5: grouped_gemm_forward_4bit(x5, *qsets[i % 3], ms5)))
        if tokens == 16384:
            legs.append(("gemm_fwd gate_proj 16384 tokens (131072 rows, 256 x 256 tiles)",
                         2.0 * (tokens * TOPK * (HIDDEN + INTER) + E * INTER * HIDDEN),
                         2.0 * tokens * TOPK * INTER * HIDDEN,
                         lambda i, x5=x5, ms5=ms5: grouped_gemm_forward(x5, w_gate, ms5)))
        if tokens <= 256:
            legs.append((f"glu_fwd_nf4 (gate + up + SiLU-mul) {tokens} tokens ({active} experts hit)",
                         2 * active * nf4_b / E + 2.0 * tokens * TOPK * (HIDDEN + INTER),
                         4.0 * tokens * TOPK * INTER * HIDDEN,
                         lambda i, x5=x5, ms5=ms5: grouped_glu_forward_4bit(x5, *qsets[i % 3], *qsets[(i + 1) % 3], ms5)))
    # the middle of the reference's row sweep (1024 tokens, 64 rows per expert): packed weights on the streaming
    # kernel's 64-row tiles, and the input gradient whose output is 2048 wide (192 x 256 tiles)
    lgt = torch.randn((1024, E), device=dev, generator=g)
    _, _, s6 = softmax_topk_raw(lgt, TOPK, True, bf)
    ms6, _, _ = get_expert_counts_and_idx(s6.view(-1), E)
    x6, dy6 = rnd(1024 * TOPK, HIDDEN), rnd(1024 * TOPK, INTER)
    io6 = 2.0 * 1024 * TOPK * (HIDDEN + INTER)
    legs += [
        ("gemm_fwd_nf4 gate_proj 1024 tokens (64-row tiles)", nf4_b + io6, 2.0 * 1024 * TOPK * INTER * HIDDEN,
         lambda i: grouped_gemm_forward_4bit(x6, *qsets[i % 3], ms6)),
        ("glu_fwd_nf4 (gate + up + SiLU-mul) 1024 tokens (64-row tiles)", 2 * nf4_b + io6,
         4.0 * 1024 * TOPK * INTER * HIDDEN,
         lambda i: grouped_glu_forward_4bit(x6, *qsets[i % 3], *qsets[(i + 1) % 3], ms6)),
        ("gemm_dx gate_proj 1024 tokens (output 2048 wide, 192 x 256 tiles)", 2.0 * E * INTER * HIDDEN + io6,
         2.0 * 1024 * TOPK * INTER * HIDDEN, lambda i: grouped_gemm_forward_transposed(dy6, w_gate, ms6)),
    ]
    # configuration 4: rank-16 adapter products at 8192 tokens under Zipf(1.2)-skewed routing (65536 rows)
    from qwen3_moe_fused.grouped_gemm.fused import grouped_gemm_forward_lora
    T4, R4, RANK = 8192, 8192 * TOPK, 16
    bias = (torch.randperm(E, device=dev, generator=g).float() + 1).pow(-1.2).log()
    _, _, s4 = softmax_topk_raw(torch.randn((T4, E), device=dev, generator=g) + bias, TOPK, True, bf)
    ms4, _, _ = get_expert_counts_and_idx(s4.view(-1), E)
    x4, dy4 = rnd(R4, HIDDEN), rnd(R4, INTER)
    t4, u4 = rnd(R4, RANK), rnd(R4, RANK)
    la, lb = rnd(E, RANK, HIDDEN, scale=0.01), rnd(E, INTER, RANK, scale=0.01)
    legs += [
        (f"gemm_dw_split dA (x 65536x2048, rank 16; largest expert {int(ms4.max().item())} rows)",
         2.0 * (R4 * HIDDEN + R4 * RANK + E * RANK * HIDDEN), 2.0 * R4 * RANK * HIDDEN,
         lambda i: grouped_gemm_backward_dw(x4, t4, ms4, bf)),
        ("gemm_dw_split dB (dy 65536x768, rank 16)", 2.0 * (R4 * INTER + R4 * RANK + E * RANK * INTER),
         2.0 * R4 * RANK * INTER, lambda i: grouped_gemm_backward_dw(u4, dy4, ms4, bf)),
        ("gemm_fwd thin output x A^T (65536x2048 -> rank 16)", 2.0 * (R4 * HIDDEN + R4 * RANK + E * RANK * HIDDEN),
         2.0 * R4 * RANK * HIDDEN, lambda i: grouped_gemm_forward(x4, la, ms4)),
        ("gemm_dx thin output dy B (65536x768 -> rank 16)", 2.0 * (R4 * INTER + R4 * RANK + E * RANK * INTER),
         2.0 * R4 * RANK * INTER, lambda i: grouped_gemm_forward_transposed(dy4, lb, ms4)),
        ("gemm_fwd_lora gate_proj + rank-16 term, 65536 rows",
         2.0 * (R4 * HIDDEN + E * INTER * HIDDEN + R4 * INTER + R4 * RANK + E * INTER * RANK),
         2.0 * R4 * INTER * (HIDDEN + RANK), lambda i: grouped_gemm_forward_lora(x4, w_gate, u4, lb, ms4)),
    ]
    for name, nbytes, flops, fn in legs:
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        print(f"{name}: {n} launches, algorithmic {nbytes / 1e6:.1f} MB, {flops / 1e9:.2f} GFLOP per launch", flush=True)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing (profiling runs)")
    ap.add_argument("--no-extra", action="store_true", help="time the forward GEMM only (profiling runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run plain 512 MiB device copies instead (reference reading for the FETCH_SIZE / "
                         "WRITE_SIZE counters of a profiling pass)")
    ap.add_argument("--kernel-tour", type=int, default=0, metavar="N",
                    help="launch every hot kernel N times at the benchmark shapes, untimed, and exit "
                         "(the program behind the per-kernel counter passes)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from qwen3_moe_fused import _lib
    from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw
    from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward
    from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_4bit
    from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed
    from qwen3_moe_fused.kernels.indexing import get_expert_counts_and_idx
    from qwen3_moe_fused.kernels.routing import softmax_topk_raw
    from qwen3_moe_fused.kernels.silu_mul import silu_mul_forward
    from qwen3_moe_fused.quantize.nf4 import dequantize_nf4, quantize_nf4

    _lib.lib()  # fail loudly when the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()

    if args.copy_calibration:
        src = torch.ones(256 * 1024 * 1024, device=dev, dtype=torch.bfloat16)   # 512 MiB
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": src.numel() * 2, "bytes_written": src.numel() * 2,
                                               "launches": 5}}))
        return 0

    if args.kernel_tour > 0:
        _kernel_tour(args.kernel_tour, dev)
        return 0

    # ---- synthetic inputs of config 2 (seeded on the CPU, then copied)
    g = torch.Generator().manual_seed(0)
    logits = torch.randn((TOKENS, E), generator=g)
    x0 = torch.randn((ROWS, HIDDEN), generator=g).to(torch.bfloat16)
    w0 = (torch.randn((E, INTER, HIDDEN), generator=g) * 0.02).to(torch.bfloat16)
    _, _, sel = softmax_topk_raw(logits.to(dev), TOPK, True, torch.bfloat16)
    m_sizes, sort_idx, inv_sort_idx = get_expert_counts_and_idx(sel.view(-1), E)
    # three rotating copies: the 403 MB weight stream must come from HBM, not from the 256 MB MALL
    NB = 3
    xs = [x0.to(dev)] + [x0.to(dev).clone() for _ in range(NB - 1)]
    ws = [w0.to(dev)] + [w0.to(dev).clone() for _ in range(NB - 1)]
    ys = [torch.empty((ROWS, INTER), device=dev, dtype=torch.bfloat16) for _ in range(NB)]

    def step(i):
        grouped_gemm_forward(xs[i % NB], ws[i % NB], m_sizes, out=ys[i % NB])

    warmup_effective = max(args.warmup, MIN_WARMUP)
    for i in range(warmup_effective):
        step(i)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_us = ev0.elapsed_time(ev1) * 1e3 / args.steps

    flop = 2.0 * ROWS * INTER * HIDDEN                              # 103.08 GFLOP
    alg_bytes = 2.0 * (ROWS * HIDDEN + E * INTER * HIDDEN + ROWS * INTER)   # 587.2 MB: x + w + y, once each
    ms_per_step = wall * 1e3 / args.steps
    tflops = flop * args.steps / wall / 1e12
    achieved_gbs = alg_bytes / (kernel_us * 1e-6) / 1e9

    out = {
        "metric": "bf16 grouped-GEMM TFLOP/s fwd/dX/dW at 30B-A3B MoE shapes + % MFMA peak",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_effective": warmup_effective,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: Qwen3-30B-A3B gate_proj forward grouped GEMM", "experts": E,
                   "rows": ROWS, "in_features": HIDDEN, "out_features": INTER, "tokens": TOKENS, "top_k": TOPK,
                   "routing": "softmax top-8 of N(0,1) logits, rows sorted by expert"},
        "roofline": {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved_gbs / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel_us": round(kernel_us, 2), "algorithmic_bytes": alg_bytes,
                     "mfma_tflops": round(flop / kernel_us / 1e6, 1),
                     "mfma_frac": round(flop / kernel_us / 1e6 / PEAK_BF16_TFLOPS, 4)},
    }

    # ---- the other two products of the metric, at config 3 (down_proj backward), same method: rotating buffer
    # sets, MIN_WARMUP untimed launches, then args.steps timed ones between two events
    dys = [torch.randn((ROWS, HIDDEN), device=dev, dtype=torch.bfloat16) for _ in range(NB)]   # grad of down_proj out
    hs = [torch.randn((ROWS, INTER), device=dev, dtype=torch.bfloat16) for _ in range(NB)]     # down_proj input
    wd = [w.view(E, HIDDEN, INTER) for w in ws]                                                # (128, 2048, 768)
    dxs = [torch.empty((ROWS, INTER), device=dev, dtype=torch.bfloat16) for _ in range(NB)]
    dws = [torch.empty((E, HIDDEN, INTER), device=dev, dtype=torch.bfloat16) for _ in range(NB)]

    def product_line(us):
        return {"us": round(us, 2), "tflops": round(flop / us / 1e6, 1),
                "mfma_frac": round(flop / us / 1e6 / PEAK_BF16_TFLOPS, 4),
                "hbm_gbs": round(alg_bytes / us / 1e3, 1), "hbm_frac": round(alg_bytes / us / 1e3 / PEAK_HBM_GBS, 4),
                "algorithmic_bytes": alg_bytes, "steps": args.steps, "warmup_effective": warmup_effective}

    us = _event_us(lambda i: grouped_gemm_forward_transposed(dys[i % NB], wd[i % NB], m_sizes, out=dxs[i % NB]),
                   args.steps, warmup_effective, stream)
    out["dx"] = dict(workload="configs[2]: down_proj input gradient, dy (32768, 2048) x w (128, 2048, 768)",
                     **product_line(us))
    us = _event_us(lambda i: grouped_gemm_backward_dw(hs[i % NB], dys[i % NB], m_sizes, torch.bfloat16,
                                                      out=dws[i % NB]), args.steps, warmup_effective, stream)
    out["dw"] = dict(workload="configs[2]: down_proj weight gradient, x (32768, 768), dy (32768, 2048)",
                     **product_line(us))
    out["fwd"] = dict(workload="configs[1]: gate_proj forward (the timed step)", **product_line(kernel_us))
    del dws, dxs

    if not args.no_extra:
        extra = {}
        it, wm = 50, MIN_WARMUP
        # the forward product with the replicate-and-sort folded into its operand load (rows gathered from the
        # 4096 token rows): 470 MB algorithmic instead of 587 MB
        from qwen3_moe_fused.grouped_gemm.fused import grouped_gemm_forward_gathered
        toks = [torch.randn((TOKENS, HIDDEN), device=dev, dtype=torch.bfloat16) for _ in range(NB)]
        us = _event_us(lambda i: grouped_gemm_forward_gathered(toks[i % NB], sort_idx, TOPK, ws[i % NB], m_sizes),
                       it, wm, stream)
        gb = 2.0 * (TOKENS * HIDDEN + E * INTER * HIDDEN + ROWS * INTER) + ROWS * 4
        extra["fwd_gate_proj_gathered"] = {"us": round(us, 1), "tflops": round(flop / us / 1e6, 1),
                                           "mfma_frac": round(flop / us / 1e6 / PEAK_BF16_TFLOPS, 4),
                                           "algorithmic_bytes": gb, "hbm_frac": round(gb / us / 1e3 / PEAK_HBM_GBS, 4)}
        del toks
        # the down projection's forward product (N = 2048, K = 768): same flops and bytes as gate_proj
        us = _event_us(lambda i: grouped_gemm_forward(hs[i % NB], wd[i % NB], m_sizes, out=dys[i % NB]), args.steps,
                       wm, stream)
        extra["fwd_down_proj"] = dict(workload="down_proj forward, h (32768, 768) x w (128, 2048, 768)",
                                      **product_line(us))
        us = _event_us(lambda i: silu_mul_forward(hs[i % NB], hs[(i + 1) % NB]), it, wm, stream)
        b = 3.0 * ROWS * INTER * 2
        extra["silu_mul_fwd"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / PEAK_HBM_GBS, 4)}
        selv = sel.view(-1)
        us = _event_us(lambda i: get_expert_counts_and_idx(selv, E), it, wm, stream)
        b = ROWS * 8 + 2 * ROWS * 4 + E * 4
        extra["expert_sort_32768"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 2)}
        lg = logits.to(dev)
        us = _event_us(lambda i: softmax_topk_raw(lg, TOPK, True, torch.bfloat16), it, wm, stream)
        b = TOKENS * E * 4 + TOKENS * TOPK * (4 + 2 + 8)
        extra["softmax_topk_4096"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 2)}
        # both as the block calls them: one library call (two launches), one allocation; eager calls are bound
        # by the host side of the call, the graph replay is the GPU side
        from qwen3_moe_fused.kernels.routing import route_and_sort
        with torch.no_grad():
            us = _event_us(lambda i: route_and_sort(lg, TOPK, True, torch.bfloat16, E), it, wm, stream)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                route_and_sort(lg, TOPK, True, torch.bfloat16, E)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                route_and_sort(lg, TOPK, True, torch.bfloat16, E)
            us_g = _event_us(lambda i: graph.replay(), it, wm, stream)
            del graph
        extra["route_and_sort_4096"] = {"us": round(us, 1), "hip_graph_replay_us": round(us_g, 1)}
        # NF4: fused dequant+GEMM vs dequant-then-GEMM at 16 / 256 / 16384 tokens (config 5 gate_proj)
        # three packed weight sets in rotation: the 113 MB of one set would stay in the 256 MB MALL between
        # launches, and the figure would not be an HBM figure
        qsets = [quantize_nf4(w, 64) for w in ws]
        packed, qstate = qsets[0]
        nf4 = {}
        for tokens in (16, 256, 16384):
            lgt = torch.randn((tokens, E), device=dev)
            _, _, s5 = softmax_topk_raw(lgt, TOPK, True, torch.bfloat16)
            ms5, _, _ = get_expert_counts_and_idx(s5.view(-1), E)
            x5 = torch.randn((tokens * TOPK, HIDDEN), device=dev, dtype=torch.bfloat16)
            n_it, n_wm = (20, 30) if tokens > 1000 else (100, 300)
            us_f = _event_us(lambda i: grouped_gemm_forward_4bit(x5, *qsets[i % NB], ms5), n_it, n_wm, stream)
            us_u = _event_us(lambda i: grouped_gemm_forward(x5, dequantize_nf4(*qsets[i % NB], torch.bfloat16), ms5),
                             n_it, n_wm, stream)
            if tokens > 1000:
                # the bf16 product alone at this size (131072 rows, about 1024 to an expert: 256 x 256 tiles)
                us_b = _event_us(lambda i: grouped_gemm_forward(x5, ws[i % NB], ms5), 60, 60, stream)
                fl = 2.0 * tokens * TOPK * INTER * HIDDEN
                extra["fwd_gate_proj_131072_rows"] = {"us": round(us_b, 1), "tflops": round(fl / us_b / 1e6, 1),
                                                      "mfma_frac": round(fl / us_b / 1e6 / PEAK_BF16_TFLOPS, 4)}
            active = int((ms5 > 0).sum().item())                       # host read outside any timed loop
            packed_bytes = active * INTER * HIDDEN * (0.5 + 4.0 / 64)
            nf4[f"tokens_{tokens}"] = {"fused_us": round(us_f, 1), "dequant_then_gemm_us": round(us_u, 1),
                                       "active_experts": active, "weight_sets_in_rotation": NB,
                                       "fused_packed_gbs": round(packed_bytes / us_f / 1e3, 1),
                                       "fused_tflops": round(2.0 * tokens * TOPK * INTER * HIDDEN / us_f / 1e6, 1)}
        extra["nf4_gate_proj"] = nf4
        # the dequant kernel alone: packed bytes + scales in, bf16 out (a fresh output tensor per call)
        us = _event_us(lambda i: dequantize_nf4(*qsets[i % NB], torch.bfloat16), 50, MIN_WARMUP, stream)
        b = E * INTER * HIDDEN * (0.5 + 4.0 / 64 + 2.0)
        extra["nf4_dequant_gate_proj"] = {"us": round(us, 1), "gbs": round(b / us / 1e3, 1),
                                          "hbm_frac": round(b / us / 1e3 / PEAK_HBM_GBS, 4)}
        # the input-gradient product on the same packed weights (seen as (E, K=768, N=2048)) at 4096 tokens
        from qwen3_moe_fused.grouped_gemm.forward_4bit import grouped_gemm_forward_transposed_4bit
        dyg = torch.randn((ROWS, INTER), device=dev, dtype=torch.bfloat16)
        us_f = _event_us(lambda i: grouped_gemm_forward_transposed_4bit(dyg, packed, qstate, m_sizes), 50, 100, stream)
        us_u = _event_us(lambda i: grouped_gemm_forward_transposed(dyg, dequantize_nf4(packed, qstate, torch.bfloat16),
                                                                  m_sizes), 50, 50, stream)
        extra["nf4_gate_proj_dx"] = {"fused_us": round(us_f, 1), "dequant_then_gemm_us": round(us_u, 1),
                                     "fused_tflops": round(flop / us_f / 1e6, 1)}
        del dyg
        extra["sweep"] = _reference_sweep(dev, stream, ws, qsets)
        del packed, qstate, qsets, x5
        # config 4: rank-16 LoRA on gate_proj, 8192 tokens, Zipf(1.2)-skewed top-8 routing (65536 rows):
        # the frozen base product and the five thin products of one forward + backward
        T4, R4, RANK = 8192, 8192 * TOPK, 16
        bias = (torch.randperm(E, device=dev).float() + 1).pow(-1.2).log()
        _, _, s4 = softmax_topk_raw(torch.randn((T4, E), device=dev) + bias, TOPK, True, torch.bfloat16)
        ms4, _, _ = get_expert_counts_and_idx(s4.view(-1), E)
        x4 = torch.randn((R4, HIDDEN), device=dev, dtype=torch.bfloat16)
        dy4 = torch.randn((R4, INTER), device=dev, dtype=torch.bfloat16)
        la = torch.randn((E, RANK, HIDDEN), device=dev, dtype=torch.bfloat16) * 0.01
        lb = torch.randn((E, INTER, RANK), device=dev, dtype=torch.bfloat16) * 0.01
        u4 = grouped_gemm_forward(x4, la, ms4)
        y4 = grouped_gemm_forward(x4, ws[0], ms4)
        t4 = grouped_gemm_forward_transposed(dy4, lb, ms4)
        flop4 = 2.0 * R4 * INTER * HIDDEN
        lora = {"rows": R4, "largest_expert_rows": int(ms4.max().item()), "smallest_expert_rows": int(ms4.min().item())}
        for name, fn, stream_bytes in (
                ("base_fwd", lambda i: grouped_gemm_forward(x4, ws[0], ms4), None),
                ("base_dx", lambda i: grouped_gemm_forward_transposed(dy4, ws[0].view(E, INTER, HIDDEN), ms4), None),
                ("lora_a_fwd", lambda i: grouped_gemm_forward(x4, la, ms4), R4 * HIDDEN * 2),
                ("lora_b_fwd_accumulate", lambda i: grouped_gemm_forward(u4, lb, ms4, out=y4, alpha=2.0, accumulate=True),
                 2 * R4 * INTER * 2),
                ("lora_dy_b", lambda i: grouped_gemm_forward_transposed(dy4, lb, ms4), R4 * INTER * 2),
                ("lora_da", lambda i: grouped_gemm_backward_dw(x4, t4, ms4, torch.bfloat16), R4 * HIDDEN * 2),
                ("lora_db", lambda i: grouped_gemm_backward_dw(u4, dy4, ms4, torch.bfloat16), R4 * INTER * 2)):
            us = _event_us(fn, 50, 100, stream)
            lora[name] = {"us": round(us, 1)}
            if stream_bytes is None:
                lora[name]["tflops"] = round(flop4 / us / 1e6, 1)
            else:
                lora[name]["wide_operand_gbs"] = round(stream_bytes / us / 1e3, 1)
        # the base product with the rank-16 term in the same reduction (one pass over the output), forward and
        # input gradient, and the expert MLP with adapters on all three projections, forward + backward
        from qwen3_moe_fused.grouped_gemm.fused import grouped_gemm_forward_lora, grouped_gemm_forward_transposed_lora
        from qwen3_moe_fused.kernels.fast_lora import fast_lora
        us = _event_us(lambda i: grouped_gemm_forward_lora(x4, ws[0], u4, lb, ms4), 50, 100, stream)
        lora["base_fwd_with_lora_term"] = {"us": round(us, 1), "tflops": round(flop4 / us / 1e6, 1)}
        us = _event_us(lambda i: grouped_gemm_forward_transposed_lora(dy4, ws[0].view(E, INTER, HIDDEN), t4, la, ms4),
                       50, 100, stream)
        lora["base_dx_with_lora_term"] = {"us": round(us, 1), "tflops": round(flop4 / us / 1e6, 1)}
        del u4, y4, t4
        adapters = []
        for n_in, n_out in ((HIDDEN, INTER), (HIDDEN, INTER), (INTER, HIDDEN)):
            adapters.append(((torch.randn((E, RANK, n_in), device=dev) * 0.01).bfloat16().requires_grad_(),
                             (torch.randn((E, n_out, RANK), device=dev) * 0.01).bfloat16().requires_grad_()))
        w_down = ws[2].view(E, HIDDEN, INTER)
        x4.requires_grad_()
        dyh = torch.randn((R4, HIDDEN), device=dev, dtype=torch.bfloat16)

        def mlp_step(i):
            (ag, bg), (au, bu), (aw, bw) = adapters
            y = fast_lora(x4, ws[0], None, ag, bg, 2.0, ws[1], None, au, bu, 2.0, w_down, None, aw, bw, 2.0, ms4)
            y.backward(dyh)
            x4.grad = None
            for a_, b_ in adapters:
                a_.grad = b_.grad = None
        us = _event_us(mlp_step, 10, 5, stream)
        lora["expert_mlp_lora_fwd_bwd"] = {"us": round(us, 1), "tokens_per_s": round(T4 / us * 1e6),
                                           "tflops": round(6 * flop4 / us / 1e6, 1)}  # 3 forward + 3 dX products
        # the same step over packed NF4 base weights (QLoRA)
        q_gate, q_up, q_down = (quantize_nf4(w, 64) for w in (ws[0], ws[1], w_down.contiguous()))

        def qlora_step(i):
            (ag, bg), (au, bu), (aw, bw) = adapters
            y = fast_lora(x4, *q_gate, ag, bg, 2.0, *q_up, au, bu, 2.0, *q_down, aw, bw, 2.0, ms4)
            y.backward(dyh)
            x4.grad = None
            for a_, b_ in adapters:
                a_.grad = b_.grad = None
        us = _event_us(qlora_step, 10, 5, stream)
        lora["expert_mlp_qlora_nf4_fwd_bwd"] = {"us": round(us, 1), "tokens_per_s": round(T4 / us * 1e6),
                                                "tflops": round(6 * flop4 / us / 1e6, 1)}
        extra["lora_rank16_zipf_config4"] = lora
        del x4, dy4, dyh, adapters, q_gate, q_up, q_down
        # config 5: the whole sparse block (router -> top-k -> sort -> gather -> gate/up -> SiLU-mul -> down ->
        # weighted combine) with NF4 experts, forward only, module calls as a user makes them
        from types import SimpleNamespace
        from qwen3_moe_fused.modular_qwen3_moe_fused import Qwen3MoeFusedSparseMoeBlock
        from qwen3_moe_fused.quantize.layer import MoeFusedLinear4bit
        cfg5 = SimpleNamespace(num_experts=E, num_experts_per_tok=TOPK, norm_topk_prob=True, hidden_size=HIDDEN,
                               moe_intermediate_size=INTER, hidden_act="silu")
        blk = Qwen3MoeFusedSparseMoeBlock(cfg5).to(torch.bfloat16)
        with torch.no_grad():
            blk.gate.weight.copy_(torch.randn(blk.gate.weight.shape) * 0.02)
            for name, (fin, fout), wsrc in (("gate_proj", (HIDDEN, INTER), ws[0]), ("up_proj", (HIDDEN, INTER), ws[1]),
                                            ("down_proj", (INTER, HIDDEN), ws[2].view(E, HIDDEN, INTER))):
                setattr(blk, name, MoeFusedLinear4bit(fin, fout, E, weight=wsrc, quant_type="nf4", compress_statistics=False, blocksize=64))
        blk = blk.to(dev)
        block = {}
        with torch.no_grad():
            for tokens in (16, 256, 1024, 16384):
                h5 = torch.randn((1, tokens, HIDDEN), device=dev, dtype=torch.bfloat16)
                # short calls need a long warm-up to leave the power-management transient of a launch burst
                n_it, n_wm = (20, 30) if tokens > 2000 else (40, 200)
                timer = _event_us if tokens > 2000 else _event_us_median
                blk.fuse_front = False                        # gather, gate_proj, up_proj, SiLU-mul one by one
                us_sep = timer(lambda i: blk(h5), n_it, n_wm, stream)
                blk.fuse_front = True                         # the default: the four as one kernel
                us = timer(lambda i: blk(h5), n_it, n_wm, stream)
                block[f"tokens_{tokens}"] = {"us": round(us, 1), "tokens_per_s": round(tokens / us * 1e6),
                                             "module_by_module_us": round(us_sep, 1)}
                if tokens <= 256:
                    # decode-sized calls are bound by the seven launches: the same forward captured once in a
                    # HIP graph and replayed (the library only enqueues kernels, so capture needs nothing special)
                    side = torch.cuda.Stream()
                    side.wait_stream(torch.cuda.current_stream())
                    with torch.cuda.stream(side):
                        blk(h5)
                    torch.cuda.current_stream().wait_stream(side)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        blk(h5)
                    us_g = _event_us_median(lambda i: graph.replay(), n_it, n_wm, stream)
                    block[f"tokens_{tokens}"]["hip_graph_replay_us"] = round(us_g, 1)
                    del graph
        extra["nf4_sparse_block_fwd_config5"] = block
        del blk
        # the same block with bf16 experts at the headline configuration's 4096 tokens, and its front half
        # (gather + gate_proj + up_proj + SiLU-mul) alone
        from qwen3_moe_fused.grouped_gemm.fused import grouped_glu_forward
        from qwen3_moe_fused.kernels.routing import _gather
        blk = Qwen3MoeFusedSparseMoeBlock(cfg5).to(torch.bfloat16)
        with torch.no_grad():
            blk.gate.weight.copy_(torch.randn(blk.gate.weight.shape) * 0.02)
            blk.gate_proj.weight.copy_(ws[0])
            blk.up_proj.weight.copy_(ws[1])
            blk.down_proj.weight.copy_(ws[2].view(E, HIDDEN, INTER))
        blk = blk.to(dev)
        toks = [torch.randn((1, TOKENS, HIDDEN), device=dev, dtype=torch.bfloat16) for _ in range(NB)]
        bf16_block = {}
        with torch.no_grad():
            blk.fuse_front = False
            us_sep = _event_us(lambda i: blk(toks[i % NB]), 50, 30, stream)
            blk.fuse_front = True
            us = _event_us(lambda i: blk(toks[i % NB]), 50, 30, stream)
            bf16_block["block_fwd"] = {"us": round(us, 1), "tokens_per_s": round(TOKENS / us * 1e6),
                                       "module_by_module_us": round(us_sep, 1)}
            _, sort_idx2, _ = get_expert_counts_and_idx(selv, E)
            wg_, wu_ = blk.gate_proj.weight, blk.up_proj.weight

            def front_separate(i):
                xg = _gather(toks[i % NB][0], sort_idx2, TOPK, None)
                return silu_mul_forward(grouped_gemm_forward(xg, wg_, m_sizes), grouped_gemm_forward(xg, wu_, m_sizes))

            us_sep = _event_us(front_separate, 50, 5, stream)
            us = _event_us(lambda i: grouped_glu_forward(toks[i % NB][0], wg_, wu_, m_sizes, sort_idx2, TOPK), 50, 5,
                           stream)
            bf16_block["front_half"] = {"fused_us": round(us, 1), "four_kernels_us": round(us_sep, 1),
                                        "fused_tflops": round(2 * flop / us / 1e6, 1)}
        # one training step of the block: forward + backward to the hidden states and all four weight matrices
        blk.zero_grad(set_to_none=True)
        gouts = [torch.randn((1, TOKENS, HIDDEN), device=dev, dtype=torch.bfloat16) for _ in range(NB)]

        def train_step(i):
            h = toks[i % NB].detach().requires_grad_()
            out, _ = blk(h)
            out.backward(gouts[i % NB])
            blk.zero_grad(set_to_none=True)

        blk.fuse_backward = True    # the gated unit's backward in the epilogue of the down projection's input gradient
        us_fb = _event_us(train_step, 30, 15, stream)
        blk.fuse_backward = False   # the default: dh is written, then read by silu_mul_backward
        us = _event_us(train_step, 30, 15, stream)
        bf16_block["block_fwd_bwd"] = {"us": round(us, 1), "tokens_per_s": round(TOKENS / us * 1e6),
                                       "tflops": round(9 * flop / us / 1e6, 1),   # 3 products x (fwd + dX + dW)
                                       "silu_mul_backward_in_dx_epilogue_us": round(us_fb, 1)}
        extra["bf16_sparse_block_fwd_config2"] = bf16_block
        del blk, toks
        out["extra"] = extra

    if not args.no_cpu_baseline:
        import oracle

        xs_np = x0.float().numpy()
        w_np = w0.float().numpy()
        sel_sorted = oracle.sel_from_m_sizes(m_sizes.cpu().numpy())
        rows_done, t_cpu, chunk = 0, 0.0, 2048
        while t_cpu < 10.0:                                   # bounded sample: about 10 s of CPU work
            start = rows_done % ROWS
            sl = slice(start, start + chunk)
            t1 = time.perf_counter()
            y_ref = oracle.linear_fwd(xs_np[sl], w_np, sel_sorted[sl])
            t_cpu += time.perf_counter() - t1
            if rows_done == 0:                                # the first chunk doubles as a parity check
                got = ys[0][:chunk].float().cpu().numpy()
                err = float(np.abs(got - y_ref).max() / np.abs(y_ref).max())
                assert err <= 1e-2, f"benchmarked output differs from the oracle: {err:.3e}"
            rows_done += chunk
        out["cpu_baseline"] = {"value": round(2.0 * rows_done * INTER * HIDDEN / t_cpu / 1e12, 5), "unit": "TFLOP/s",
                               "cores": oracle.num_threads(), "kind": "port",
                               "sample": f"{rows_done} rows of the same batch in 2048-row chunks (wrapping over its "
                                         f"{ROWS} rows), oracle/moe_oracle.c orc_linear_fwd_f32, OpenMP over rows, "
                                         f"{t_cpu:.1f} s; first chunk checked against the GPU output",
                               "host_cpus": os.cpu_count()}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
