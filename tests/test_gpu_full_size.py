"""Benchmark configurations 4 and 5 at their full sizes against the CPU oracle (sampled rows, whole
experts, and size-independent properties), the way tests/test_gpu_gemm.py covers configurations 2
and 3.  At these sizes the kernels pick other tile configurations than at the reduced sizes of
tests/test_gpu_modules.py (square tiles from 512 rows per expert on, the rank-16 configurations,
the register-decode and the pipelined NF4 kernels), and the routing is as skewed or as sparse as the
configurations state.  Method of the reference: test_moe_fused_linear.py:39-58 (the 4-bit product
against the naive forward on dequantised weights), test_lora.py / test_fast_lora.py:51-66."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, randn, to_np32, topk_routing, zipf_bias

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.grouped_gemm.backward_dw import grouped_gemm_backward_dw  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward  # noqa: E402
from qwen3_moe_fused.grouped_gemm.forward_4bit import (grouped_gemm_forward_4bit,  # noqa: E402
                                                       grouped_gemm_forward_transposed_4bit)
from qwen3_moe_fused.grouped_gemm.forward_transposed import grouped_gemm_forward_transposed  # noqa: E402
from qwen3_moe_fused.quantize.nf4 import Nf4QuantState, nf4_code  # noqa: E402

DEV = "cuda"
E, K8, H, I = 128, 8, 2048, 768


def _sample_rows(ms: np.ndarray, n_random: int, seed: int, experts=()) -> np.ndarray:
    """Random rows plus the first and last row of the named experts (tile edges)."""
    R = int(ms.sum())
    rows = np.random.default_rng(seed).choice(R, n_random, replace=False)
    starts = np.concatenate([[0], np.cumsum(ms)])
    edges = [r for e in experts if ms[e] > 0 for r in (starts[e], starts[e + 1] - 1)]
    return np.unique(np.concatenate([rows, np.asarray(edges, dtype=np.int64)])).astype(np.int64)


def _expert_slice(ms: np.ndarray, e: int) -> slice:
    starts = np.concatenate([[0], np.cumsum(ms)])
    return slice(int(starts[e]), int(starts[e + 1]))


# ------------------------------------------------------------------ configuration 4

def test_config4_lora_rank16_zipf_full_size():
    """Rank-16 fused-format LoRA on gate_proj at 8192 tokens, Zipf(1.2)-skewed top-8 routing
    (65536 rows: hot experts > 2000 rows, cold ones < 50, one empty): the frozen base product and
    its input gradient, A, B accumulated into the base output, dy B, dA, dB."""
    T, r, s = 8192, 16, 2.0
    g = gen(404)
    bias = zipf_bias(E, 1.2, g)
    cold = int(bias.argmin())
    bias[cold] = -1e9                         # the least popular expert gets no token at all
    _, ms_t = topk_routing(T, E, K8, g, bias=bias)
    ms = ms_t.numpy().astype(np.int64)
    R = T * K8
    assert ms.sum() == R and ms.max() > 2000 and ms[cold] == 0 and (ms < 50).sum() >= 2
    hot, mid = int(ms.argmax()), int(np.argsort(ms)[E // 2])
    small = int(np.where(ms > 0, ms, R).argmin())          # the smallest expert that has rows
    sel = oracle.sel_from_m_sizes(ms)

    x = randn((R, H), g, 1.0, torch.bfloat16)
    dy = randn((R, I), g, 1.0, torch.bfloat16)
    w = randn((E, I, H), g, 0.02, torch.bfloat16)
    a = randn((E, r, H), g, 0.01, torch.bfloat16)
    b = randn((E, I, r), g, 0.01, torch.bfloat16)
    xd, dyd, wd, ad, bd, msd = (t.to(DEV) for t in (x, dy, w, a, b, ms_t))
    w32, a32, b32 = to_np32(w), to_np32(a), to_np32(b)

    rows = _sample_rows(ms, 768, 1, experts=(hot, mid, small))
    rt = torch.from_numpy(rows)

    # forward: base, A, B accumulated into the base output (one rounding of base + s * u B^T)
    y_base = grouped_gemm_forward(xd, wd, msd)
    check_close(y_base[rt], oracle.linear_fwd(to_np32(x[rt]), w32, sel[rows]), what="config 4 base fwd")
    u = grouped_gemm_forward(xd, ad, msd)
    check_close(u[rt], oracle.linear_fwd(to_np32(x[rt]), a32, sel[rows]), what="config 4 A fwd")
    y = y_base.clone()
    grouped_gemm_forward(u, bd, msd, out=y, alpha=s, accumulate=True)
    exp_y = to_np32(y_base[rt]) + s * oracle.linear_fwd(to_np32(u[rt]), b32, sel[rows])
    check_close(y[rt], exp_y, what="config 4 B fwd accumulated")

    # backward: dy B, base dX, dA, dB
    t = grouped_gemm_forward_transposed(dyd, bd, msd)                      # (R, r)
    check_close(t[rt], oracle.linear_bwd_input(to_np32(dy[rt]), b32, sel[rows]), what="config 4 dy B")
    dx = grouped_gemm_forward_transposed(dyd, wd, msd)                     # (R, H)
    check_close(dx[rt], oracle.linear_bwd_input(to_np32(dy[rt]), w32, sel[rows]), what="config 4 base dX")
    dA = grouped_gemm_backward_dw(xd, t, msd, torch.bfloat16)              # (E, r, H)
    dB = grouped_gemm_backward_dw(u, dyd, msd, torch.bfloat16)             # (E, I, r)
    assert dA.shape == (E, r, H) and dB.shape == (E, I, r)
    zero = np.zeros(0, np.int64)
    for e in (hot, mid, small, cold):
        sl = _expert_slice(ms, e)
        z = np.zeros(sl.stop - sl.start, np.int64) if sl.stop > sl.start else zero
        exp_a = oracle.linear_bwd_weight(to_np32(t[sl]), to_np32(x[sl]), z, 1)[0]
        exp_b = oracle.linear_bwd_weight(to_np32(dy[sl]), to_np32(u[sl]), z, 1)[0]
        check_close(dA[e], exp_a, 1e-2, 1e-2 * max(np.abs(exp_a).max(), 1e-30), f"config 4 dA expert {e} ({ms[e]} rows)")
        check_close(dB[e], exp_b, 1e-2, 1e-2 * max(np.abs(exp_b).max(), 1e-30), f"config 4 dB expert {e} ({ms[e]} rows)")
    assert torch.count_nonzero(dA[cold]).item() == 0 and torch.count_nonzero(dB[cold]).item() == 0
    # size-independent: sum_e dA[e] == t^T x over all rows; run-to-run bit equality
    tot = dA.float().sum(dim=0)
    ref = t.float().t() @ xd.float()
    check_close(tot, to_np32(ref), 2e-2, 2e-2 * float(ref.abs().max()), "sum_e dA == t^T x")
    assert torch.equal(grouped_gemm_backward_dw(xd, t, msd, torch.bfloat16), dA)
    assert torch.equal(grouped_gemm_forward(xd, wd, msd), y_base)


def test_config4_lora_layer_autograd_full_size():
    """The LoRA layer itself (lora.py:134) at the same size: forward and the three gradients."""
    from qwen3_moe_fused.lora import LoraMoeFusedLinear
    from qwen3_moe_fused.modular_qwen3_moe_fused import MoeFusedLinear

    T, r = 8192, 16
    g = gen(405)
    _, ms_t = topk_routing(T, E, K8, g, bias=zipf_bias(E, 1.2, g))
    ms = ms_t.numpy().astype(np.int64)
    R = T * K8
    sel = oracle.sel_from_m_sizes(ms)
    base = MoeFusedLinear(H, I, E)
    layer = LoraMoeFusedLinear(base, "default", r=r, lora_alpha=32)
    with torch.no_grad():
        base.weight.copy_(torch.randn(base.weight.shape, generator=g) * 0.02)
        layer.lora_A["default"].weight.copy_(torch.randn((E, r, H), generator=g) * 0.01)
        layer.lora_B["default"].weight.copy_(torch.randn((E, I, r), generator=g) * 0.01)
    base.weight.requires_grad_(False)
    layer = layer.to(torch.bfloat16).to(DEV)
    s = layer.scaling["default"]
    x = randn((R, H), g, 1.0, torch.bfloat16)
    dy = randn((R, I), g, 1.0, torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    y = layer(xd, ms_t.to(DEV))
    y.backward(dy.to(DEV))

    W = to_np32(layer.base_layer.weight)
    A = to_np32(layer.lora_A["default"].weight)
    B = to_np32(layer.lora_B["default"].weight)
    hot, mid = int(ms.argmax()), int(np.argsort(ms)[E // 2])
    rows = _sample_rows(ms, 512, 2, experts=(hot, mid))
    rt = torch.from_numpy(rows)
    xs, dys, ss = to_np32(x[rt]), to_np32(dy[rt]), sel[rows]
    check_close(y[rt], oracle.lora_linear_fwd(xs, W, A, B, s, ss), what="lora layer fwd")
    tt = oracle.linear_bwd_input(dys, B, ss)
    exp_dx = oracle.linear_bwd_input(dys, W, ss) + s * oracle.linear_bwd_input(tt, A, ss)
    check_close(xd.grad[rt], exp_dx, 2e-2, 2e-2, "lora layer dx")
    gA, gB = layer.lora_A["default"].weight.grad, layer.lora_B["default"].weight.grad
    for e in (hot, mid):
        sl = _expert_slice(ms, e)
        z = np.zeros(sl.stop - sl.start, np.int64)
        xe, dye = to_np32(x[sl]), to_np32(dy[sl])
        te = oracle.linear_bwd_input(dye, B[e:e + 1], z)
        ue = oracle.linear_fwd(xe, A[e:e + 1], z)
        exp_a = s * oracle.linear_bwd_weight(te, xe, z, 1)[0]
        exp_b = s * oracle.linear_bwd_weight(dye, ue, z, 1)[0]
        check_close(gA[e], exp_a, 2e-2, 2e-2 * np.abs(exp_a).max(), f"lora layer dA expert {e}")
        check_close(gB[e], exp_b, 2e-2, 2e-2 * np.abs(exp_b).max(), f"lora layer dB expert {e}")
    assert layer.base_layer.weight.grad is None


# ------------------------------------------------------------------ configuration 5

def _nf4_matrix(shape, seed, blocksize=64):
    """N(0, 0.02) weights quantised by the oracle: packed bytes and state on the GPU, and the
    oracle's bf16-rounded dequantisation (what every product on these weights must see)."""
    w = randn(shape, gen(seed), 0.02).numpy()
    q, absmax = oracle.nf4_quant(w, blocksize)
    w_deq = oracle.round_bf16(oracle.nf4_dequant(q, absmax, blocksize)).reshape(shape)
    state = Nf4QuantState(absmax=torch.from_numpy(absmax).to(DEV), shape=tuple(shape), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=torch.bfloat16)
    return torch.from_numpy(q).view(-1, 1).to(DEV), state, w_deq, w


@pytest.fixture(scope="module")
def nf4_experts():
    return {"gate": _nf4_matrix((E, I, H), 51), "up": _nf4_matrix((E, I, H), 52), "down": _nf4_matrix((E, H, I), 53)}


@pytest.mark.parametrize("which,tokens", [("down", 256), ("gate", 16384), ("down", 16384)])
def test_config5_fused_nf4_forward_full_size(nf4_experts, which, tokens):
    """grouped_gemm_forward_4bit with the down_proj shape (N=2048, K=768) at 2048 rows, and both
    shapes at 16384 tokens (131072 rows, 1024 per expert: the square-tile pipelined NF4 kernel)."""
    packed, state, w_deq, _ = nf4_experts[which]
    _, N, K = state.shape
    g = gen(tokens + N)
    _, ms_t = topk_routing(tokens, E, K8, g)
    ms = ms_t.numpy().astype(np.int64)
    R = tokens * K8
    sel = oracle.sel_from_m_sizes(ms)
    x = randn((R, K), g, 1.0, torch.bfloat16)
    y = grouped_gemm_forward_4bit(x.to(DEV), packed, state, ms_t.to(DEV))
    assert y.shape == (R, N) and y.dtype == torch.bfloat16
    rows = _sample_rows(ms, min(R, 1024), 3, experts=(0, 63, 127))
    rt = torch.from_numpy(rows)
    check_close(y[rt], oracle.linear_fwd(to_np32(x[rt]), w_deq, sel[rows]), what=f"nf4 {which} fwd, {tokens} tokens")
    assert torch.equal(grouped_gemm_forward_4bit(x.to(DEV), packed, state, ms_t.to(DEV)), y)


def test_config5_fused_nf4_input_gradient_full_size(nf4_experts):
    """dx = dy W on the packed down_proj weight (E, 2048, 768) at 16384 tokens."""
    packed, state, w_deq, _ = nf4_experts["down"]
    tokens = 16384
    g = gen(77)
    _, ms_t = topk_routing(tokens, E, K8, g)
    ms = ms_t.numpy().astype(np.int64)
    R = tokens * K8
    sel = oracle.sel_from_m_sizes(ms)
    dy = randn((R, H), g, 1.0, torch.bfloat16)
    dx = grouped_gemm_forward_transposed_4bit(dy.to(DEV), packed, state, ms_t.to(DEV))
    rows = _sample_rows(ms, 1024, 4, experts=(0, 127))
    rt = torch.from_numpy(rows)
    check_close(dx[rt], oracle.linear_bwd_input(to_np32(dy[rt]), w_deq, sel[rows]), what="nf4 down dX, 16384 tokens")


def _near_tied(logits_row: np.ndarray, a: int, b: int) -> bool:
    """Two experts whose bf16 router logits differ by a few units in the last place: either order
    is a correct top-k answer for a router GEMM that rounds its sums to bf16."""
    la, lb = float(logits_row[a]), float(logits_row[b])
    return abs(la - lb) <= 2.0 ** -5 * max(abs(la), abs(lb), 1.0)


@pytest.mark.parametrize("tokens", [16, 256, 16384])
def test_config5_nf4_sparse_block_matches_oracle(nf4_experts, tokens):
    """The whole sparse block with NF4 experts (router -> top-8 of 128 -> sort -> gate/up -> SiLU-mul
    -> down -> weighted sum) against oracle.moe_block_fwd on the oracle-dequantised weights.  Tokens are
    independent given their routing, so at 16384 tokens the oracle evaluates a seeded sample of 320 of them;
    the routing that is compared is the block's own (its top-k kernel's expert ids), not a second top-k."""
    from types import SimpleNamespace

    from qwen3_moe_fused.modular_qwen3_moe_fused import Qwen3MoeFusedSparseMoeBlock
    from qwen3_moe_fused.quantize.layer import MoeFusedLinear4bit

    cfg = SimpleNamespace(num_experts=E, num_experts_per_tok=K8, norm_topk_prob=True, hidden_size=H,
                          moe_intermediate_size=I, hidden_act="silu")
    blk = Qwen3MoeFusedSparseMoeBlock(cfg).to(torch.bfloat16)
    gate_w = randn((E, H), gen(60), 0.02, torch.bfloat16)
    with torch.no_grad():
        blk.gate.weight.copy_(gate_w)
    for name, key, (fin, fout) in (("gate_proj", "gate", (H, I)), ("up_proj", "up", (H, I)), ("down_proj", "down", (I, H))):
        packed, state, _, w = nf4_experts[key]
        layer = MoeFusedLinear4bit(fin, fout, E, weight=torch.from_numpy(w), quant_type="nf4", compress_statistics=False, blocksize=64).to(DEV)
        # the module's own quantiser must produce the oracle's bytes and scales
        assert torch.equal(layer.weight.data.view(-1), packed.view(-1)), name
        assert torch.equal(layer.weight.quant_state.absmax.view(-1), state.absmax.view(-1)), name
        setattr(blk, name, layer)
    blk = blk.to(DEV)
    hidden = randn((1, tokens, H), gen(tokens), 1.0, torch.bfloat16)
    sample = np.arange(tokens) if tokens <= 320 else np.sort(np.random.default_rng(tokens).choice(tokens, 320, replace=False))
    st = torch.from_numpy(sample)
    out_ref, logits_ref = oracle.moe_block_fwd(to_np32(hidden[0][st]), to_np32(gate_w), nf4_experts["gate"][2],
                                               nf4_experts["up"][2], nf4_experts["down"][2], K8, True, oracle.round_bf16)
    blk.keep_routing = True
    for fuse in (True, False):
        blk.fuse_front = fuse
        with torch.no_grad():
            out, logits = blk(hidden.to(DEV))
        assert out.shape == (1, tokens, H) and logits.shape == (tokens, E)
        sel_all = blk.last_selected
        assert sel_all.shape == (tokens, K8)
        # the block's selections are a top-k of the block's own logits (ties aside: compare probabilities)
        p_gpu = torch.softmax(logits.float(), -1)
        kth = torch.gather(p_gpu, 1, sel_all.long()).min(dim=1).values
        rest = p_gpu.scatter(1, sel_all.long(), -1.0).max(dim=1).values
        assert (kth >= rest).all(), "a selected expert has a smaller probability than one left out"
        out, logits = out[:, st.to(out.device)], logits[st.to(logits.device)]
        check_close(logits, logits_ref, 2e-2, 2e-2, "router logits")
        sel_gpu = sel_all[st.to(sel_all.device)].cpu().numpy()
        sel_ref = oracle.softmax_topk(logits_ref, K8, True)[1]
        same = np.array([set(a) == set(b) for a, b in zip(sel_gpu, sel_ref)])
        assert same.mean() >= 0.9
        for t in np.nonzero(~same)[0]:
            only_gpu, only_ref = set(sel_gpu[t]) - set(sel_ref[t]), set(sel_ref[t]) - set(sel_gpu[t])
            assert len(only_gpu) == len(only_ref) == 1, f"token {t}: routing differs by more than one expert"
            assert _near_tied(logits_ref[t], only_gpu.pop(), only_ref.pop()), f"token {t}: swapped experts are not near-tied"
        check_close(out[0][torch.from_numpy(same)], out_ref[same], 2e-2, 2e-2, f"nf4 block output (fuse_front={fuse})")
