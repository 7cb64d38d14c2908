"""Module-level parity: the sparse MoE block, the fused-format LoRA layer, the fast-LoRA
autograd function and the 4-bit layer, against the oracle's compositions and against torch
autograd of the reference's formulas."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, randn, to_np32, topk_routing, zipf_bias

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.fast_lora import (fast_Qwen3MoeFusedSparseMoeBlock_forward, get_lora_parameters)  # noqa: E402
from qwen3_moe_fused.kernels.fast_lora import fast_lora  # noqa: E402
from qwen3_moe_fused.lora import LoraMoeFusedLinear  # noqa: E402
from qwen3_moe_fused.modular_qwen3_moe_fused import MoeFusedLinear, Qwen3MoeFusedSparseMoeBlock  # noqa: E402
from qwen3_moe_fused.quantize.layer import MoeFusedLinear4bit  # noqa: E402
from qwen3_moe_fused.quantize.nf4 import dequantize_nf4  # noqa: E402

DEV = "cuda"


def _config(E, k, H, I, renorm=True):
    return SimpleNamespace(num_experts=E, num_experts_per_tok=k, norm_topk_prob=renorm, hidden_size=H,
                           moe_intermediate_size=I, hidden_act="silu")


def _block(cfg, dtype, seed):
    torch.manual_seed(seed)
    blk = Qwen3MoeFusedSparseMoeBlock(cfg)
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn(p.shape, generator=gen(seed + p.numel() % 97)) * 0.05)
    return blk.to(dtype)


def test_module_init_bound():
    m = MoeFusedLinear(64, 32, 4)
    bound = (15.0 / 64) ** 0.5                       # modular_qwen3_moe_fused.py:25
    assert m.weight.shape == (4, 32, 64)
    assert m.weight.abs().max() <= bound and m.weight.abs().max() > 0.8 * bound
    assert "num_experts=4" in repr(m)


@pytest.mark.parametrize("T,E,k,H,I,dtype", [(7 * 13, 11, 3, 16, 3, torch.float32),     # test_model.py tiny config
                                             (256, 8, 2, 64, 128, torch.float32),
                                             (512, 128, 8, 256, 96, torch.bfloat16)])
def test_sparse_block_forward(T, E, k, H, I, dtype):
    cfg = _config(E, k, H, I)
    blk = _block(cfg, dtype, 3)
    hidden = randn((1, T, H), gen(T), 1.0, dtype)
    params = {n: to_np32(p) for n, p in blk.named_parameters()}
    rnd = oracle.round_bf16 if dtype == torch.bfloat16 else None
    out_ref, logits_ref = oracle.moe_block_fwd(to_np32(hidden[0]), params["gate.weight"], params["gate_proj.weight"],
                                               params["up_proj.weight"], params["down_proj.weight"], k, True, rnd)
    blk = blk.to(DEV)
    blk.keep_routing = True
    out, logits = blk(hidden.to(DEV))
    assert out.shape == (1, T, H) and logits.shape == (T, E)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    check_close(logits, logits_ref, tol, tol, "router logits")
    # the routing under test is the block's own: the expert ids its top-k kernel wrote
    sel_gpu = blk.last_selected.cpu().numpy()
    assert sel_gpu.shape == (T, k)
    if dtype == torch.bfloat16:
        # a bf16 router can flip near-tied experts between implementations; compare only tokens
        # whose oracle routing matches the GPU's
        sel_ref = oracle.softmax_topk(logits_ref, k, True)[1]
        same = (np.sort(sel_gpu, 1) == np.sort(sel_ref, 1)).all(1)
        assert same.mean() > 0.97
        check_close(out[0][torch.from_numpy(same)], out_ref[same], tol, tol, "block output")
        # the other tokens: the two routings differ by exactly one expert, and the swapped pair's
        # bf16 logits lie within a few units in the last place of each other
        for t in np.nonzero(~same)[0]:
            only_gpu, only_ref = set(sel_gpu[t]) - set(sel_ref[t]), set(sel_ref[t]) - set(sel_gpu[t])
            assert len(only_gpu) == len(only_ref) == 1, f"token {t}: routing differs by more than one expert"
            la, lb = float(logits_ref[t, only_gpu.pop()]), float(logits_ref[t, only_ref.pop()])
            assert abs(la - lb) <= 2.0 ** -5 * max(abs(la), abs(lb), 1.0), f"token {t}: swapped experts are not near-tied"
    else:
        assert np.array_equal(np.sort(sel_gpu, 1), np.sort(oracle.softmax_topk(logits_ref, k, True)[1], 1))
        check_close(out[0], out_ref, tol, tol, "block output")


def test_sparse_block_backward_fp32_matches_autograd():
    T, E, k, H, I = 60, 6, 2, 32, 24
    cfg = _config(E, k, H, I)
    blk = _block(cfg, torch.float32, 5).to(DEV)
    hidden = randn((2, T // 2, H), gen(1)).to(DEV).requires_grad_()
    out, _ = blk(hidden)
    gout = randn((2, T // 2, H), gen(2)).to(DEV)
    out.backward(gout)
    grads = {n: p.grad.clone() for n, p in blk.named_parameters()}
    gh = hidden.grad.clone()

    # the reference formulation in stock torch ops (modular_qwen3_moe_fused.py:79-118)
    h2 = hidden.detach().clone().requires_grad_()
    ps = {n: p.detach().clone().requires_grad_() for n, p in blk.named_parameters()}
    x = h2.view(T, H)
    logits = x @ ps["gate.weight"].t()
    rw, sel = torch.topk(torch.softmax(logits, dim=1, dtype=torch.float32), k, dim=-1)
    rw = rw / rw.sum(dim=-1, keepdim=True)
    xr = x.unsqueeze(1).expand(T, k, H).reshape(T * k, H)
    sf = sel.reshape(-1)
    lin = lambda a, w: torch.einsum("bnk,bk->bn", w[sf], a)
    y = lin(torch.nn.functional.silu(lin(xr, ps["gate_proj.weight"])) * lin(xr, ps["up_proj.weight"]),
            ps["down_proj.weight"])
    out2 = torch.einsum("beo,be->bo", y.view(T, k, H), rw).view(2, T // 2, H)
    out2.backward(gout)
    torch.testing.assert_close(out, out2, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(gh, h2.grad, rtol=1e-3, atol=1e-5)
    for n in grads:
        torch.testing.assert_close(grads[n], ps[n].grad, rtol=1e-3, atol=1e-5, msg=n)


def _lora_layer(in_f, out_f, E, r, alpha, dtype, seed, rslora=False):
    base = MoeFusedLinear(in_f, out_f, E)
    layer = LoraMoeFusedLinear(base, "default", r=r, lora_alpha=alpha, use_rslora=rslora)
    with torch.no_grad():
        base.weight.copy_(torch.randn(base.weight.shape, generator=gen(seed)) * 0.02)
        layer.lora_A["default"].weight.copy_(torch.randn((E, r, in_f), generator=gen(seed + 1)) * 0.01)
        layer.lora_B["default"].weight.copy_(torch.randn((E, out_f, r), generator=gen(seed + 2)) * 0.01)
    base.weight.requires_grad_(False)
    return layer.to(dtype)


def test_lora_layer_init_and_scaling():
    layer = LoraMoeFusedLinear(MoeFusedLinear(32, 48, 4), "default", r=4, lora_alpha=8)
    assert layer.scaling["default"] == 2.0                                  # alpha / r
    assert layer.lora_A["default"].weight.shape == (4, 4, 32)
    assert layer.lora_B["default"].weight.shape == (4, 48, 4)
    assert torch.count_nonzero(layer.lora_B["default"].weight) == 0         # B starts at zero
    rs = LoraMoeFusedLinear(MoeFusedLinear(32, 48, 4), "default", r=16, lora_alpha=8, use_rslora=True)
    assert rs.scaling["default"] == 2.0                                     # alpha / sqrt(r)
    with pytest.raises(NotImplementedError):
        layer.merge()
    with pytest.raises(NotImplementedError):
        LoraMoeFusedLinear(MoeFusedLinear(8, 8, 2), "default", r=2, use_dora=True)
    with pytest.raises(ValueError):
        LoraMoeFusedLinear(MoeFusedLinear(8, 8, 2), "default", r=0)


def test_lora_config4_rank16_zipf_bf16():
    """benchmark configuration 4 at reduced hidden size for the oracle: rank-16 fused-format LoRA,
    Zipf(1.2)-skewed top-8 routing, forward + backward in bf16."""
    E, k, T, H, I, r = 128, 8, 1024, 256, 96, 16
    g = gen(44)
    sel, ms = topk_routing(T, E, k, g, bias=zipf_bias(E, 1.2, g))
    assert ms.max() > 20 * max(1, ms.min())                                # hot vs cold experts
    R = T * k
    layer = _lora_layer(H, I, E, r, 32, torch.bfloat16, 9).to(DEV)
    x = randn((R, H), g, 1.0, torch.bfloat16)
    dy = randn((R, I), g, 1.0, torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    y = layer(xd, ms.to(DEV))
    y.backward(dy.to(DEV))

    W = to_np32(layer.base_layer.weight)
    A = to_np32(layer.lora_A["default"].weight)
    B = to_np32(layer.lora_B["default"].weight)
    s = layer.scaling["default"]
    sel_sorted = oracle.sel_from_m_sizes(ms.numpy())
    check_close(y, oracle.lora_linear_fwd(to_np32(x), W, A, B, s, sel_sorted), what="lora fwd")
    # gradients of y = x W^T + s (x A^T) B^T
    u = oracle.linear_fwd(to_np32(x), A, sel_sorted)
    t = oracle.linear_bwd_input(to_np32(dy), B, sel_sorted)
    dA = s * oracle.linear_bwd_weight(t, to_np32(x), sel_sorted, E)
    dB = s * oracle.linear_bwd_weight(to_np32(dy), u, sel_sorted, E)
    dx = oracle.linear_bwd_input(to_np32(dy), W, sel_sorted) + s * oracle.linear_bwd_input(t, A, sel_sorted)
    check_close(xd.grad, dx, 2e-2, 2e-2, "lora dx")
    check_close(layer.lora_A["default"].weight.grad, dA, 2e-2, 2e-2 * np.abs(dA).max(), "lora dA")
    check_close(layer.lora_B["default"].weight.grad, dB, 2e-2, 2e-2 * np.abs(dB).max(), "lora dB")
    assert layer.base_layer.weight.grad is None


def _lora_block(cfg, dtype, r=4):
    blk = _block(cfg, dtype, 21)
    for i, name in enumerate(("gate_proj", "up_proj", "down_proj")):
        base = getattr(blk, name)
        base.weight.requires_grad_(False)
        layer = LoraMoeFusedLinear(base, "default", r=r, lora_alpha=2 * r, use_rslora=True)
        with torch.no_grad():  # B re-initialised non-zero so the adapter matters (test_lora.py:72-75)
            layer.lora_B["default"].weight.copy_(torch.randn(layer.lora_B["default"].weight.shape,
                                                             generator=gen(50 + i)) * 0.05)
        setattr(blk, name, layer.to(dtype))
    return blk


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)])
def test_fast_lora_block_matches_module_path(dtype, tol):
    """The reference's own check (test_fast_lora.py:51-66): module-by-module forward/backward vs
    the single fast_lora function -- outputs and every trainable gradient."""
    T, E, k, H, I = 96, 11, 3, 32, 24
    cfg = _config(E, k, H, I)
    blk = _lora_block(cfg, dtype).to(DEV)
    hidden = randn((1, T, H), gen(4), 1.0, dtype).to(DEV)
    gout = randn((1, T, H), gen(5), 1.0, dtype).to(DEV)

    h1 = hidden.clone().requires_grad_()
    out1, _ = blk(h1)
    out1.backward(gout)
    g1 = {n: p.grad.clone() for n, p in blk.named_parameters() if p.grad is not None}
    blk.zero_grad()

    h2 = hidden.clone().requires_grad_()
    out2, _ = fast_Qwen3MoeFusedSparseMoeBlock_forward(blk, h2)
    out2.backward(gout)
    g2 = {n: p.grad.clone() for n, p in blk.named_parameters() if p.grad is not None}
    lora_names = {n for n in g1 if "lora_" in n}
    assert lora_names and lora_names <= set(g2)
    check_close(out2, to_np32(out1), tol, tol, "fast lora output")
    check_close(h2.grad, to_np32(h1.grad), tol, tol * float(h1.grad.abs().max()), "fast lora d hidden")
    for n in sorted(lora_names):
        check_close(g2[n], to_np32(g1[n]), tol, tol * float(g1[n].abs().max() + 1e-12), n)
    W, qs, A, B, s = get_lora_parameters(blk.gate_proj)
    assert qs is None and A.shape == (E, 4, H) and B.shape == (E, I, 4) and s == 4.0


@pytest.mark.parametrize("dtype,R,E,H,M,r", [(torch.float32, 300, 5, 64, 40, 4), (torch.bfloat16, 2048, 16, 256, 96, 16),
                                            (torch.bfloat16, 700, 8, 128, 64, 8),
                                            # from 4096 rows on: split-row dA/dB, and with equal scalings the gate
                                            # and up adapters share their passes over x
                                            (torch.bfloat16, 4608, 6, 256, 256, 16)])
def test_fast_lora_matches_oracle_composition(dtype, R, E, H, M, r):
    """fast_lora (one autograd function for the expert MLP with LoRA on its three projections)
    against the oracle's composition of the reference's formulas (kernels/fast_lora.py:3-46): the
    output and all seven gradients, not only against the module-by-module HIP path."""
    g = gen(R + H)
    Sg, Su, Sw = (2.0, 2.0, 1.5) if R >= 4096 else (2.0, 0.5, 1.5)
    mk = lambda *shape, scale: randn(shape, g, scale, dtype)
    G, U, W = mk(E, M, H, scale=0.05), mk(E, M, H, scale=0.05), mk(E, H, M, scale=0.05)
    Ag, Bg = mk(E, r, H, scale=0.05), mk(E, M, r, scale=0.05)
    Au, Bu = mk(E, r, H, scale=0.05), mk(E, M, r, scale=0.05)
    Aw, Bw = mk(E, r, M, scale=0.05), mk(E, H, r, scale=0.05)
    x, dy = mk(R, H, scale=1.0), mk(R, H, scale=1.0)
    ms = torch.bincount(torch.randint(0, E, (R,), generator=g), minlength=E).int()
    ms[E // 2] += ms[0]
    ms[0] = 0                                               # one expert without rows
    sel = oracle.sel_from_m_sizes(ms.numpy())
    rnd = oracle.round_bf16 if dtype == torch.bfloat16 else None
    ref = oracle.lora_mlp_fwd_bwd(to_np32(x), to_np32(G), to_np32(Ag), to_np32(Bg), Sg, to_np32(U), to_np32(Au),
                                  to_np32(Bu), Su, to_np32(W), to_np32(Aw), to_np32(Bw), Sw, sel, to_np32(dy), rnd)
    lora = [t.to(DEV).requires_grad_() for t in (Ag, Bg, Au, Bu, Aw, Bw)]
    xd = x.to(DEV).requires_grad_()
    y = fast_lora(xd, G.to(DEV), None, lora[0], lora[1], Sg, U.to(DEV), None, lora[2], lora[3], Su,
                  W.to(DEV), None, lora[4], lora[5], Sw, ms.to(DEV))
    y.backward(dy.to(DEV))
    tol = 3e-2 if dtype == torch.bfloat16 else 2e-4
    check_close(y, ref["y"], tol, tol, "fast_lora y")
    check_close(xd.grad, ref["dx"], tol, tol * float(np.abs(ref["dx"]).max()), "fast_lora dx")
    for t, name in zip(lora, ("dAg", "dBg", "dAu", "dBu", "dAw", "dBw")):
        check_close(t.grad, ref[name], tol, tol * float(np.abs(ref[name]).max()), "fast_lora " + name)
        assert torch.count_nonzero(t.grad[0]).item() == 0, "expert without rows: exact zeros"


def test_4bit_layer_and_fast_lora_on_nf4_base():
    E, H, I, r, R = 8, 128, 64, 8, 512
    g = gen(31)
    base = MoeFusedLinear(H, I, E)
    with torch.no_grad():
        base.weight.copy_(torch.randn(base.weight.shape, generator=g) * 0.02)
    q = MoeFusedLinear4bit(H, I, E, weight=base.weight, quant_type="nf4", compress_statistics=False, blocksize=64).to(DEV)
    assert q.weight.dtype == torch.uint8 and q.weight.quant_state is not None
    assert q.weight.numel() == E * I * H // 2 and not q.weight.requires_grad
    sd = q.state_dict()
    assert "weight.absmax" in sd and "weight.quant_map" in sd

    ms = torch.bincount(torch.randint(0, E, (R,), generator=g), minlength=E).int()
    sel = oracle.sel_from_m_sizes(ms.numpy())
    x = randn((R, H), g, 1.0, torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    y = q(xd, ms.to(DEV))
    w_q, am = oracle.nf4_quant(to_np32(base.weight), 64)
    assert np.array_equal(q.weight.cpu().numpy().reshape(-1), w_q)
    w_deq = oracle.round_bf16(oracle.nf4_dequant(w_q, am, 64)).reshape(E, I, H)
    check_close(y, oracle.linear_fwd(to_np32(x), w_deq, sel), what="4bit layer fwd")
    dy = randn((R, I), g, 1.0, torch.bfloat16)
    y.backward(dy.to(DEV))
    check_close(xd.grad, oracle.linear_bwd_input(to_np32(dy), w_deq, sel), what="4bit layer dx")

    # fast_lora with quantised bases == fast_lora with the dequantised bases
    def lora_params(out_f, in_f, seed):
        a = (torch.randn((E, r, in_f), generator=gen(seed)) * 0.05).bfloat16().to(DEV).requires_grad_()
        b = (torch.randn((E, out_f, r), generator=gen(seed + 1)) * 0.05).bfloat16().to(DEV).requires_grad_()
        return a, b

    def qbase(out_f, in_f, seed):
        m = MoeFusedLinear(in_f, out_f, E)
        with torch.no_grad():
            m.weight.copy_(torch.randn(m.weight.shape, generator=gen(seed)) * 0.05)
        return MoeFusedLinear4bit(in_f, out_f, E, weight=m.weight, quant_type="nf4", compress_statistics=False).to(DEV).weight

    Gq, Uq, Wq = qbase(I, H, 1), qbase(I, H, 2), qbase(H, I, 3)
    (Ag, Bg), (Au, Bu), (Aw, Bw) = lora_params(I, H, 10), lora_params(I, H, 20), lora_params(H, I, 30)
    gout = randn((R, H), g, 1.0, torch.bfloat16).to(DEV)
    x1 = x.to(DEV).requires_grad_()
    y1 = fast_lora(x1, Gq.data, Gq.quant_state, Ag, Bg, 2.0, Uq.data, Uq.quant_state, Au, Bu, 2.0,
                   Wq.data, Wq.quant_state, Aw, Bw, 2.0, ms.to(DEV))
    y1.backward(gout)
    g_q = [p.grad.clone() for p in (x1, Ag, Bg, Au, Bu, Aw, Bw)]
    for p in (Ag, Bg, Au, Bu, Aw, Bw):
        p.grad = None
    dq = lambda p: dequantize_nf4(p.data, p.quant_state, torch.bfloat16)
    x2 = x.to(DEV).requires_grad_()
    y2 = fast_lora(x2, dq(Gq), None, Ag, Bg, 2.0, dq(Uq), None, Au, Bu, 2.0, dq(Wq), None, Aw, Bw, 2.0, ms.to(DEV))
    y2.backward(gout)
    g_d = [p.grad for p in (x2, Ag, Bg, Au, Bu, Aw, Bw)]
    check_close(y1, to_np32(y2), 2e-2, 2e-2, "fast_lora nf4 vs dense")
    for a, b, n in zip(g_q, g_d, ("dx", "dAg", "dBg", "dAu", "dBu", "dAw", "dBw")):
        check_close(a, to_np32(b), 2e-2, 2e-2 * float(b.abs().max() + 1e-12), n)


def _grads_close(a, b, what):
    a, b = a.float(), b.float()
    err = (a - b).abs().max().item() / max(b.abs().max().item(), 1e-30)
    assert err <= 2e-2, f"{what}: normalised max error {err:.3e}"


@pytest.mark.parametrize("T,E,k,H,I", [(384, 16, 4, 256, 96), (40, 64, 8, 128, 64)])
def test_fused_front_of_block_matches_module_by_module_path(T, E, k, H, I):
    cfg = _config(E, k, H, I)
    blk = _block(cfg, torch.bfloat16, 11).to(DEV)
    hidden = randn((1, T, H), gen(T), 1.0, torch.bfloat16).to(DEV)
    gout = randn((1, T, H), gen(T + 1), 1.0, torch.bfloat16).to(DEV)
    results = []
    for fuse, fuse_backward in ((True, True), (False, False), (True, False)):
        blk.fuse_front, blk.fuse_backward = fuse, fuse_backward
        blk.zero_grad(set_to_none=True)
        h = hidden.clone().requires_grad_()
        out, logits = blk(h)
        out.backward(gout)
        results.append((out.detach(), h.grad, {n: p.grad.clone() for n, p in blk.named_parameters()}))
    (o1, g1, p1), (o2, g2, p2), (o3, g3, p3) = results
    assert torch.equal(o3, o1) and torch.equal(g3, g1), "the backward epilogue changes no bit of the fused path"
    for n in p1:
        assert torch.equal(p3[n], p1[n]), n
    assert torch.equal(o1, o2), "same kernels' arithmetic, same roundings"
    _grads_close(g1, g2, "d hidden")
    for n in p1:
        _grads_close(p1[n], p2[n], n)
    # the gated unit's backward in the down projection's input gradient returns the bits of the separate kernel:
    # the three weight gradients, products over the same de, dg and h, are the same bits too
    for n in ("gate_proj.weight", "up_proj.weight", "down_proj.weight"):
        assert torch.equal(p1[n], p2[n]), n
    # inference: no products are kept, same output
    blk.fuse_front = True
    with torch.no_grad():
        o3, _ = blk(hidden)
    assert torch.equal(o3, o1)


def test_fused_front_of_block_with_4bit_projections():
    T, E, k, H, I = 96, 8, 2, 128, 64
    cfg = _config(E, k, H, I)
    blk = _block(cfg, torch.bfloat16, 13)
    for name, (i, o) in {"gate_proj": (H, I), "up_proj": (H, I), "down_proj": (I, H)}.items():
        setattr(blk, name, MoeFusedLinear4bit(i, o, E, weight=getattr(blk, name).weight, quant_type="nf4", compress_statistics=False))
    blk = blk.to(DEV)
    hidden = randn((1, T, H), gen(3), 1.0, torch.bfloat16).to(DEV)
    gout = randn((1, T, H), gen(4), 1.0, torch.bfloat16).to(DEV)
    outs = []
    for fuse in (False, True, True):  # the first call attaches the quant states; fused from the second on
        blk.fuse_front = fuse
        h = hidden.clone().requires_grad_()
        out, _ = blk(h)
        out.backward(gout)
        outs.append((out.detach(), h.grad))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[1][0], outs[2][0])
    _grads_close(outs[1][1], outs[0][1], "d hidden, 4-bit")


def test_fused_model_matches_installed_transformers_model():
    """The method of the reference's test_model.py (tiny fp32 model, same weights in both
    layouts, same hidden states), against the transformers release that is installed."""
    transformers = pytest.importorskip("transformers")
    from transformers import Qwen3MoeConfig, Qwen3MoeModel

    from qwen3_moe_fused.modular_qwen3_moe_fused import Qwen3MoeFusedModel

    torch.manual_seed(42)
    inter = 3
    config = Qwen3MoeConfig(vocab_size=500, hidden_size=16, intermediate_size=5, num_hidden_layers=2,
                            num_attention_heads=8, num_key_value_heads=4, max_window_layers=2,
                            moe_intermediate_size=inter, num_experts=11, norm_topk_prob=True,   # test_model.py:29-40
                            experts_implementation="eager")   # torch's grouped mm refuses rows of 3 elements
    model = Qwen3MoeModel(config).to(DEV, torch.float32).eval()
    fused = Qwen3MoeFusedModel(config).to(DEV, torch.float32).eval()
    sd = {}
    for key, value in model.state_dict().items():
        if key.endswith("mlp.experts.gate_up_proj"):      # (E, 2 * inter, hidden): gate rows first
            stem = key[: -len("experts.gate_up_proj")]
            sd[stem + "gate_proj.weight"] = value[:, :inter].contiguous()
            sd[stem + "up_proj.weight"] = value[:, inter:].contiguous()
        elif key.endswith("mlp.experts.down_proj"):
            sd[key[: -len("experts.down_proj")] + "down_proj.weight"] = value
        elif ".mlp.experts." in key:                      # per-expert layout of older releases
            pytest.skip("installed transformers keeps one matrix per expert; covered by tests/test_convert.py")
        else:
            sd[key] = value
    missing, unexpected = fused.load_state_dict(sd, strict=False)
    assert not unexpected and not [k for k in missing if "rotary" not in k], (missing, unexpected)
    ids = torch.randint(0, 500, (7, 13), generator=gen(1)).to(DEV)
    with torch.no_grad():
        h_ref = model(input_ids=ids).last_hidden_state
        h = fused(input_ids=ids).last_hidden_state
    torch.testing.assert_close(h, h_ref, rtol=1e-4, atol=1e-4)


def test_fused_causal_lm_reports_router_logits_and_aux_loss():
    """output_router_logits: one (tokens, experts) tensor per sparse layer, equal to that layer's
    gate applied to its input, and a load-balancing loss that is not silently zero (the reference's
    block hands the logits up through its return value, modular_qwen3_moe_fused.py:118; the
    installed transformers release collects them with hooks on the router module)."""
    transformers = pytest.importorskip("transformers")
    from transformers import Qwen3MoeConfig

    from qwen3_moe_fused.modular_qwen3_moe_fused import Qwen3MoeFusedForCausalLM, Qwen3MoeFusedRouter

    torch.manual_seed(7)
    config = Qwen3MoeConfig(vocab_size=300, hidden_size=32, intermediate_size=24, num_hidden_layers=3,
                            num_attention_heads=4, num_key_value_heads=2, moe_intermediate_size=16, num_experts=8,
                            num_experts_per_tok=2, norm_topk_prob=True, mlp_only_layers=[1],
                            output_router_logits=True, router_aux_loss_coef=0.01)
    model = Qwen3MoeFusedForCausalLM(config).to(DEV, torch.float32).eval()
    seen = []
    hooks = [m.register_forward_hook(lambda mod, args, out: seen.append((args[0].detach(), out.detach())))
             for m in model.modules() if isinstance(m, Qwen3MoeFusedRouter)]
    assert len(hooks) == 2                                       # layers 0 and 2 are sparse, layer 1 is dense
    ids = torch.randint(0, 300, (3, 11), generator=gen(2)).to(DEV)
    with torch.no_grad():
        out = model(input_ids=ids, labels=ids, output_router_logits=True)
    for h in hooks:
        h.remove()
    assert out.router_logits is not None and len(out.router_logits) == 2
    for logits, (x, recorded) in zip(out.router_logits, seen):
        assert logits.shape == (33, 8)
        assert torch.equal(logits, recorded)
        torch.testing.assert_close(logits, x @ model.model.layers[0].mlp.gate.weight.t()
                                   if recorded is seen[0][1] else x @ model.model.layers[2].mlp.gate.weight.t(),
                                   rtol=1e-4, atol=1e-5)
    assert out.aux_loss is not None and float(out.aux_loss) > 0.0


@pytest.mark.parametrize("four_bit", [False, True])
def test_block_forward_replays_from_a_hip_graph(four_bit):
    """The library only enqueues kernels (no allocation, no synchronisation, no memset), so a
    decode-sized block forward can be captured once and replayed: every replay must equal the
    eager result for the input that is in the static buffer at that time."""
    T, E, k, H, I = 24, 16, 4, 128, 64
    cfg = _config(E, k, H, I)
    blk = _block(cfg, torch.bfloat16, 17)
    if four_bit:
        for name, (i, o) in {"gate_proj": (H, I), "up_proj": (H, I), "down_proj": (I, H)}.items():
            setattr(blk, name, MoeFusedLinear4bit(i, o, E, weight=getattr(blk, name).weight, quant_type="nf4", compress_statistics=False))
    blk = blk.to(DEV)
    static_in = randn((1, T, H), gen(0), 1.0, torch.bfloat16).to(DEV)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):          # first calls attach quant states and set kernel attributes
                blk(static_in)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out, static_logits = blk(static_in)
        for seed in (1, 2, 3):
            x = randn((1, T, H), gen(seed), 1.0, torch.bfloat16).to(DEV)
            eager_out, eager_logits = blk(x)            # eager work between the replays
            static_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, eager_out) and torch.equal(static_logits, eager_logits), seed


@pytest.mark.filterwarnings("ignore:The AccumulateGrad node's stream does not match")   # warm-up runs on a side stream
def test_lora_mlp_step_replays_from_a_hip_graph():
    """Forward and backward of the LoRA expert MLP (the products with the rank-r term in their reduction, the
    split-row dA/dB kernels with their workspace, the shared passes over x) captured once and replayed: every replay
    must equal the eager result for the inputs that are in the static buffers at that time."""
    R, E, H, M, r = 4608, 6, 256, 256, 16
    g = gen(5)
    mk = lambda *shape, scale: randn(shape, g, scale, torch.bfloat16).to(DEV)  # noqa: E731
    G, U, W = mk(E, M, H, scale=0.05), mk(E, M, H, scale=0.05), mk(E, H, M, scale=0.05)
    lora = [mk(*s, scale=0.05).requires_grad_() for s in ((E, r, H), (E, M, r), (E, r, H), (E, M, r), (E, r, M), (E, H, r))]
    ms = torch.bincount(torch.randint(0, E, (R,), generator=g), minlength=E).int().to(DEV)
    static_x = mk(R, H, scale=1.0).requires_grad_()
    static_dy = mk(R, H, scale=1.0)

    def step(x, dy):
        y = fast_lora(x, G, None, lora[0], lora[1], 2.0, U, None, lora[2], lora[3], 2.0, W, None, lora[4], lora[5], 1.5, ms)
        grads = torch.autograd.grad(y, [x] + lora, dy)
        return (y,) + grads

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(static_x, static_dy)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_x, static_dy)
    for seed in (1, 2, 3):
        gs = gen(100 + seed)
        x = randn((R, H), gs, 1.0, torch.bfloat16).to(DEV).requires_grad_()
        dy = randn((R, H), gs, 1.0, torch.bfloat16).to(DEV)
        eager = step(x, dy)                                   # eager work between the replays
        with torch.no_grad():
            static_x.copy_(x)
            static_dy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(static_out, eager):
            assert torch.equal(a, b), seed
