"""Expert MLP with LoRA on gate/up/down as ONE autograd function
(reference: qwen3_moe_fused/kernels/fast_lora.py).

Shapes (rows B, hidden H, intermediate M, rank r, experts E):
    x (B,H);  G,U (E,M,H);  W (E,H,M);  Ag,Au (E,r,H);  Bg,Bu (E,M,r);  Aw (E,r,M);  Bw (E,H,r)
    e = G x + Sg Bg (Ag x),  g = U x + Su Bu (Au x),  h = silu(e) g,  y = W h + Sw Bw (Aw h)
Only e, g and the two rank-r activations Sg Ag x, Su Au x are kept for the backward pass.

Gradients.  With t = dOut Bproj (rows x r) and u = In Aproj^T (rows x r) for a projection
Out = (Wp + S Bp Ap) In:
    dAp = S t^T In        dBp = S dOut^T u        dIn = dOut Wp + S t Ap
Every LoRA gradient is therefore a rank-r grouped GEMM; the full (E, out, in) weight gradient
that the reference forms and then contracts (fast_lora.py:139-149) is never built.  Base weights
may be NF4 (``*qs`` not None): the forward and the input-gradient products decode them inside
the GEMM (the reference dequantises, fast_lora.py:57-62 "TODO: Fuse dequant and linear").
"""
from __future__ import annotations

import torch

from ..grouped_gemm.backward_dw import grouped_gemm_backward_dw as _dw
from ..grouped_gemm.forward import grouped_gemm_forward as _fwd
from ..grouped_gemm.forward_4bit import grouped_gemm_forward_4bit as _fwd4
from ..grouped_gemm.forward_4bit import grouped_gemm_forward_transposed_4bit as _dx4
from ..grouped_gemm.forward_transposed import grouped_gemm_forward_transposed as _dx
from ..grouped_gemm.fused import grouped_gemm_forward_4bit_lora as _fwd4_lora
from ..grouped_gemm.fused import grouped_gemm_forward_lora as _fwd_lora
from ..grouped_gemm.fused import grouped_glu_forward_lora as _glu_lora
from ..grouped_gemm.fused import grouped_gemm_forward_transposed_4bit_lora as _dx4_lora
from ..grouped_gemm.fused import grouped_gemm_forward_transposed_lora as _dx_lora
from ..quantize.nf4 import dequantize_nf4
from .silu_mul import silu_mul_backward_inplace, silu_mul_forward


def _base_fwd(x, wq, wqs, m_sizes):
    if wqs is None:
        return _fwd(x, wq.to(x.dtype), m_sizes)
    if x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and int(wqs.blocksize) >= 8:
        return _fwd4(x, wq, wqs, m_sizes)
    return _fwd(x, dequantize_nf4(wq, wqs, x.dtype), m_sizes)


def _dense(wq, wqs, dtype):
    return wq.to(dtype) if wqs is None else dequantize_nf4(wq, wqs, dtype)


def _proj_fwd(x, wq, wqs, a, b, s, m_sizes, us=None):
    """y = x W^T + (s x A^T) B^T; returns y and the scaled rank-r activation s x A^T (rows x r)."""
    if us is None:
        us = _fwd(x, a, m_sizes, alpha=s)
    if wqs is None and x.dtype == torch.bfloat16:
        # bf16 weights: the rank-r term rides in the reduction of the base product (no second pass over y)
        return _fwd_lora(x, wq.to(x.dtype), us, b, m_sizes), us
    if wqs is not None and x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and int(wqs.blocksize) >= 8:
        return _fwd4_lora(x, wq, wqs, us, b, m_sizes), us   # the same over packed NF4 weights
    y = _base_fwd(x, wq, wqs, m_sizes)
    _fwd(us, b, m_sizes, out=y, accumulate=True)             # y += us b^T
    return y, us


def _proj_bwd_input(dout, ts, wq, wqs, a, m_sizes, out=None):
    """dIn (+)= dOut W + ts A with ts = s dOut B (rows x r)."""
    if wqs is None and dout.dtype == torch.bfloat16 and out is None:
        return _dx_lora(dout, wq.to(dout.dtype), ts, a, m_sizes)
    if wqs is not None and dout.dtype == torch.bfloat16 and out is None:
        return _dx4_lora(dout, wq, wqs, ts, a, m_sizes)
    if wqs is not None and dout.dtype == torch.bfloat16:
        out = _dx4(dout, wq, wqs, m_sizes, out=out, accumulate=out is not None)
    else:
        out = _dx(dout, _dense(wq, wqs, dout.dtype), m_sizes, out=out, accumulate=out is not None)
    return _dx(ts, a, m_sizes, out=out, accumulate=True)


# from this many rows on, two thin products that stream the same wide operand are run as one of twice the rank
_WIDE_ROWS = 4096


class FastLora(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, Gq, Gqs, Ag, Bg, Sg, Uq, Uqs, Au, Bu, Su, Wq, Wqs, Aw, Bw, Sw, m_sizes):
        dt = x.dtype
        x = x.contiguous()
        Ag, Bg, Au, Bu, Aw, Bw = (p.to(dt).contiguous() for p in (Ag, Bg, Au, Bu, Aw, Bw))
        ug = uu = ucat = None
        if Sg == Su and Ag.shape == Au.shape and x.shape[0] >= _WIDE_ROWS:
            # one pass over x for both adapters' rank-r activations
            r = Ag.shape[1]
            ucat = _fwd(x, torch.cat((Ag, Au), dim=1), m_sizes, alpha=Sg)
            ug, uu = ucat[:, :r].contiguous(), ucat[:, r:].contiguous()
        if (ucat is not None and Gqs is None and Uqs is None and dt == torch.bfloat16 and Gq.dtype == dt
                and Uq.dtype == dt and Bg.shape == Bu.shape):
            # gate, up, both rank-r terms and the SiLU-mul in one launch: each matrix's thin weights are its
            # adapter's B over its own columns of ucat and zeros over the other's
            zeros = torch.zeros_like(Bg)
            h, e, g = _glu_lora(x, Gq, Uq, ucat, torch.cat((Bg, zeros), dim=2), torch.cat((zeros, Bu), dim=2), m_sizes)
        else:
            e, ug = _proj_fwd(x, Gq, Gqs, Ag, Bg, Sg, m_sizes, ug)
            g, uu = _proj_fwd(x, Uq, Uqs, Au, Bu, Su, m_sizes, uu)
            h = silu_mul_forward(e, g)
        y, _ = _proj_fwd(h, Wq, Wqs, Aw, Bw, Sw, m_sizes)
        ctx.frozen = (Gq, Gqs, Sg, Uq, Uqs, Su, Wq, Wqs, Sw, m_sizes)
        ctx.save_for_backward(x, Ag, Bg, Au, Bu, Aw, Bw, e, g, ug, uu)
        return y

    @staticmethod
    def backward(ctx, dy):
        Gq, Gqs, Sg, Uq, Uqs, Su, Wq, Wqs, Sw, m_sizes = ctx.frozen
        x, Ag, Bg, Au, Bu, Aw, Bw, e, g, ug, uu = ctx.saved_tensors
        dt = x.dtype
        dy = dy.contiguous()

        # The rank-r activations carry the adapter's scaling (ug, uu from the forward pass; tw, tu, tg here),
        # so every product below takes them as they are.
        # down projection
        tw = _dx(dy, Bw, m_sizes, alpha=Sw)                            # Sw dy Bw, rows x r
        dh = _proj_bwd_input(dy, tw, Wq, Wqs, Aw, m_sizes)
        silu_mul_backward_inplace(dh, e, g)                            # (dh, e, g) <- (h, de, dg)
        h, de, dg = dh, e, g
        dAw = _dw(h, tw, m_sizes, dt)                                  # (E, r, M)
        dBw = _dw(_fwd(h, Aw, m_sizes, alpha=Sw), dy, m_sizes, dt)     # (E, H, r)

        # up and gate projections
        tu = _dx(dg, Bu, m_sizes, alpha=Su)
        tg = _dx(de, Bg, m_sizes, alpha=Sg)
        tcat = torch.cat((tg, tu), dim=1)
        if tg.shape == tu.shape and x.shape[0] >= _WIDE_ROWS and 2 * tg.shape[1] <= 64:
            # one pass over x for both: (E, 2 r, H)
            r = tg.shape[1]
            dAcat = _dw(x, tcat, m_sizes, dt)
            dAg, dAu = dAcat[:, :r].contiguous(), dAcat[:, r:].contiguous()  # gradients of their own, not views
        else:
            dAu = _dw(x, tu, m_sizes, dt)                              # (E, r, H)
            dAg = _dw(x, tg, m_sizes, dt)
        dBu = _dw(uu, dg, m_sizes, dt)                                 # (E, M, r)
        dBg = _dw(ug, de, m_sizes, dt)

        dx = None
        if ctx.needs_input_grad[0]:
            if Gqs is None and Uqs is None and dt == torch.bfloat16 and Gq.dtype == dt and Uq.dtype == dt:
                # both base terms and both rank-r terms (side by side as one term of rank 2 r) in one reduction
                dx = _dx_lora(de, Gq, tcat, torch.cat((Ag, Au), dim=1), m_sizes, dy2=dg, w2=Uq)
            else:
                # both rank-r terms with the first base product, the second base product accumulates
                dx = _proj_bwd_input(de, tcat, Gq, Gqs, torch.cat((Ag, Au), dim=1), m_sizes)
                if Uqs is not None and dt == torch.bfloat16:
                    _dx4(dg, Uq, Uqs, m_sizes, out=dx, accumulate=True)
                else:
                    _dx(dg, _dense(Uq, Uqs, dt), m_sizes, out=dx, accumulate=True)

        return (dx, None, None, dAg, dBg, None, None, None, dAu, dBu, None, None, None, dAw, dBw, None, None)


fast_lora = FastLora.apply
