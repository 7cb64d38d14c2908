#!/usr/bin/env python3
"""Writes tests/golden/config1.npz: benchmark configuration 1 (seed 0; 8 experts, 64 -> 128 features,
256 tokens routed top-2 -> 512 rows) with expected outputs.

The reference holds no golden vectors for this path, and every function on it reduces to a
library routine, so the expected values are produced here by stock torch routines in float64
(einsum, autograd, softmax/topk, stable argsort) -- neither by the reference (not imported)
nor by the oracle (which these vectors are used to check).  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1.npz")


def main() -> None:
    g = torch.Generator().manual_seed(0)
    E, K, N, T, k = 8, 64, 128, 256, 2
    hidden = torch.randn((T, K), generator=g)
    weight = torch.randn((E, N, K), generator=g) * 0.02
    logits = torch.randn((T, E), generator=g)
    grad_out = torch.randn((T * k, N), generator=g)

    p = torch.softmax(logits, dim=1, dtype=torch.float32)
    routing_weights, selected = torch.topk(p, k, dim=-1)
    gaps = (routing_weights[:, :-1] - routing_weights[:, 1:]).min()
    kth_vs_next = (routing_weights[:, -1] - torch.sort(p, descending=True).values[:, k]).min()
    assert gaps > 1e-6 and kth_vs_next > 1e-6, "config 1 routing must be tie-free"
    sel = selected.reshape(-1)                                   # (512,) unsorted, token-major
    x = hidden.repeat_interleave(k, dim=0)                       # row b = token b // k

    xd = x.double().requires_grad_()
    wd = weight.double().requires_grad_()
    out = torch.einsum("bnk,bk->bn", wd[sel], xd)
    out.backward(grad_out.double())

    order = torch.argsort(sel, stable=True)
    inv = torch.empty_like(order)
    inv[order] = torch.arange(order.numel())
    np.savez_compressed(
        OUT,
        hidden=hidden.numpy(), weight=weight.numpy(), logits=logits.numpy(), grad_out=grad_out.numpy(),
        routing_weights=routing_weights.numpy(), selected_experts=selected.numpy(),
        m_sizes=torch.bincount(sel, minlength=E).to(torch.int32).numpy(),
        sort_idx=order.to(torch.int32).numpy(), inv_sort_idx=inv.to(torch.int32).numpy(),
        out=out.detach().float().numpy(), grad_input=xd.grad.float().numpy(), grad_weight=wd.grad.float().numpy(),
    )
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
