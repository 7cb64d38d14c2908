"""GPU parity of SiLU-mul and of NF4 / 8-bit blockwise (de)quantisation."""
import numpy as np
import pytest
import torch

import oracle
from util import check_close, gen, randn, to_np32

pytestmark = pytest.mark.gpu

from qwen3_moe_fused.kernels.silu_mul import (silu_mul, silu_mul_backward, silu_mul_backward_inplace,  # noqa: E402
                                              silu_mul_forward)
from qwen3_moe_fused.quantize.nf4 import (BlockwiseState, Nf4QuantState, dequantize_nf4, nf4_code,  # noqa: E402
                                          quantize_nf4)

DEV = "cuda"


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16)


def _ulp_diff_bf16(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, 0x8000 - (u & 0x7FFF) - 1, u + 0x8000)
    return np.abs(key(a_bits) - key(b_bits))


def _two_roundings_close(d: np.ndarray) -> None:
    """bf16 steps between two results of `round(round(silu(e)) * x)`: at most two, and rarely any."""
    assert d.max() <= 2
    assert (d > 1).sum() <= max(1, 1e-5 * d.size) and (d > 0).sum() <= max(2, 1e-3 * d.size)


@pytest.mark.parametrize("shape", [(32768, 768), (91, 3), (1, 1), (1000, 7)])
def test_silu_mul_bf16(shape):
    g = gen(shape[0])
    e, gg, dh = (randn(shape, g, 2.0, torch.bfloat16) for _ in range(3))
    h = silu_mul_forward(e.to(DEV), gg.to(DEV))
    h_ref = oracle.silu_mul_fwd_bf16(_bits(e), _bits(gg))
    # same rounding chain; the sigmoid differs by a few fp32 ulps between CPU and GPU, which now
    # and then moves silu(e) by one bf16 step, and the rounding of the product can add one more
    _two_roundings_close(_ulp_diff_bf16(_bits(h), h_ref))
    de, dg = silu_mul_backward(dh.to(DEV), e.to(DEV), gg.to(DEV))
    h_r, de_r, dg_r = oracle.silu_mul_bwd_bf16(_bits(dh), _bits(e), _bits(gg))
    assert _ulp_diff_bf16(_bits(de), de_r).max() <= 2 and (_ulp_diff_bf16(_bits(de), de_r) > 0).mean() < 5e-3
    _two_roundings_close(_ulp_diff_bf16(_bits(dg), dg_r))  # dg = silu(e) * dh: two roundings, like h
    # in-place variant: (dh, e, g) <- (h, de, dg)
    a, b, c = dh.to(DEV).clone(), e.to(DEV).clone(), gg.to(DEV).clone()
    silu_mul_backward_inplace(a, b, c)
    assert torch.equal(a, h) and torch.equal(b, de) and torch.equal(c, dg)


def test_silu_mul_fp32_and_autograd():
    g = gen(3)
    e, gg, dh = (randn((333, 17), g, 2.0) for _ in range(3))
    h = silu_mul_forward(e.to(DEV), gg.to(DEV))
    np.testing.assert_allclose(h.cpu().numpy(), oracle.silu_mul_fwd_f32(e.numpy(), gg.numpy()), rtol=1e-5, atol=1e-6)
    ed, gd = e.to(DEV).requires_grad_(), gg.to(DEV).requires_grad_()
    silu_mul(ed, gd).backward(dh.to(DEV))
    e2, g2 = e.double().requires_grad_(), gg.double().requires_grad_()
    (torch.nn.functional.silu(e2) * g2).backward(dh.double())
    np.testing.assert_allclose(ed.grad.cpu().numpy(), e2.grad.float().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gd.grad.cpu().numpy(), g2.grad.float().numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("blocksize", [64, 256, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_nf4_dequant_bit_exact(blocksize, dtype):
    n = 8 * 96 * 128
    w = randn((8, 96, 128), gen(blocksize), 0.02)
    q_ref, absmax_ref = oracle.nf4_quant(w.numpy(), blocksize)
    state = Nf4QuantState(absmax=torch.from_numpy(absmax_ref).to(DEV), shape=(8, 96, 128), code=nf4_code(DEV),
                          blocksize=blocksize, dtype=dtype)
    out = dequantize_nf4(torch.from_numpy(q_ref).view(-1, 1).to(DEV), state)
    assert out.shape == (8, 96, 128) and out.dtype == dtype
    ref32 = oracle.nf4_dequant(q_ref, absmax_ref, blocksize)
    if dtype == torch.bfloat16:
        ref_bits = oracle.nf4_dequant(q_ref, absmax_ref, blocksize, bf16=True)
        assert np.array_equal(_bits(out).reshape(-1), ref_bits), "NF4 -> bf16 must be bit exact"
    elif dtype == torch.float32:
        assert np.array_equal(out.cpu().numpy().reshape(-1), ref32)
    else:
        assert np.array_equal(out.cpu().numpy().reshape(-1), ref32.astype(np.float16))
    assert n == out.numel()


@pytest.mark.parametrize("shape,blocksize", [((5, 36, 20), 8), ((7, 40, 24), 32), ((3, 50, 14), 4), ((1, 2, 2), 2),
                                             ((2, 1000, 264), 64)])
def test_nf4_dequant_ragged_sizes(shape, blocksize):
    # sizes that end inside a wave's group of packed dwords, and blocks too small for the vector path
    w = randn(shape, gen(blocksize + shape[1]), 0.02)
    q_ref, absmax_ref = oracle.nf4_quant(w.numpy(), blocksize)
    for dtype in (torch.bfloat16, torch.float32):
        state = Nf4QuantState(absmax=torch.from_numpy(absmax_ref).to(DEV), shape=shape, code=nf4_code(DEV),
                              blocksize=blocksize, dtype=dtype)
        out = dequantize_nf4(torch.from_numpy(q_ref).view(-1, 1).to(DEV), state)
        assert out.shape == shape and out.dtype == dtype
        if dtype == torch.bfloat16:
            ref_bits = oracle.nf4_dequant(q_ref, absmax_ref, blocksize, bf16=True)
            assert np.array_equal(_bits(out).reshape(-1), ref_bits)
        else:
            assert np.array_equal(out.cpu().numpy().reshape(-1), oracle.nf4_dequant(q_ref, absmax_ref, blocksize))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_nf4_quant_matches_oracle_and_round_trips(dtype):
    w = randn((4, 64, 128), gen(77), 0.02, dtype)
    packed, state = quantize_nf4(w.to(DEV), 64)
    q_ref, absmax_ref = oracle.nf4_quant(to_np32(w), 64)
    assert packed.shape == (w.numel() // 2, 1) and packed.dtype == torch.uint8
    assert np.array_equal(packed.cpu().numpy().reshape(-1), q_ref)
    assert np.array_equal(state.absmax.cpu().numpy(), absmax_ref)
    # quantising the dequantised weights reproduces the same codes
    deq = dequantize_nf4(packed, state, torch.float32)
    packed2, state2 = quantize_nf4(deq, 64)
    assert torch.equal(packed2, packed)
    # error bound of 4-bit blockwise quantisation: half the widest code gap times absmax
    err = (deq.cpu() - w.float()).abs().view(-1, 64)
    assert (err <= 0.16 * state.absmax.cpu()[:, None] + 1e-7).all()


def test_nested_absmax():
    """Double-quantised absmax: absmax = code256[u8] * absmax2[i / 256] + offset (forward_4bit.py:149-152)."""
    g = gen(8)
    w = randn((2, 64, 256), g, 0.02)
    q_ref, absmax_ref = oracle.nf4_quant(w.numpy(), 64)
    nblk = absmax_ref.size                                   # 512
    code256 = torch.sort(torch.rand(256, generator=g) * 2 - 1).values.contiguous()
    u8 = torch.randint(0, 256, (nblk,), generator=g, dtype=torch.uint8)
    absmax2 = torch.rand(nblk // 256, generator=g) + 0.5
    offset = torch.tensor(0.0123)
    am_ref = oracle.dequant_blockwise_u8(u8.numpy(), code256.numpy(), absmax2.numpy(), 256, float(offset))
    state = Nf4QuantState(absmax=u8.to(DEV), shape=(2, 64, 256), code=nf4_code(DEV), blocksize=64,
                          dtype=torch.bfloat16, offset=offset.to(DEV),
                          state2=BlockwiseState(absmax=absmax2.to(DEV), code=code256.to(DEV), blocksize=256))
    out = dequantize_nf4(torch.from_numpy(q_ref).view(-1, 1).to(DEV), state)
    ref_bits = oracle.nf4_dequant(q_ref, am_ref, 64, bf16=True)
    assert np.array_equal(_bits(out).reshape(-1), ref_bits)
