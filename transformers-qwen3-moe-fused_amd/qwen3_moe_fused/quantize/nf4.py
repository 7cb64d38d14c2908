"""NF4 blockwise quantisation state and the (de)quantise calls of the 4-bit path.

bitsandbytes supplies these to the reference (``quantize_nf4`` / ``dequantize_4bit`` /
``QuantState``; call sites qwen3_moe_fused/quantize/layer.py:21, kernels/fast_lora.py:62,
grouped_gemm/forward_4bit.py:142-152).  It is an optional import here: when present its
``QuantState`` objects are accepted as they are (the fields read are the ones the reference
reads: quant_type, blocksize, code, absmax, nested, state2, offset, shape, dtype); when absent
``Nf4QuantState`` carries the same fields.  The arithmetic is done by the HIP library either way.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Tuple

import torch

from .. import _lib

# The NF4 code book (16 quantiles of N(0,1) normalised to [-1, 1], with an exact zero).
NF4_CODE = (
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0,
)


def nf4_code(device) -> torch.Tensor:
    return torch.tensor(NF4_CODE, dtype=torch.float32, device=device)


@dataclass
class Nf4QuantState:
    """Field-compatible stand-in for bitsandbytes' ``QuantState`` (NF4 only)."""

    absmax: torch.Tensor                 # fp32 (n_blocks,), or uint8 when nested
    shape: Tuple[int, ...]               # logical shape of the unquantised weight
    code: torch.Tensor                   # fp32 (16,)
    blocksize: int = 64
    quant_type: str = "nf4"
    dtype: torch.dtype = torch.bfloat16  # dtype dequantize_4bit returns
    offset: Optional[torch.Tensor] = None
    state2: Optional[Any] = None         # nested: state of the 8-bit absmax (code (256,), absmax, blocksize)

    @property
    def nested(self) -> bool:
        return self.state2 is not None

    def to(self, device) -> "Nf4QuantState":
        self.absmax = self.absmax.to(device)
        self.code = self.code.to(device)
        if self.offset is not None:
            self.offset = self.offset.to(device)
        if self.state2 is not None:
            self.state2.absmax = self.state2.absmax.to(device)
            self.state2.code = self.state2.code.to(device)
        return self


@dataclass
class BlockwiseState:
    """State of an 8-bit blockwise-quantised tensor (the nested absmax)."""

    absmax: torch.Tensor
    code: torch.Tensor
    blocksize: int = 256


def resolve_absmax(quant_state) -> torch.Tensor:
    """fp32 absmax of an NF4 state, un-nesting a double-quantised one:
    ``dequantize_blockwise(absmax_u8, state2) + offset`` (forward_4bit.py:149-152)."""
    absmax = quant_state.absmax
    if getattr(quant_state, "nested", False):
        st2 = quant_state.state2
        out = torch.empty(absmax.numel(), device=absmax.device, dtype=torch.float32)
        code2 = st2.code.to(device=absmax.device, dtype=torch.float32).contiguous()
        absmax2 = st2.absmax.to(torch.float32).contiguous()
        rc = _lib.lib().mfl_dequant_blockwise_u8(_lib.ptr(absmax.contiguous()), _lib.ptr(code2), _lib.ptr(absmax2),
                                                 int(st2.blocksize), 0.0, _lib.ptr(out), absmax.numel(),
                                                 _lib.stream())
        _lib.check(rc, "mfl_dequant_blockwise_u8")
        offset = quant_state.offset
        if offset is not None:
            # the offset is a device scalar: add it on the device, never read it on the host
            out += offset.to(device=out.device, dtype=torch.float32) if torch.is_tensor(offset) else float(offset)
        return out
    assert absmax.dtype == torch.float32
    return absmax.contiguous()


def quantize_nf4(w: torch.Tensor, blocksize: int = 64) -> Tuple[torch.Tensor, Nf4QuantState]:
    """Blockwise NF4 quantisation on the GPU: returns (packed uint8 (numel/2, 1), state).
    Element 2i goes to the high nibble of byte i, 2i+1 to the low nibble."""
    assert w.is_cuda and w.is_contiguous()
    n = w.numel()
    assert n % blocksize == 0 and blocksize % 2 == 0
    code = nf4_code(w.device)
    packed = torch.empty((n // 2, 1), device=w.device, dtype=torch.uint8)
    absmax = torch.empty(n // blocksize, device=w.device, dtype=torch.float32)
    rc = _lib.lib().mfl_nf4_quant(_lib.ptr(w), _lib.dtype_code(w.dtype), n, blocksize, _lib.ptr(code), _lib.ptr(packed),
                                  _lib.ptr(absmax), _lib.stream())
    _lib.check(rc, "mfl_nf4_quant")
    return packed, Nf4QuantState(absmax=absmax, shape=tuple(w.shape), code=code, blocksize=blocksize, dtype=w.dtype)


def dequantize_nf4(packed: torch.Tensor, quant_state, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``code[nibble] * absmax[block]`` in fp32, rounded once to ``dtype`` (default: the state's)."""
    assert quant_state.quant_type == "nf4"
    assert packed.is_cuda and packed.is_contiguous()
    dtype = quant_state.dtype if dtype is None else dtype
    shape = tuple(quant_state.shape)
    n = packed.numel() * 2
    out = torch.empty(shape, device=packed.device, dtype=dtype)
    assert out.numel() == n
    absmax = resolve_absmax(quant_state)
    code = quant_state.code.to(device=packed.device, dtype=torch.float32).contiguous()
    rc = _lib.lib().mfl_nf4_dequant(_lib.ptr(packed), _lib.ptr(code), _lib.ptr(absmax), int(quant_state.blocksize),
                                    _lib.ptr(out), n, _lib.dtype_code(dtype), _lib.stream())
    _lib.check(rc, "mfl_nf4_dequant")
    return out


# name used at the reference's call sites
dequantize_4bit = dequantize_nf4
