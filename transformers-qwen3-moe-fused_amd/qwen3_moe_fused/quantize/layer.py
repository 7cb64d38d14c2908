"""4-bit (NF4) expert projection (reference: qwen3_moe_fused/quantize/layer.py).

``moe_fused_linear_4bit`` runs the forward product straight off the packed weights (NF4 decode
fused into the grouped GEMM) instead of materialising the (E, N, K) weight as the reference does
(quantize/layer.py:17-22), and so does the input gradient.
``MoeFusedLinear4bit`` keeps the module contract: frozen packed ``weight`` carrying a
``quant_state``, compute-dtype handling (:54-74, :83-96) and quant-state entries in the state
dict (:76-81).
"""
from __future__ import annotations

import warnings
from typing import Any, Optional

import torch
from torch import nn

from ..grouped_gemm.forward import grouped_gemm_forward
from ..grouped_gemm.forward_4bit import grouped_gemm_forward_4bit, grouped_gemm_forward_transposed_4bit
from ..modular_qwen3_moe_fused import MoeFusedLinear
from .nf4 import Nf4QuantState, dequantize_nf4, quantize_nf4


class _GroupedGemm4bit(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, packed, quant_state, m_sizes):
        ctx.quant_state = quant_state
        ctx.save_for_backward(packed, m_sizes)
        if x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and int(quant_state.blocksize) >= 8:
            return grouped_gemm_forward_4bit(x, packed, quant_state, m_sizes)
        return grouped_gemm_forward(x, dequantize_nf4(packed, quant_state, x.dtype), m_sizes)

    @staticmethod
    def backward(ctx, dy):
        packed, m_sizes = ctx.saved_tensors
        dx = None
        if ctx.needs_input_grad[0]:
            dx = grouped_gemm_forward_transposed_4bit(dy.contiguous(), packed, ctx.quant_state, m_sizes, dy.dtype)
        return dx, None, None, None


def moe_fused_linear_4bit(input: torch.Tensor, weight: torch.Tensor, m_sizes: torch.Tensor) -> torch.Tensor:
    """``weight``: packed NF4 tensor with a ``quant_state`` attribute (shape (E, N, K)); frozen."""
    assert not weight.requires_grad
    return _GroupedGemm4bit.apply(input, weight.data if isinstance(weight, nn.Parameter) else weight,
                                  weight.quant_state, m_sizes)


class Nf4Params(nn.Parameter):
    """Frozen parameter that is quantised to NF4 when it first reaches the GPU (the behaviour of
    bitsandbytes' ``Params4bit`` that the reference module relies on, quantize/layer.py:40-47)."""

    def __new__(cls, data: Optional[torch.Tensor] = None, quant_state: Optional[Nf4QuantState] = None,
                blocksize: int = 64, module: Optional[nn.Module] = None):
        data = torch.empty(0) if data is None else data
        self = torch.Tensor._make_subclass(cls, data, False)
        self.quant_state = quant_state
        self.blocksize = blocksize
        self.module = module
        return self

    def _quantized_on(self, device) -> "Nf4Params":
        w = self.data.contiguous().to(device)
        packed, state = quantize_nf4(w, self.blocksize)
        out = Nf4Params(packed, quant_state=state, blocksize=self.blocksize, module=self.module)
        if self.module is not None:
            self.module.quant_state = state
        return out

    def to(self, *args, **kwargs):
        device, dtype, non_blocking, _ = torch._C._nn._parse_to(*args, **kwargs)
        if device is not None and device.type == "cuda" and self.quant_state is None:
            return self._quantized_on(device)
        if self.quant_state is not None and device is not None:
            self.quant_state.to(device)
        new = Nf4Params(self.data.to(device=device, non_blocking=non_blocking), quant_state=self.quant_state,
                        blocksize=self.blocksize, module=self.module)
        return new

    def cuda(self, device=None, non_blocking: bool = False):
        return self.to(device="cuda" if device is None else device, non_blocking=non_blocking)


class MoeFusedLinear4bit(MoeFusedLinear):
    def __init__(self, in_features: int, out_features: int, num_experts: int, *,
                 weight: Optional[nn.Parameter] = None, compute_dtype: Optional[torch.dtype] = None,
                 compress_statistics: bool = False, quant_type: str = "nf4", blocksize: int = 64,
                 quant_storage: torch.dtype = torch.uint8, device: Optional[torch.device] = None) -> None:
        super().__init__(in_features, out_features, num_experts, device=device)
        if quant_type != "nf4":
            raise NotImplementedError("only NF4 is implemented")
        if compress_statistics:
            raise NotImplementedError("double quantisation is accepted on load (nested quant states) but not produced")
        source = self.weight.data if weight is None else weight.data
        self.weight = Nf4Params(source, blocksize=blocksize, module=self)
        self.compute_dtype = compute_dtype
        self.compute_type_is_set = compute_dtype is not None
        self.quant_state = None
        self.quant_storage = quant_storage

    def _apply(self, fn, recurse=True):
        # nn.Module._apply would swap the data under the Parameter subclass and drop its quant state:
        # take the packed weight out, let the module move everything else, move the weight ourselves.
        packed = self._parameters.pop("weight")
        try:
            super()._apply(fn, recurse)
            target = fn(torch.empty(0, device=packed.device)).device
            moved = packed.to(target) if isinstance(packed, Nf4Params) else fn(packed)
        finally:
            self._parameters["weight"] = packed
        self._parameters["weight"] = moved
        self.quant_state = getattr(moved, "quant_state", None)
        return self

    def set_compute_type(self, x: torch.Tensor) -> None:
        if x.dtype in (torch.float32, torch.bfloat16):
            self.compute_dtype = x.dtype  # safe to compute in the input type
        elif x.dtype == torch.float16 and self.compute_dtype in (None, torch.float32):
            warnings.warn("fp16 input with an fp32 compute dtype: the 4-bit expert projection will be slow")

    def _save_to_state_dict(self, destination: dict[str, Any], prefix: str, keep_vars: bool) -> None:
        super()._save_to_state_dict(destination, prefix, keep_vars)
        qs = getattr(self.weight, "quant_state", None)
        if qs is not None:
            entries = {"absmax": qs.absmax, "quant_map": qs.code,
                       "quant_state.blocksize": torch.tensor(int(qs.blocksize)),
                       "quant_state.shape": torch.tensor(list(qs.shape))}
            for name, value in entries.items():
                destination[prefix + "weight." + name] = value if keep_vars else value.detach()

    def forward(self, x: torch.Tensor, m_sizes: torch.Tensor) -> torch.Tensor:
        if getattr(self.weight, "quant_state", None) is None:
            if self.quant_state is None:
                raise RuntimeError("MoeFusedLinear4bit has no quantised weight yet: move the module to the GPU first")
            self.weight.quant_state = self.quant_state
        if not self.compute_type_is_set:
            self.set_compute_type(x)
            self.compute_type_is_set = True
        in_dtype = x.dtype
        if self.compute_dtype is not None:
            x = x.to(self.compute_dtype)
        return moe_fused_linear_4bit(x, self.weight, m_sizes).to(in_dtype)
