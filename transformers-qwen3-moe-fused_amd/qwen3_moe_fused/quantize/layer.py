"""4-bit (NF4) expert projection (reference: qwen3_moe_fused/quantize/layer.py).

``moe_fused_linear_4bit`` runs the forward product straight off the packed weights (NF4 decode
fused into the grouped GEMM) instead of materialising the (E, N, K) weight as the reference does
(quantize/layer.py:17-22), and so does the input gradient.
``MoeFusedLinear4bit`` keeps the module contract: frozen packed ``weight`` carrying a
``quant_state``, compute-dtype handling (:54-74, :83-96) and the quant-state entries of
bitsandbytes' packed format in the state dict (:76-81): ``weight`` (uint8), ``weight.absmax``,
``weight.quant_map``, ``weight.quant_state.bitsandbytes__nf4`` (a JSON object as bytes) and, for a
double-quantised state, ``weight.nested_absmax`` / ``weight.nested_quant_map``.  The same entries
are read back by ``load_state_dict``.  bitsandbytes itself is not needed (and is not importable in
every environment); bit parity with its quantiser is not established, only the format.
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
                blocksize: int = 64, module: Optional[nn.Module] = None, quant_type: str = "nf4",
                compress_statistics: bool = False):
        data = torch.empty(0) if data is None else data
        self = torch.Tensor._make_subclass(cls, data, False)
        self.quant_state = quant_state
        self.blocksize = blocksize
        self.module = module
        self.quant_type = quant_type
        self.compress_statistics = compress_statistics
        return self

    def _like(self, data: torch.Tensor, quant_state) -> "Nf4Params":
        return Nf4Params(data, quant_state=quant_state, blocksize=self.blocksize, module=self.module,
                         quant_type=self.quant_type, compress_statistics=self.compress_statistics)

    def _quantized_on(self, device) -> "Nf4Params":
        w = self.data.contiguous().to(device)
        packed, state = quantize_nf4(w, self.blocksize, self.quant_type, self.compress_statistics)
        out = self._like(packed, state)
        if self.module is not None:
            self.module.quant_state = state
        return out

    def to(self, *args, **kwargs):
        device, dtype, non_blocking, _ = torch._C._nn._parse_to(*args, **kwargs)
        if device is not None and device.type == "cuda" and self.quant_state is None:
            return self._quantized_on(device)
        if self.quant_state is not None and device is not None:
            self.quant_state.to(device)
        return self._like(self.data.to(device=device, non_blocking=non_blocking), self.quant_state)

    def cuda(self, device=None, non_blocking: bool = False):
        return self.to(device="cuda" if device is None else device, non_blocking=non_blocking)


class MoeFusedLinear4bit(MoeFusedLinear):
    """Constructor arguments and their defaults are the reference's (quantize/layer.py:26-38);
    ``blocksize`` is an addition (bitsandbytes' default of 64)."""

    def __init__(self, in_features: int, out_features: int, num_experts: int, *,
                 weight: Optional[nn.Parameter] = None, compute_dtype: Optional[torch.dtype] = None,
                 compress_statistics: bool = True, quant_type: str = "fp4", blocksize: int = 64,
                 quant_storage: torch.dtype = torch.uint8, device: Optional[torch.device] = None) -> None:
        super().__init__(in_features, out_features, num_experts, device=device)
        if quant_type not in ("nf4", "fp4"):
            raise NotImplementedError(f"4-bit quantisation type {quant_type!r}")
        if quant_storage != torch.uint8:
            raise NotImplementedError("packed weights are stored as uint8")
        source = self.weight.data if weight is None else weight.data
        self.weight = Nf4Params(source, blocksize=blocksize, module=self, quant_type=quant_type,
                                compress_statistics=compress_statistics)
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
            for name, value in qs.as_dict(packed=True).items():
                destination[prefix + "weight." + name] = value if keep_vars else value.detach()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs) -> None:
        """Accepts what ``_save_to_state_dict`` writes (packed weight + quant-state entries) and, for a
        module that is still to be quantised, a plain floating-point (E, out, in) weight."""
        wkey = prefix + "weight"
        if wkey not in state_dict:
            if strict:
                missing_keys.append(wkey)
            return
        data = state_dict[wkey]
        entries = {k[len(wkey) + 1:]: v for k, v in state_dict.items() if k.startswith(wkey + ".")}
        old = self.weight
        shape = (self.num_experts, self.out_features, self.in_features)
        try:
            if entries:
                qs = Nf4QuantState.from_dict(entries, device=data.device)
                n = 1
                for d in qs.shape:
                    n *= int(d)
                if tuple(qs.shape) != shape or data.dtype != torch.uint8 or data.numel() * 2 != n:
                    raise ValueError(f"packed weight of {data.numel()} bytes / quant state of shape {tuple(qs.shape)} "
                                     f"do not describe a {shape} weight")
                new = Nf4Params(data.reshape(-1, 1).contiguous(), quant_state=qs, blocksize=int(qs.blocksize),
                                module=self, quant_type=qs.quant_type, compress_statistics=qs.nested)
                self.quant_state = qs
            else:
                if not data.dtype.is_floating_point or tuple(data.shape) != shape:
                    raise ValueError(f"expected a floating-point weight of shape {shape} or a packed weight with its "
                                     f"quant-state entries, got {tuple(data.shape)} {data.dtype}")
                new = Nf4Params(data.detach().clone(), blocksize=old.blocksize, module=self, quant_type=old.quant_type,
                                compress_statistics=old.compress_statistics)
                self.quant_state = None
                if data.is_cuda:
                    new = new.to(data.device)      # quantise right away, as moving the module would
        except (ValueError, KeyError) as exc:
            error_msgs.append(f"While loading {wkey}: {exc}")
            return
        self._parameters["weight"] = new

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
