"""Fused-format LoRA for ``MoeFusedLinear`` (reference: qwen3_moe_fused/lora.py).

``lora_A`` is a ``MoeFusedLinear(in, r, E)`` and ``lora_B`` a ``MoeFusedLinear(r, out, E)``
(lora.py:71-72), so an adapter is two rank-r grouped GEMMs:
    result = base(x, m_sizes) + lora_B(lora_A(dropout(x), m_sizes), m_sizes) * scaling   (lora.py:134)
with scaling = alpha / r, or alpha / sqrt(r) for rsLoRA (:74-77); A is Kaiming-uniform, B zero (:94-95).
Merging, DoRA, LoRA bias and mixed-adapter batches are not implemented, as in the reference.

When PEFT is installed the class derives from its ``LoraLayer`` and ``patch_lora_config``
registers it as the custom module for ``MoeFusedLinear``; without PEFT a small stand-in base
keeps the same attributes (r, lora_alpha, scaling, lora_dropout, lora_A, lora_B, active adapter
bookkeeping) so the layer, and the fast path that reads those attributes, work unchanged.
"""
from __future__ import annotations

import math
from typing import Optional, Union

import torch
from torch import nn

from .modular_qwen3_moe_fused import MoeFusedLinear, moe_fused_kaiming_uniform_

try:  # pragma: no cover - depends on the environment
    from peft import LoraConfig
    from peft.tuners.lora.layer import LoraLayer

    HAVE_PEFT = True
except ImportError:
    HAVE_PEFT = False
    LoraConfig = None

    class LoraLayer:  # type: ignore[no-redef]
        """The slice of PEFT's ``LoraLayer`` that a single-adapter LoRA layer uses."""

        adapter_layer_names = ("lora_A", "lora_B")

        def __init__(self, base_layer: nn.Module, **kwargs) -> None:
            self.base_layer = base_layer
            self.r, self.lora_alpha, self.scaling = {}, {}, {}
            self.lora_dropout = nn.ModuleDict()
            self.lora_A = nn.ModuleDict()
            self.lora_B = nn.ModuleDict()
            self._disable_adapters = False
            self.merged_adapters: list[str] = []
            self.in_features = base_layer.in_features
            self.out_features = base_layer.out_features
            self.kwargs = kwargs

        def get_base_layer(self) -> nn.Module:
            return self.base_layer

        @property
        def merged(self) -> bool:
            return bool(self.merged_adapters)

        @property
        def disable_adapters(self) -> bool:
            return self._disable_adapters

        def enable_adapters(self, enabled: bool) -> None:
            self._disable_adapters = not enabled
            for p in list(self.lora_A.parameters()) + list(self.lora_B.parameters()):
                p.requires_grad_(enabled)

        @property
        def active_adapter(self):
            return self._active_adapter

        @property
        def active_adapters(self) -> list[str]:
            a = self._active_adapter
            return [a] if isinstance(a, str) else list(a)

        def set_adapter(self, adapter_names) -> None:
            names = [adapter_names] if isinstance(adapter_names, str) else list(adapter_names)
            for key, mod in list(self.lora_A.items()) + list(self.lora_B.items()):
                mod.requires_grad_(key in names)
            self._active_adapter = names

        def _move_adapter_to_device_of_base_layer(self, adapter_name: str) -> None:
            weight = self.base_layer.weight
            dtype = weight.dtype if weight.dtype.is_floating_point else None
            self.lora_A[adapter_name].to(device=weight.device, dtype=dtype)
            self.lora_B[adapter_name].to(device=weight.device, dtype=dtype)

        def _check_forward_args(self, x, *args, **kwargs) -> None:
            return None

        def _cast_input_dtype(self, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
            return x if x.dtype == dtype else x.to(dtype)


class LoraMoeFusedLinear(nn.Module, LoraLayer):
    def __init__(self, base_layer: MoeFusedLinear, adapter_name: str, r: int = 0, lora_alpha: int = 1,
                 lora_dropout: float = 0.0, init_lora_weights: Union[bool, str] = True, use_rslora: bool = False,
                 use_dora: bool = False, lora_bias: bool = False, **kwargs) -> None:
        if init_lora_weights not in (True, False) or use_dora or lora_bias:
            raise NotImplementedError("only plain LoRA (no DoRA, no LoRA bias, default/no init) is implemented")
        nn.Module.__init__(self)
        LoraLayer.__init__(self, base_layer, **kwargs)
        self.num_experts = base_layer.num_experts
        self._active_adapter = adapter_name
        self.update_layer(adapter_name, r, lora_alpha=lora_alpha, lora_dropout=lora_dropout,
                          init_lora_weights=init_lora_weights, use_rslora=use_rslora)

    def update_layer(self, adapter_name: str, r: int, lora_alpha: int, lora_dropout: float,
                     init_lora_weights: Union[bool, str], use_rslora: bool, **kwargs) -> None:
        if r <= 0:
            raise ValueError(f"`r` should be a positive integer value but the value passed is {r}")
        self.r[adapter_name] = r
        self.lora_alpha[adapter_name] = lora_alpha
        self.lora_dropout.update({adapter_name: nn.Dropout(p=lora_dropout) if lora_dropout > 0.0 else nn.Identity()})
        self.lora_A[adapter_name] = MoeFusedLinear(self.in_features, r, self.num_experts)
        self.lora_B[adapter_name] = MoeFusedLinear(r, self.out_features, self.num_experts)
        self.scaling[adapter_name] = lora_alpha / (math.sqrt(r) if use_rslora else r)
        if init_lora_weights is True:
            self.reset_lora_parameters(adapter_name, init_lora_weights)
        self._move_adapter_to_device_of_base_layer(adapter_name)
        self.set_adapter(self.active_adapters)

    def reset_lora_parameters(self, adapter_name: str, init_lora_weights: Union[bool, str]) -> None:
        if init_lora_weights is False or adapter_name not in self.lora_A:
            return
        if init_lora_weights is not True:
            raise ValueError(f"Unknown initialization {init_lora_weights=}")
        moe_fused_kaiming_uniform_(self.lora_A[adapter_name].weight)
        nn.init.zeros_(self.lora_B[adapter_name].weight)

    def merge(self, safe_merge: bool = False, adapter_names: Optional[list[str]] = None) -> None:
        raise NotImplementedError

    def unmerge(self) -> None:
        raise NotImplementedError

    def forward(self, x: torch.Tensor, m_sizes: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        self._check_forward_args(x, *args, **kwargs)
        if kwargs.pop("adapter_names", None) is not None:
            raise NotImplementedError("mixed-adapter batches are not implemented")
        result = self.base_layer(x, m_sizes, *args, **kwargs)
        if self.disable_adapters or self.merged:
            return result
        out_dtype = result.dtype
        for name in self.active_adapters:
            if name not in self.lora_A:
                continue
            a, b = self.lora_A[name], self.lora_B[name]
            x = self._cast_input_dtype(x, a.weight.dtype)
            low_rank = a(self.lora_dropout[name](x), m_sizes)
            result = result + b(low_rank, m_sizes) * self.scaling[name]
        return result.to(out_dtype)

    def __repr__(self) -> str:
        return "lora." + super().__repr__()


def patch_lora_config(*, rank_pattern: Optional[dict[str, int]] = None) -> None:
    """Make every new PEFT ``LoraConfig`` map ``MoeFusedLinear`` to ``LoraMoeFusedLinear`` and, if
    given, carry ``rank_pattern`` (lora.py:145-154).  Needs PEFT."""
    if not HAVE_PEFT:
        raise ImportError("patch_lora_config needs the `peft` package; wrap modules with LoraMoeFusedLinear directly")
    original = LoraConfig.__init__

    def patched(self, *args, **kwargs):
        original(self, *args, **kwargs)
        self._register_custom_module({MoeFusedLinear: LoraMoeFusedLinear})
        if rank_pattern is not None:
            self.rank_pattern = rank_pattern

    LoraConfig.__init__ = patched
