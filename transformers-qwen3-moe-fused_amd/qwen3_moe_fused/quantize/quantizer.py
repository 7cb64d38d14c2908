"""bitsandbytes-4-bit loading of fused MoE models through transformers' quantizer hook
(reference: qwen3_moe_fused/quantize/quantizer.py).

transformers' ``Bnb4BitHfQuantizer`` swaps ``nn.Linear`` for bitsandbytes' ``Linear4bit`` before the
weights are loaded; it does not know ``MoeFusedLinear``.  ``patch_bnb_quantizer()`` replaces its
``_process_model_before_weight_loading`` (quantizer.py:109-133 of the reference) with one that also
swaps ``MoeFusedLinear`` for ``MoeFusedLinear4bit`` (:21-88), honouring ``modules_to_not_convert``.
The hook is written against the transformers release that is installed (its signature has no
``keep_in_fp32_modules`` argument any more: the list comes from the model) and still accepts the older
keyword.

``nn.Linear`` / ``Conv1D`` modules are converted to bitsandbytes' ``Linear4bit`` as in the reference
when bitsandbytes is importable; without it they are left as they are (the expert projections, which
are what the fused format is about, do not need it).  A full ``from_pretrained(quantization_config=...)``
additionally passes transformers' own environment check, which requires bitsandbytes.
"""
from __future__ import annotations

from inspect import signature
from typing import Any, Optional, Union

import torch
from torch import nn

from ..modular_qwen3_moe_fused import MoeFusedLinear
from .layer import MoeFusedLinear4bit

try:  # pragma: no cover - depends on the environment
    from bitsandbytes.nn import Linear4bit
except ImportError:
    Linear4bit = None

try:
    from transformers.pytorch_utils import Conv1D
except ImportError:  # pragma: no cover
    Conv1D = ()


def _skipped(name: str, path: str, modules_to_not_convert: list[str]) -> bool:
    """The reference's test (quantizer.py:31-36): by the module's own name, by its full path, or by a
    listed prefix of the path."""
    if name in modules_to_not_convert:
        return True
    return any((key + "." in path) or (key == path) for key in modules_to_not_convert)


def _replace(model: nn.Module, modules_to_not_convert: list[str], path: list[str], config: Any) -> bool:
    replaced = False
    for name, module in model.named_children():
        path.append(name)
        is_linear = isinstance(module, nn.Linear) or (Conv1D != () and isinstance(module, Conv1D))
        if isinstance(module, MoeFusedLinear) and not isinstance(module, MoeFusedLinear4bit):
            if not _skipped(name, ".".join(path), modules_to_not_convert):
                new = MoeFusedLinear4bit(module.in_features, module.out_features, module.num_experts,
                                         compute_dtype=config.bnb_4bit_compute_dtype,
                                         compress_statistics=config.bnb_4bit_use_double_quant,
                                         quant_type=config.bnb_4bit_quant_type,
                                         quant_storage=config.bnb_4bit_quant_storage, device=module.weight.device)
                new.source_cls = type(module)
                new.requires_grad_(False)
                model._modules[name] = new
                replaced = True
        elif is_linear and Linear4bit is not None and not _skipped(name, ".".join(path), modules_to_not_convert):
            if isinstance(module, nn.Linear):
                in_features, out_features = module.in_features, module.out_features
            else:
                in_features, out_features = module.weight.shape
            extra = ({"quant_storage": config.bnb_4bit_quant_storage}
                     if "quant_storage" in signature(Linear4bit).parameters else {})
            new = Linear4bit(in_features, out_features, module.bias is not None, config.bnb_4bit_compute_dtype,
                             compress_statistics=config.bnb_4bit_use_double_quant,
                             quant_type=config.bnb_4bit_quant_type, **extra)
            new.source_cls = type(module)
            new.requires_grad_(False)
            model._modules[name] = new
            replaced = True
        if len(list(module.children())) > 0:
            replaced = _replace(module, modules_to_not_convert, path, config) or replaced
        path.pop()
    return replaced


def replace_with_bnb_moe_fused_linear(model: nn.Module, modules_to_not_convert: Optional[list[str]],
                                      quantization_config: Any) -> bool:
    """Swaps the modules in place (quantizer.py:93-106); returns whether anything was replaced."""
    skip = ["lm_head"] if modules_to_not_convert is None else list(modules_to_not_convert)
    replaced = _replace(model, skip, [], quantization_config)
    if not replaced:
        import warnings

        warnings.warn("4-bit loading was requested but the model holds no module to convert")
    return replaced


def _process_model_before_weight_loading(self, model, device_map: Union[str, dict[str, Any], None] = None,
                                         keep_in_fp32_modules: Optional[list[str]] = None, **kwargs) -> None:
    if keep_in_fp32_modules is None:
        keep_in_fp32_modules = getattr(model, "_keep_in_fp32_modules", None)
    self.modules_to_not_convert = self.get_modules_to_not_convert(
        model, self.quantization_config.llm_int8_skip_modules, keep_in_fp32_modules)
    # modules that a device map sends to the CPU or to disk stay unquantised (quantizer.py:119-122)
    if isinstance(device_map, dict) and len(device_map) > 1:
        self.modules_to_not_convert.extend(key for key, value in device_map.items() if value in ("disk", "cpu"))
    replace_with_bnb_moe_fused_linear(model, self.modules_to_not_convert, self.quantization_config)
    if getattr(model, "config", None) is not None:
        model.config.quantization_config = self.quantization_config


def _param_needs_quantization(self, model, param_name: str, **kwargs) -> bool:
    from transformers.quantizers.quantizers_utils import get_module_from_name

    module, name = get_module_from_name(model, param_name)
    if isinstance(module, MoeFusedLinear4bit):
        return name == "weight"
    return Linear4bit is not None and isinstance(module, Linear4bit) and name != "bias"


def patch_bnb_quantizer() -> None:
    """quantizer.py:132-133 of the reference."""
    from transformers.quantizers.quantizer_bnb_4bit import Bnb4BitHfQuantizer

    Bnb4BitHfQuantizer._process_model_before_weight_loading = _process_model_before_weight_loading
    if hasattr(Bnb4BitHfQuantizer, "param_needs_quantization"):
        Bnb4BitHfQuantizer.param_needs_quantization = _param_needs_quantization
