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


def _first(value):
    return value[0] if isinstance(value, (list, tuple)) else value


def _conversion_ops():
    """The two weight-loading operations of the installed transformers release (its loader hands every
    checkpoint tensor of a parameter that ``param_needs_quantization`` names to the quantizer's operation, and
    the entries of a pre-quantised parameter to its deserialising one), extended to the fused modules.  The
    stock operations build bitsandbytes' ``Params4bit``; for a ``MoeFusedLinear4bit`` these build the library's
    own ``Nf4Params`` instead and leave every other module to the stock operation."""
    from transformers.core_model_loading import ConversionOps
    from transformers.quantizers.quantizers_utils import get_module_from_name

    from .layer import Nf4Params
    from .nf4 import Nf4QuantState

    class FusedQuantize(ConversionOps):
        """A floating-point (E, out, in) checkpoint tensor becomes an ``Nf4Params`` that is quantised on the
        device it was loaded to (on the CPU: when the module first reaches the GPU)."""

        def __init__(self, hf_quantizer, stock):
            self.hf_quantizer, self.stock = hf_quantizer, stock

        def convert(self, input_dict, full_layer_name=None, model=None, **kwargs):
            result, rest = {}, {}
            for param_name, value in input_dict.items():
                module, _ = get_module_from_name(model, param_name)
                if not isinstance(module, MoeFusedLinear4bit):
                    rest[param_name] = value
                    continue
                value = _first(value)
                old = module.weight
                new = Nf4Params(value.contiguous(), blocksize=old.blocksize, module=module, quant_type=old.quant_type,
                                compress_statistics=old.compress_statistics)
                if value.is_cuda:
                    new = new.to(value.device)
                module._is_hf_initialized = True
                result[param_name] = new
            if rest:
                result.update(self.stock.convert(rest, full_layer_name=full_layer_name, model=model, **kwargs))
            return result

    class FusedDeserialize(ConversionOps):
        """The packed weight of a pre-quantised checkpoint with its quant-state entries (bitsandbytes' names:
        ``absmax``, ``quant_map``, ``nested_absmax``, ``nested_quant_map``, ``quant_state.bitsandbytes__nf4``)."""

        def __init__(self, hf_quantizer, stock):
            self.hf_quantizer, self.stock = hf_quantizer, stock

        def convert(self, input_dict, model=None, full_layer_name=None, **kwargs):
            module, _ = get_module_from_name(model, full_layer_name)
            if not isinstance(module, MoeFusedLinear4bit):
                return self.stock.convert(input_dict, model=model, full_layer_name=full_layer_name, **kwargs)
            if len(input_dict) == 1:
                return input_dict
            entries = {key: _first(value) for key, value in input_dict.items()}
            packed = entries.pop("weight")
            state = Nf4QuantState.from_dict({k.split("weight.", 1)[-1]: v for k, v in entries.items()},
                                            device=packed.device)
            new = Nf4Params(packed.reshape(-1, 1).contiguous(), quant_state=state, blocksize=int(state.blocksize),
                            module=module, quant_type=state.quant_type, compress_statistics=state.nested)
            module.quant_state = state
            module._is_hf_initialized = True
            return {"weight": new}

    return FusedQuantize, FusedDeserialize


def patch_bnb_quantizer() -> None:
    """quantizer.py:132-133 of the reference, plus what the installed transformers release needs beyond the
    module swap: which parameters its loader sends through the quantizer, and the two operations that turn
    checkpoint tensors into parameters (releases without them load through ``_load_from_state_dict``)."""
    from transformers.quantizers.quantizer_bnb_4bit import Bnb4BitHfQuantizer

    Bnb4BitHfQuantizer._process_model_before_weight_loading = _process_model_before_weight_loading
    if hasattr(Bnb4BitHfQuantizer, "param_needs_quantization"):
        Bnb4BitHfQuantizer.param_needs_quantization = _param_needs_quantization
    if hasattr(Bnb4BitHfQuantizer, "get_quantize_ops") and not hasattr(Bnb4BitHfQuantizer, "_mfl_stock_ops"):
        FusedQuantize, FusedDeserialize = _conversion_ops()
        stock_quantize, stock_conversions = Bnb4BitHfQuantizer.get_quantize_ops, Bnb4BitHfQuantizer.get_weight_conversions
        Bnb4BitHfQuantizer._mfl_stock_ops = (stock_quantize, stock_conversions)

        def get_quantize_ops(self):
            return FusedQuantize(self, stock_quantize(self))

        def get_weight_conversions(self):
            converters = stock_conversions(self)
            for converter in converters:
                converter.operations = [FusedDeserialize(self, op) if type(op).__name__ == "Bnb4bitDeserialize" else op
                                        for op in converter.operations]
            return converters

        Bnb4BitHfQuantizer.get_quantize_ops = get_quantize_ops
        Bnb4BitHfQuantizer.get_weight_conversions = get_weight_conversions
