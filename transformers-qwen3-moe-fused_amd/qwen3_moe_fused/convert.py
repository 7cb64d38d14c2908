"""Checkpoint converters between the per-expert layout of Hugging Face Qwen3-MoE
(``...mlp.experts.<e>.<proj>.weight``, one (out, in) matrix per expert) and the fused layout of
this package (``...mlp.<proj>.weight``, one (E, out, in) tensor), for model weights and for LoRA
adapters (reference: qwen3_moe_fused/convert.py:18-211; same function names and directory
conventions).  Pure key renaming plus ``torch.stack`` / slicing on the CPU; nothing here touches
the GPU.

The optimizer-state converter of the reference (convert.py:214-312) re-quantises 8-bit optimizer
states with bitsandbytes and is not provided.
"""
from __future__ import annotations

import json
import os
import re
import shutil
from typing import Dict, Iterable, List, Optional, Union

import torch

TStateDict = Dict[str, torch.Tensor]

EXPERT_PROJECTIONS = ("gate_proj", "up_proj", "down_proj")
EXPERT_LORA_PARAMS = tuple(f"{proj}.lora_{ab}" for proj in EXPERT_PROJECTIONS for ab in "AB")

# wrappers (PEFT, task heads) put these in front of "layers.<i>...."
_KEY_PREFIXES = ("", "model.", "model.model.", "base_model.", "base_model.model.", "base_model.model.model.")


def load_sharded_state_dict(save_directory: Union[str, os.PathLike]) -> TStateDict:
    """All tensors of a safetensors checkpoint directory, sharded (index file present) or not."""
    import safetensors.torch

    index_path = os.path.join(save_directory, "model.safetensors.index.json")
    if not os.path.exists(index_path):
        return safetensors.torch.load_file(os.path.join(save_directory, "model.safetensors"))
    with open(index_path, "r", encoding="utf-8") as f:
        shard_names = sorted(set(json.load(f)["weight_map"].values()))
    state_dict: TStateDict = {}
    for name in shard_names:
        state_dict.update(safetensors.torch.load_file(os.path.join(save_directory, name)))
    return state_dict


def find_key_prefix(state_dict: TStateDict, *, is_fused: bool) -> str:
    """What precedes ``layers.0.mlp...`` in this state dict (model or LoRA adapter keys)."""
    stem = "layers.0.mlp.down_proj" if is_fused else "layers.0.mlp.experts.0.down_proj"
    for prefix in _KEY_PREFIXES:
        if prefix + stem + ".weight" in state_dict or prefix + stem + ".lora_A.weight" in state_dict:
            return prefix
    raise RuntimeError("Key prefix not found.")


def _fused_key(prefix: str, layer: int, param: str) -> str:
    return f"{prefix}layers.{layer}.mlp.{param}.weight"


def _expert_key(prefix: str, layer: int, expert: int, param: str) -> str:
    return f"{prefix}layers.{layer}.mlp.experts.{expert}.{param}.weight"


def convert_state_dict_to_fused_(state_dict: TStateDict, *, param_names: Iterable[str], num_hidden_layers: int,
                                 num_experts: int) -> None:
    """In place: the ``num_experts`` per-expert tensors of every (layer, param) become one stacked
    tensor with the expert index in front."""
    prefix = find_key_prefix(state_dict, is_fused=False)
    for layer in range(num_hidden_layers):
        for param in param_names:
            per_expert = [state_dict.pop(_expert_key(prefix, layer, e, param)) for e in range(num_experts)]
            state_dict[_fused_key(prefix, layer, param)] = torch.stack(per_expert)


def convert_state_dict_to_unfused_(state_dict: TStateDict, *, param_names: Iterable[str], num_hidden_layers: int,
                                   num_experts: int) -> None:
    """In place: inverse of ``convert_state_dict_to_fused_``.  Every slice is cloned: safetensors
    refuses to save tensors that share storage."""
    prefix = find_key_prefix(state_dict, is_fused=True)
    for layer in range(num_hidden_layers):
        for param in param_names:
            fused = state_dict.pop(_fused_key(prefix, layer, param))
            assert fused.shape[0] == num_experts, (fused.shape, num_experts)
            for e in range(num_experts):
                state_dict[_expert_key(prefix, layer, e, param)] = fused[e].clone()


# ---------------------------------------------------------------------------- whole models

def _rewrite_model_config(in_dir, out_dir, old: str, new: str) -> dict:
    """Copies config.json with the architecture name switched; returns the config as a dict."""
    with open(os.path.join(in_dir, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    archs: List[str] = list(config.get("architectures") or [])
    if archs:
        archs[0] = archs[0].replace(old, new)
        config["architectures"] = archs
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config, f, indent=2)
    for extra in ("generation_config.json",):
        if os.path.exists(os.path.join(in_dir, extra)):
            shutil.copyfile(os.path.join(in_dir, extra), os.path.join(out_dir, extra))
    return config


def _save_model_state(state_dict: TStateDict, out_dir, max_shard_size: Optional[Union[int, str]]) -> None:
    from huggingface_hub.serialization import save_torch_state_dict

    kwargs = {} if max_shard_size is None else {"max_shard_size": max_shard_size}
    save_torch_state_dict(state_dict, out_dir, **kwargs)


def _convert_model(in_dir, out_dir, to_fused: bool, max_shard_size) -> None:
    old, new = ("Qwen3Moe", "Qwen3MoeFused") if to_fused else ("Qwen3MoeFused", "Qwen3Moe")
    config = _rewrite_model_config(in_dir, out_dir, old, new)
    state_dict = load_sharded_state_dict(in_dir)
    convert = convert_state_dict_to_fused_ if to_fused else convert_state_dict_to_unfused_
    convert(state_dict, param_names=EXPERT_PROJECTIONS, num_hidden_layers=int(config["num_hidden_layers"]),
            num_experts=int(config["num_experts"]))
    _save_model_state(state_dict, out_dir, max_shard_size)


def convert_model_to_fused(in_dir, out_dir, *, max_shard_size: Optional[Union[int, str]] = None) -> None:
    """Hugging Face Qwen3-MoE checkpoint directory -> fused-expert checkpoint directory."""
    _convert_model(in_dir, out_dir, True, max_shard_size)


def convert_model_to_unfused(in_dir, out_dir, *, max_shard_size: Optional[Union[int, str]] = None) -> None:
    _convert_model(in_dir, out_dir, False, max_shard_size)


# ---------------------------------------------------------------------------- LoRA adapters

def _count_matches(state_dict: TStateDict, pattern: str) -> int:
    rx = re.compile(pattern)
    return sum(1 for key in state_dict if rx.fullmatch(key))


def _convert_lora(in_dir, out_dir, to_fused: bool) -> None:
    import safetensors.torch

    state_dict = safetensors.torch.load_file(os.path.join(in_dir, "adapter_model.safetensors"))
    prefix = re.escape(find_key_prefix(state_dict, is_fused=not to_fused))
    if to_fused:
        layers = _count_matches(state_dict, prefix + r"layers\.\d+\.mlp\.experts\.0\.down_proj\.lora_A\.weight")
        experts = _count_matches(state_dict, prefix + r"layers\.0\.mlp\.experts\.\d+\.down_proj\.lora_A\.weight")
        convert = convert_state_dict_to_fused_
    else:
        layers = _count_matches(state_dict, prefix + r"layers\.\d+\.mlp\.down_proj\.lora_A\.weight")
        experts = state_dict[find_key_prefix(state_dict, is_fused=True) + "layers.0.mlp.down_proj.lora_A.weight"].shape[0]
        convert = convert_state_dict_to_unfused_
    convert(state_dict, param_names=EXPERT_LORA_PARAMS, num_hidden_layers=layers, num_experts=experts)
    os.makedirs(out_dir, exist_ok=True)
    # the adapter's own configuration (rank, alpha, target modules) is the same in both layouts
    for name in ("adapter_config.json", "README.md"):
        if os.path.exists(os.path.join(in_dir, name)):
            shutil.copyfile(os.path.join(in_dir, name), os.path.join(out_dir, name))
    safetensors.torch.save_file(state_dict, os.path.join(out_dir, "adapter_model.safetensors"))


def convert_lora_to_fused(in_dir, out_dir, *, max_shard_size: Optional[Union[int, str]] = None) -> None:
    """PEFT adapter directory trained on the per-expert model -> adapter for the fused model
    (``lora_A`` (E, r, in), ``lora_B`` (E, out, r) per projection).  ``max_shard_size`` is accepted
    for signature parity and unused: an adapter is one file."""
    _convert_lora(in_dir, out_dir, True)


def convert_lora_to_unfused(in_dir, out_dir, *, max_shard_size: Optional[Union[int, str]] = None) -> None:
    _convert_lora(in_dir, out_dir, False)
