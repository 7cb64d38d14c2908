"""Checkpoint converters (per-expert <-> fused layout), CPU only: key sets, shapes, exact round
trips through safetensors directories, for model weights and LoRA adapters."""
import json
import os

import pytest
import safetensors.torch
import torch

from qwen3_moe_fused import convert

L, E, H, I, R = 2, 3, 8, 4, 2


def _model_state(prefix="model."):
    g = torch.Generator().manual_seed(0)
    sd = {prefix + "embed_tokens.weight": torch.randn(10, H, generator=g)}
    for layer in range(L):
        sd[f"{prefix}layers.{layer}.mlp.gate.weight"] = torch.randn(E, H, generator=g)
        sd[f"{prefix}layers.{layer}.self_attn.q_proj.weight"] = torch.randn(H, H, generator=g)
        for e in range(E):
            for proj, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
                sd[f"{prefix}layers.{layer}.mlp.experts.{e}.{proj}.weight"] = torch.randn(shape, generator=g)
    return sd


def _lora_state(prefix="base_model.model.model."):
    g = torch.Generator().manual_seed(1)
    sd = {}
    for layer in range(L):
        sd[f"{prefix}layers.{layer}.self_attn.q_proj.lora_A.weight"] = torch.randn(R, H, generator=g)
        for e in range(E):
            for proj, (o, i) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
                sd[f"{prefix}layers.{layer}.mlp.experts.{e}.{proj}.lora_A.weight"] = torch.randn(R, i, generator=g)
                sd[f"{prefix}layers.{layer}.mlp.experts.{e}.{proj}.lora_B.weight"] = torch.randn(o, R, generator=g)
    return sd


@pytest.mark.parametrize("prefix", ["", "model.", "base_model.model.model."])
def test_state_dict_fuse_and_unfuse_round_trip(prefix):
    ref = _model_state(prefix)
    sd = dict(ref)
    assert convert.find_key_prefix(sd, is_fused=False) == prefix
    convert.convert_state_dict_to_fused_(sd, param_names=convert.EXPERT_PROJECTIONS, num_hidden_layers=L, num_experts=E)
    assert not any(".experts." in k for k in sd)
    assert convert.find_key_prefix(sd, is_fused=True) == prefix
    w = sd[f"{prefix}layers.1.mlp.down_proj.weight"]
    assert w.shape == (E, H, I)
    for e in range(E):  # expert e of the fused tensor is that expert's matrix
        assert torch.equal(w[e], ref[f"{prefix}layers.1.mlp.experts.{e}.down_proj.weight"])
    assert torch.equal(sd[prefix + "embed_tokens.weight"], ref[prefix + "embed_tokens.weight"])
    convert.convert_state_dict_to_unfused_(sd, param_names=convert.EXPERT_PROJECTIONS, num_hidden_layers=L,
                                           num_experts=E)
    assert sd.keys() == ref.keys() and all(torch.equal(sd[k], ref[k]) for k in ref)


def test_unknown_layout_is_reported():
    with pytest.raises(RuntimeError):
        convert.find_key_prefix({"foo.weight": torch.zeros(1)}, is_fused=True)


def test_model_directories_round_trip(tmp_path):
    src, fused, back = (str(tmp_path / n) for n in ("src", "fused", "back"))
    os.makedirs(src)
    ref = _model_state()
    safetensors.torch.save_file(ref, os.path.join(src, "model.safetensors"))
    with open(os.path.join(src, "config.json"), "w") as f:
        json.dump({"architectures": ["Qwen3MoeForCausalLM"], "num_hidden_layers": L, "num_experts": E,
                   "hidden_size": H, "moe_intermediate_size": I}, f)
    convert.convert_model_to_fused(src, fused, max_shard_size="1KB")     # forces several shards + an index
    assert os.path.exists(os.path.join(fused, "model.safetensors.index.json"))
    assert json.load(open(os.path.join(fused, "config.json")))["architectures"] == ["Qwen3MoeFusedForCausalLM"]
    sd = convert.load_sharded_state_dict(fused)
    assert sd["model.layers.0.mlp.gate_proj.weight"].shape == (E, I, H)
    assert len(sd) == len(ref) - L * 3 * (E - 1)
    convert.convert_model_to_unfused(fused, back)
    assert json.load(open(os.path.join(back, "config.json")))["architectures"] == ["Qwen3MoeForCausalLM"]
    sd2 = convert.load_sharded_state_dict(back)
    assert sd2.keys() == ref.keys() and all(torch.equal(sd2[k], ref[k]) for k in ref)


def test_lora_directories_round_trip(tmp_path):
    src, fused, back = (str(tmp_path / n) for n in ("src", "fused", "back"))
    os.makedirs(src)
    ref = _lora_state()
    safetensors.torch.save_file(ref, os.path.join(src, "adapter_model.safetensors"))
    with open(os.path.join(src, "adapter_config.json"), "w") as f:
        json.dump({"r": R, "lora_alpha": 4, "target_modules": ["gate_proj", "up_proj", "down_proj", "q_proj"]}, f)
    convert.convert_lora_to_fused(src, fused)
    sd = safetensors.torch.load_file(os.path.join(fused, "adapter_model.safetensors"))
    p = "base_model.model.model."
    assert sd[p + "layers.0.mlp.gate_proj.lora_A.weight"].shape == (E, R, H)     # lora.py:71-77 layout
    assert sd[p + "layers.0.mlp.down_proj.lora_B.weight"].shape == (E, H, R)
    assert torch.equal(sd[p + "layers.1.mlp.up_proj.lora_B.weight"][2], ref[p + "layers.1.mlp.experts.2.up_proj.lora_B.weight"])
    assert p + "layers.0.self_attn.q_proj.lora_A.weight" in sd
    assert json.load(open(os.path.join(fused, "adapter_config.json")))["r"] == R
    convert.convert_lora_to_unfused(fused, back)
    sd2 = safetensors.torch.load_file(os.path.join(back, "adapter_model.safetensors"))
    assert sd2.keys() == ref.keys() and all(torch.equal(sd2[k], ref[k]) for k in ref)
