"""What of the 4-bit path runs without a GPU: the quant-state entries of the state dict (the packed
format of bitsandbytes' QuantState, which the reference module writes, quantize/layer.py:76-81),
reloading them, and the transformers quantizer hook (quantize/quantizer.py:21-133) on a tiny fused
model.  bitsandbytes is not importable in this environment and holds no fixture in the reference:
the key names and the JSON object are checked against hand-written entries; bit parity with its
quantiser stays unpinned."""
import json
from types import SimpleNamespace

import pytest
import torch

from qwen3_moe_fused.modular_qwen3_moe_fused import MoeFusedLinear
from qwen3_moe_fused.quantize.layer import MoeFusedLinear4bit
from qwen3_moe_fused.quantize.nf4 import FP4_CODE, NF4_CODE, BlockwiseState, Nf4QuantState, dynamic_map_8bit

E, N, K, BS = 2, 8, 16, 64


def _hand_written_entries(nested: bool):
    """State-dict entries of a (2, 8, 16) NF4 weight as a 4-bit checkpoint holds them."""
    n = E * N * K
    g = torch.Generator().manual_seed(0)
    meta = {"quant_type": "nf4", "blocksize": BS, "dtype": "bfloat16", "shape": [E, N, K]}
    entries = {"weight": torch.randint(0, 256, (n // 2, 1), generator=g, dtype=torch.uint8),
               "weight.quant_map": torch.tensor(NF4_CODE)}
    if nested:
        entries["weight.absmax"] = torch.randint(0, 256, (n // BS,), generator=g, dtype=torch.uint8)
        entries["weight.nested_absmax"] = torch.rand((1,), generator=g)
        entries["weight.nested_quant_map"] = dynamic_map_8bit()
        meta.update({"nested_blocksize": 256, "nested_dtype": "float32", "nested_offset": 0.015625})
    else:
        entries["weight.absmax"] = torch.rand((n // BS,), generator=g)
    entries["weight.quant_state.bitsandbytes__nf4"] = torch.tensor(list(json.dumps(meta).encode()), dtype=torch.uint8)
    return entries


@pytest.mark.parametrize("nested", [False, True])
def test_state_dict_round_trip_in_the_packed_quant_state_format(nested):
    entries = _hand_written_entries(nested)
    layer = MoeFusedLinear4bit(K, N, E, quant_type="nf4", compress_statistics=nested)
    missing, unexpected = layer.load_state_dict(entries, strict=True)
    assert not missing and not unexpected
    qs = layer.weight.quant_state
    assert layer.weight.dtype == torch.uint8 and layer.weight.shape == (E * N * K // 2, 1)
    assert qs.quant_type == "nf4" and qs.blocksize == BS and tuple(qs.shape) == (E, N, K)
    assert qs.dtype == torch.bfloat16 and qs.nested == nested
    if nested:
        assert qs.absmax.dtype == torch.uint8 and isinstance(qs.state2, BlockwiseState)
        assert qs.state2.blocksize == 256 and float(qs.offset) == 0.015625
    # what the module saves is what it was given, key for key and bit for bit (the JSON object by content)
    saved = layer.state_dict()
    assert set(saved) == set(entries)
    for key, value in entries.items():
        if "quant_state" in key:
            assert json.loads(bytes(saved[key].tolist()).decode()) == json.loads(bytes(value.tolist()).decode())
        else:
            assert torch.equal(saved[key], value), key
    # a second module loads the saved dict
    other = MoeFusedLinear4bit(K, N, E)
    other.load_state_dict(saved)
    assert torch.equal(other.weight.data, layer.weight.data) and other.weight.quant_state.nested == nested


def test_state_dict_errors_and_plain_weights():
    layer = MoeFusedLinear4bit(K, N, E, quant_type="nf4", compress_statistics=False)
    # a floating-point weight is accepted (it is quantised when the module reaches the GPU)
    w = torch.randn(E, N, K)
    layer.load_state_dict({"weight": w})
    assert layer.weight.quant_state is None and torch.equal(layer.weight.data, w)
    # wrong shape in the quant state, missing weight
    bad = _hand_written_entries(False)
    meta = {"quant_type": "nf4", "blocksize": BS, "dtype": "bfloat16", "shape": [E, N, K * 2]}
    bad["weight.quant_state.bitsandbytes__nf4"] = torch.tensor(list(json.dumps(meta).encode()), dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="do not describe"):
        layer.load_state_dict(bad)
    with pytest.raises(RuntimeError, match="Missing key"):
        layer.load_state_dict({})


def test_constructor_defaults_and_code_books():
    layer = MoeFusedLinear4bit(K, N, E)                      # the reference's defaults (quantize/layer.py:26-38)
    assert layer.weight.quant_type == "fp4" and layer.weight.compress_statistics is True
    assert layer.compute_dtype is None and not layer.compute_type_is_set and not layer.weight.requires_grad
    with pytest.raises(NotImplementedError):
        MoeFusedLinear4bit(K, N, E, quant_type="int4")
    assert len(FP4_CODE) == 16 and max(FP4_CODE) == 1.0 and min(FP4_CODE) == -1.0 and FP4_CODE[1] == 0.0625 / 12
    dm = dynamic_map_8bit()
    assert dm.shape == (256,) and dm[-1] == 1.0 and (dm[1:] >= dm[:-1]).all() and (dm == 0).sum() == 1
    qs = Nf4QuantState(absmax=torch.ones(4), shape=(2, 8, 16), code=torch.tensor(NF4_CODE), blocksize=64)
    back = Nf4QuantState.from_dict(qs.as_dict(packed=True), device="cpu")
    assert back.shape == (2, 8, 16) and back.blocksize == 64 and torch.equal(back.code, qs.code)
    with pytest.raises(ValueError):
        Nf4QuantState.from_dict({"absmax": torch.ones(4)}, device="cpu")


def _tiny_model():
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate = torch.nn.Linear(16, 4, bias=False)
            self.gate_proj = MoeFusedLinear(16, 8, 4)
            self.up_proj = MoeFusedLinear(16, 8, 4)
            self.down_proj = MoeFusedLinear(8, 16, 4)

    class Model(torch.nn.Module):
        _keep_in_fp32_modules = None

        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Block(), Block()])
            self.lm_head = torch.nn.Linear(16, 32, bias=False)
            self.config = SimpleNamespace()

    return Model()


def test_quantizer_hook_swaps_fused_modules_and_respects_the_skip_list():
    transformers = pytest.importorskip("transformers")
    from transformers import BitsAndBytesConfig
    from transformers.quantizers.quantizer_bnb_4bit import Bnb4BitHfQuantizer

    from qwen3_moe_fused.quantize.quantizer import patch_bnb_quantizer

    original = Bnb4BitHfQuantizer._process_model_before_weight_loading
    try:
        patch_bnb_quantizer()
        cfg = BitsAndBytesConfig(load_in_4bit=True, bnb_4bit_quant_type="nf4", bnb_4bit_use_double_quant=True,
                                 bnb_4bit_compute_dtype=torch.bfloat16,
                                 llm_int8_skip_modules=["lm_head", "layers.1.down_proj"])
        quantizer = Bnb4BitHfQuantizer(cfg)
        model = _tiny_model()
        quantizer._process_model_before_weight_loading(model, device_map=None)
        for i, block in enumerate(model.layers):
            for name in ("gate_proj", "up_proj", "down_proj"):
                mod = getattr(block, name)
                if i == 1 and name == "down_proj":
                    assert type(mod) is MoeFusedLinear, "listed in llm_int8_skip_modules"
                else:
                    assert type(mod) is MoeFusedLinear4bit and mod.source_cls is MoeFusedLinear
                    assert (mod.in_features, mod.out_features, mod.num_experts) == ((16, 8, 4) if name != "down_proj"
                                                                                     else (8, 16, 4))
                    assert mod.compute_dtype == torch.bfloat16 and mod.weight.quant_type == "nf4"
                    assert mod.weight.compress_statistics is True and not mod.weight.requires_grad
                    assert quantizer.param_needs_quantization(model, f"layers.{i}.{name}.weight")
            assert type(block.gate) is torch.nn.Linear          # no bitsandbytes here: plain linears stay
        assert type(model.lm_head) is torch.nn.Linear
        assert model.config.quantization_config is cfg
        assert "layers.1.down_proj" in quantizer.modules_to_not_convert
    finally:
        Bnb4BitHfQuantizer._process_model_before_weight_loading = original


def test_quantizer_operations_build_the_librarys_own_parameters():
    """The installed transformers release routes checkpoint tensors through the quantizer's conversion
    operations, not through ``_load_from_state_dict``: after ``patch_bnb_quantizer`` those operations turn a
    fused module's tensors into ``Nf4Params`` (a float tensor: still to be quantised on the CPU; a packed one
    with its bitsandbytes-named entries: with its quant state) and never touch bitsandbytes for them."""
    pytest.importorskip("transformers")
    from transformers import BitsAndBytesConfig
    from transformers.quantizers.quantizer_bnb_4bit import Bnb4BitHfQuantizer

    from qwen3_moe_fused.quantize.layer import Nf4Params
    from qwen3_moe_fused.quantize.nf4 import Nf4QuantState, code_of
    from qwen3_moe_fused.quantize.quantizer import patch_bnb_quantizer

    if not hasattr(Bnb4BitHfQuantizer, "get_quantize_ops"):
        pytest.skip("this transformers release loads through _load_from_state_dict")
    saved = {n: getattr(Bnb4BitHfQuantizer, n) for n in ("_process_model_before_weight_loading", "param_needs_quantization",
                                                         "get_quantize_ops", "get_weight_conversions")}
    try:
        patch_bnb_quantizer()
        cfg = BitsAndBytesConfig(load_in_4bit=True, bnb_4bit_quant_type="nf4", bnb_4bit_use_double_quant=False,
                                 bnb_4bit_compute_dtype=torch.bfloat16, llm_int8_skip_modules=["lm_head"])
        quantizer = Bnb4BitHfQuantizer(cfg)
        model = _tiny_model()
        quantizer._process_model_before_weight_loading(model, device_map=None)
        name = "layers.0.gate_proj.weight"
        module = model.layers[0].gate_proj

        # a floating-point checkpoint: one tensor per parameter through the quantize operation
        w = torch.randn(4, 8, 16)
        out = quantizer.get_quantize_ops().convert({name: [w]}, full_layer_name=name, model=model)
        assert set(out) == {name} and isinstance(out[name], Nf4Params)
        assert out[name].quant_state is None and torch.equal(out[name].data, w)       # quantised on reaching the GPU
        assert out[name].quant_type == "nf4" and out[name].module is module

        # a pre-quantised checkpoint: packed bytes and bitsandbytes' entries through the deserialise operation
        quantizer.pre_quantized = True
        converters = quantizer.get_weight_conversions()
        assert len(converters) == 1
        op = converters[0].operations[0]
        state = Nf4QuantState(absmax=torch.rand(4 * 8 * 16 // 64) + 0.5, shape=(4, 8, 16), code=code_of("nf4", "cpu"),
                              blocksize=64, quant_type="nf4", dtype=torch.bfloat16)
        packed = torch.randint(0, 256, (4 * 8 * 16 // 2, 1), dtype=torch.uint8)
        entries = {"weight." + k: [v] for k, v in state.as_dict(packed=True).items()}
        entries["weight"] = [packed]
        got = op.convert(entries, model=model, full_layer_name=name)
        assert set(got) == {"weight"} and isinstance(got["weight"], Nf4Params)
        qs = got["weight"].quant_state
        assert qs is not None and tuple(qs.shape) == (4, 8, 16) and qs.blocksize == 64 and qs.quant_type == "nf4"
        assert torch.equal(qs.absmax, state.absmax) and torch.equal(got["weight"].data, packed)
        assert module.quant_state is qs
    finally:
        for n, f in saved.items():
            setattr(Bnb4BitHfQuantizer, n, f)
        if hasattr(Bnb4BitHfQuantizer, "_mfl_stock_ops"):
            del Bnb4BitHfQuantizer._mfl_stock_ops
