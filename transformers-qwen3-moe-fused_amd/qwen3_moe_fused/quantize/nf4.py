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


# The FP4 code book of bitsandbytes (sign, two exponent bits, one mantissa bit; values
# 0, 0.0625, 8, 12, 4, 6, 2, 3 and their negatives, divided by 12).
FP4_CODE = tuple(v / 12.0 for v in (0.0, 0.0625, 8.0, 12.0, 4.0, 6.0, 2.0, 3.0, -0.0, -0.0625, -8.0, -12.0, -4.0,
                                    -6.0, -2.0, -3.0))

QUANT_TYPES = ("nf4", "fp4")


def nf4_code(device) -> torch.Tensor:
    return torch.tensor(NF4_CODE, dtype=torch.float32, device=device)


def code_of(quant_type: str, device) -> torch.Tensor:
    """16-entry code book of a 4-bit type; the kernels take the table as an argument."""
    if quant_type == "nf4":
        return nf4_code(device)
    if quant_type == "fp4":
        return torch.tensor(FP4_CODE, dtype=torch.float32, device=device)
    raise NotImplementedError(f"4-bit quantisation type {quant_type!r}")


def dynamic_map_8bit() -> torch.Tensor:
    """The signed 8-bit "dynamic" code book that bitsandbytes uses for the second level of a
    double quantisation (its ``create_dynamic_map(signed=True, max_exponent_bits=7, total_bits=8)``):
    for each of seven decades 10^-6 .. 10^0, the midpoints of 2^i equal slices of [0.1, 1], both
    signs, plus 0 and 1.  The table is stored with every quantised tensor (``nested_quant_map``),
    so a reader never has to rebuild it."""
    data = []
    for i in range(7):
        boundaries = torch.linspace(0.1, 1, 2 ** i + 1)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        scale = 10.0 ** (-6 + i)
        data += (scale * means).tolist()
        data += (-scale * means).tolist()
    data += [0.0, 1.0]
    assert len(data) == 256
    return torch.tensor(sorted(data), dtype=torch.float32)


@dataclass
class Nf4QuantState:
    """Field-compatible stand-in for bitsandbytes' ``QuantState`` (the 4-bit types: NF4 and FP4)."""

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

    # ---- serialisation: the entries bitsandbytes' QuantState.as_dict(packed=True) / from_dict use, which is
    # what the reference module writes into its state dict (quantize/layer.py:76-81) and what 4-bit
    # checkpoints on the hub hold: tensors under their own names, everything else as a JSON object
    # packed into a uint8 tensor named "quant_state.bitsandbytes__<quant_type>".
    def as_dict(self, packed: bool = False) -> dict:
        import json

        plain = {"quant_type": self.quant_type, "absmax": self.absmax, "blocksize": int(self.blocksize),
                 "quant_map": self.code, "dtype": str(self.dtype).replace("torch.", ""), "shape": tuple(self.shape)}
        if self.nested:
            off = self.offset
            plain.update({"nested_absmax": self.state2.absmax, "nested_blocksize": int(self.state2.blocksize),
                          "nested_quant_map": self.state2.code.clone(),
                          "nested_dtype": str(getattr(self.state2, "dtype", torch.float32)).replace("torch.", ""),
                          "nested_offset": float(off.item()) if torch.is_tensor(off) else float(off)})
        if not packed:
            return plain
        out = {k: v for k, v in plain.items() if torch.is_tensor(v)}
        rest = {k: (list(v) if isinstance(v, tuple) else v) for k, v in plain.items() if not torch.is_tensor(v)}
        blob = torch.tensor(list(json.dumps(rest).encode("utf-8")), dtype=torch.uint8)
        out["quant_state.bitsandbytes__" + self.quant_type] = blob
        return out

    @classmethod
    def from_dict(cls, qs_dict: dict, device) -> "Nf4QuantState":
        import json

        d = dict(qs_dict)
        packed_keys = [k for k, v in d.items() if "quant_state" in k and torch.is_tensor(v)]
        if not packed_keys and "quant_type" not in d:
            raise ValueError("quant state entries hold neither a packed quant_state nor a quant_type")
        if len(packed_keys) > 1 or (packed_keys and not any(t in packed_keys[0] for t in QUANT_TYPES)):
            raise ValueError(f"there should be exactly one quant_state entry of a 4-bit type, found {packed_keys}")
        if packed_keys:
            blob = d.pop(packed_keys[0])
            d.update(json.loads(bytes(blob.detach().cpu().to(torch.uint8).tolist()).decode("utf-8")))
        d = {k.split(".")[-1]: v for k, v in d.items()}          # names may come with a parameter prefix
        offset = state2 = None
        if "nested_absmax" in d:
            offset = torch.tensor(float(d["nested_offset"]), dtype=torch.float32, device=device)
            state2 = BlockwiseState(absmax=d["nested_absmax"].to(device), code=d["nested_quant_map"].to(device),
                                    blocksize=int(d["nested_blocksize"]))
        return cls(absmax=d["absmax"].to(device), shape=tuple(int(v) for v in d["shape"]),
                   code=d["quant_map"].to(device=device, dtype=torch.float32), blocksize=int(d["blocksize"]),
                   quant_type=d["quant_type"], dtype=getattr(torch, d["dtype"]), offset=offset, state2=state2)

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
    dtype: torch.dtype = torch.float32


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


# rows per expert up to which the library's NF4 products run on the kernels that read tile-ordered scales (the plain
# forward product up to 128, the gated one up to 384: a copy brought along above that is not read)
_TILED_ROWS_PER_EXPERT = 384


def tiled_absmax(quant_state, absmax: torch.Tensor, rows: int):
    """The scales of an (E, N, K) NF4 matrix once more in the order in which the decode-sized kernels consume
    them (``mfl_nf4_tile_absmax``), built on the first decode-sized call and kept on the quant state; ``None``
    where it does not apply (a larger batch, a double-quantised state whose fp32 scales are rebuilt per call,
    a shape without such a copy).  Costs as many bytes again as ``absmax`` (3 % of the packed weights)."""
    cached = getattr(quant_state, "_mfl_absmax_tiled", None)
    if cached is not None and cached[0] is absmax and cached[1] == absmax._version:
        return cached[3] if rows <= cached[2] else None  # the path of every call but the first
    if getattr(quant_state, "nested", False) or len(quant_state.shape) != 3:
        return None
    experts, n, k = (int(v) for v in quant_state.shape)
    max_rows = _TILED_ROWS_PER_EXPERT * experts
    if rows > max_rows:
        return None
    blocksize = int(quant_state.blocksize)
    count = int(_lib.lib().mfl_nf4_tiled_absmax_floats(blocksize, n, k, experts))
    out = None
    if count > 0:
        out = torch.empty(count, device=absmax.device, dtype=torch.float32)
        rc = _lib.lib().mfl_nf4_tile_absmax(_lib.ptr(absmax), blocksize, n, k, experts, _lib.ptr(out), _lib.stream())
        _lib.check(rc, "mfl_nf4_tile_absmax")
    try:
        quant_state._mfl_absmax_tiled = (absmax, absmax._version, max_rows, out)
    except AttributeError:  # a state type with fixed attributes: rebuilt per call
        pass
    return out


def _quantize_absmax(absmax: torch.Tensor, blocksize2: int = 256):
    """Second level of a double quantisation, as bitsandbytes does it: subtract the mean, then blockwise
    8-bit quantisation against the dynamic code book (nearest entry of x / max|block|).  Load-time work on
    a tensor of E*N*K / blocksize floats: plain torch ops on the device."""
    offset = absmax.mean()
    centred = absmax - offset
    n = centred.numel()
    pad = (-n) % blocksize2
    blocks = torch.nn.functional.pad(centred, (0, pad)).view(-1, blocksize2)
    absmax2 = blocks.abs().amax(dim=1)
    scaled = blocks / absmax2.clamp_min(torch.finfo(torch.float32).tiny).unsqueeze(1)
    code = dynamic_map_8bit().to(absmax.device)
    mid = (code[:-1] + code[1:]) / 2
    q = torch.bucketize(scaled, mid).to(torch.uint8).view(-1)[:n]
    return q, BlockwiseState(absmax=absmax2, code=code, blocksize=blocksize2), offset


def quantize_nf4(w: torch.Tensor, blocksize: int = 64, quant_type: str = "nf4",
                 compress_statistics: bool = False) -> Tuple[torch.Tensor, Nf4QuantState]:
    """Blockwise 4-bit quantisation on the GPU: returns (packed uint8 (numel/2, 1), state).
    Element 2i goes to the high nibble of byte i, 2i+1 to the low nibble.  With
    ``compress_statistics`` the fp32 absmax is itself quantised to 8 bits (nested state)."""
    assert w.is_cuda and w.is_contiguous()
    n = w.numel()
    assert n % blocksize == 0 and blocksize % 2 == 0
    code = code_of(quant_type, w.device)
    packed = torch.empty((n // 2, 1), device=w.device, dtype=torch.uint8)
    absmax = torch.empty(n // blocksize, device=w.device, dtype=torch.float32)
    rc = _lib.lib().mfl_nf4_quant(_lib.ptr(w), _lib.dtype_code(w.dtype), n, blocksize, _lib.ptr(code), _lib.ptr(packed),
                                  _lib.ptr(absmax), _lib.stream())
    _lib.check(rc, "mfl_nf4_quant")
    state = Nf4QuantState(absmax=absmax, shape=tuple(w.shape), code=code, blocksize=blocksize, quant_type=quant_type,
                          dtype=w.dtype)
    if compress_statistics:
        state.absmax, state.state2, state.offset = _quantize_absmax(absmax)
    return packed, state


def dequantize_nf4(packed: torch.Tensor, quant_state, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``code[nibble] * absmax[block]`` in fp32, rounded once to ``dtype`` (default: the state's)."""
    assert quant_state.quant_type in QUANT_TYPES
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
