"""ctypes binding of ``libmoe_fused_linear.so`` (the gfx950 HIP library).

PyTorch supplies device memory and the current HIP stream; every computation on the
hot path happens in the library.  There is no fallback: if the shared object is absent
the first call raises, it never silently computes on another path.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoe_fused_linear.so")
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "csrc"))

BF16, F32, F16 = 0, 1, 2
I32, I64 = 0, 1

_DTYPES = {torch.bfloat16: BF16, torch.float32: F32, torch.float16: F16}
_ITYPES = {torch.int32: I32, torch.int64: I64}

_vp, _i, _i64, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/moe_fused_linear.h
_SIGNATURES = {
    "mfl_abi_version": (_i, []),
    "mfl_strerror": (ctypes.c_char_p, [_i]),
    "mfl_gemm_fwd": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "mfl_gemm_dx": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "mfl_gemm_dw": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "mfl_gemm_dw_split_workspace": (_sz, [_i64, _i, _i, _i]),
    "mfl_gemm_dw_split": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _f, _vp, _sz, _vp]),
    "mfl_gemm_fwd_nf4": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_dx_nf4": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "mfl_gemm_dx_dual": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_dx_silu_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "mfl_gemm_fwd_lora": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_dx_lora": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_fwd_nf4_lora": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_dx_nf4_lora": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_fwd_gather": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "mfl_gemm_fwd_nf4_gather": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i,
                                     _vp]),
    "mfl_glu_fwd": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "mfl_glu_fwd_lora": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "mfl_glu_fwd_nf4": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _i64,
                             _i, _i, _i, _i, _vp]),
    "mfl_nf4_tiled_absmax_floats": (_i64, [_i, _i, _i, _i]),
    "mfl_nf4_tile_absmax": (_i, [_vp, _i, _i, _i, _i, _vp, _vp]),
    "mfl_gemm_fwd_nf4_tiled": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _i, _i, _i, _i,
                                    _i, _vp]),
    "mfl_glu_fwd_nf4_tiled": (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp,
                                   _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "mfl_nf4_dequant": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _i, _vp]),
    "mfl_dequant_blockwise_u8": (_i, [_vp, _vp, _vp, _i, _f, _vp, _i64, _vp]),
    "mfl_nf4_quant": (_i, [_vp, _i, _i64, _i, _vp, _vp, _vp, _vp]),
    "mfl_route_softmax_topk": (_i, [_vp, _i, _i64, _i, _i, _i, _vp, _vp, _i, _vp, _vp]),
    "mfl_route_softmax_topk_bwd": (_i, [_vp, _i, _i64, _i, _i, _i, _vp, _vp, _vp, _i, _vp, _vp]),
    "mfl_route_sort_small": (_i, [_vp, _i, _i64, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "mfl_route_sort_workspace": (_sz, [_i64, _i, _i]),
    "mfl_route_sort": (_i, [_vp, _i, _i64, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "mfl_expert_sort_workspace": (_sz, [_i64, _i]),
    "mfl_expert_sort": (_i, [_vp, _i, _i64, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "mfl_expert_sort_static": (_i, [_vp, _i, _i64, _i, _vp, _vp, _vp, _vp]),
    "mfl_gather_rows": (_i, [_vp, _vp, _i, _vp, _vp, _i64, _i, _i, _vp]),
    "mfl_scatter_rows": (_i, [_vp, _vp, _i, _vp, _vp, _i64, _i, _i, _vp]),
    "mfl_combine_rows": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "mfl_rows_dot": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "mfl_silu_mul_fwd": (_i, [_vp, _vp, _vp, _i64, _i, _vp]),
    "mfl_silu_mul_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _vp]),
}

# the entry points declared in include/moe_fused_linear.h: the library exports these and nothing else
ABI_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


class MflError(RuntimeError):
    """A library entry point returned a non-zero status."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MflError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` (hipcc, gfx950). "
                "There is no fallback path."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.mfl_abi_version() != 1:
            raise MflError("libmoe_fused_linear.so has an unexpected ABI version")
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().mfl_strerror(rc).decode()
        raise MflError(f"{what} failed with status {rc}: {msg}")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported element type {dt}; expected bfloat16, float32 or float16") from None


def itype_code(dt: torch.dtype) -> int:
    try:
        return _ITYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported index type {dt}; expected int32 or int64") from None


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def as_index_tensor(m_sizes: torch.Tensor) -> torch.Tensor:
    """int32/int64 pass straight through; the narrower integer types the reference also
    accepts are widened on the device (no host sync)."""
    if m_sizes.dtype in _ITYPES:
        return m_sizes
    return m_sizes.to(torch.int32)
