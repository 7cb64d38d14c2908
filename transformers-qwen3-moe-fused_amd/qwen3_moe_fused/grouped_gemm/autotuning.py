"""Tile selection of the grouped-GEMM kernels.

The reference searches 1000 Triton configurations per (N, K, E) at run time
(qwen3_moe_fused/grouped_gemm/autotuning.py:9-106).  The HIP kernels are compiled ahead of
time in a handful of CDNA4 tile shapes and the library picks among them from the problem shape,
so nothing is tuned at run time and the library has no tuning switch; this module keeps the helper
callers use.
"""
from __future__ import annotations

import torch


def get_num_sms() -> int:
    """Compute units of the current GPU (256 on MI355X)."""
    return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
