"""The C-ABI library loads without a GPU, exports every symbol include/moe_fused_linear.h
declares, and rejects bad arguments with its documented error codes before touching a device."""
import ctypes
import os
import re

from qwen3_moe_fused import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "moe_fused_linear.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mfl_[a-z0-9_]+)\s*\(", text)))


def _exported():
    """Dynamic symbols the shared object defines (nm -D), without the per-object identifiers that
    hipcc itself emits (__hip_cuid_*)."""
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], check=True, capture_output=True, text=True)
    names = [line.split()[-1] for line in out.stdout.splitlines() if line.strip()]
    return sorted(n for n in names if not n.startswith("__hip_"))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared()
    assert len(names) >= 17
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} is declared in the header but not exported"
    assert sorted(_lib.ABI_SYMBOLS) == names, "python binding table and header disagree"


def test_exported_symbols_are_exactly_the_declared_ones():
    """Nothing undeclared leaves the library: no tuning hook, no internal C++ symbol."""
    assert _exported() == _declared()


def test_version_and_strerror():
    lib = _lib.lib()
    assert lib.mfl_abi_version() == 1
    assert lib.mfl_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert lib.mfl_strerror(code) not in (b"ok", b"unknown error code")
    assert lib.mfl_strerror(-99) == b"unknown error code"


def test_argument_errors_without_device_work():
    lib = _lib.lib()
    BF16, I32 = _lib.BF16, _lib.I32
    buf = ctypes.create_string_buffer(256)
    p = ctypes.addressof(buf)
    p = (p + 63) // 64 * 64
    # NULL m_sizes
    assert lib.mfl_gemm_fwd(p, p, None, I32, p, 4, 8, 8, 2, BF16, BF16, 1.0, 0, None) == -1
    # bad shape
    assert lib.mfl_gemm_fwd(p, p, p, I32, p, 4, 0, 8, 2, BF16, BF16, 1.0, 0, None) == -2
    assert lib.mfl_gemm_dw(p, p, p, I32, p, -1, 8, 8, 2, BF16, BF16, 1.0, 0, None) == -2
    # bad dtypes
    assert lib.mfl_gemm_dx(p, p, p, I32, p, 4, 8, 8, 2, 7, BF16, 1.0, 0, None) == -3
    assert lib.mfl_gemm_fwd(p, p, p, 5, p, 4, 8, 8, 2, BF16, BF16, 1.0, 0, None) == -3
    # misaligned operand
    assert lib.mfl_gemm_fwd(p + 1, p, p, I32, p, 4, 8, 8, 2, BF16, BF16, 1.0, 0, None) == -4
    # NF4: blocksize not a power of two, odd K
    assert lib.mfl_gemm_fwd_nf4(p, p, p, p, 48, p, I32, p, 4, 8, 8, 2, BF16, BF16, None) == -2
    assert lib.mfl_gemm_fwd_nf4(p, p, p, p, 64, p, I32, p, 4, 8, 7, 2, BF16, BF16, None) == -2
    assert lib.mfl_nf4_dequant(p, p, p, 64, p, 63, BF16, None) == -2
    # routing: k > E; sort: missing counts
    assert lib.mfl_route_softmax_topk(p, _lib.F32, 4, 8, 9, 1, None, None, BF16, p, None) == -2
    assert lib.mfl_expert_sort(p, _lib.I64, 16, 4, None, None, None, None, 0, None) == -1
    assert lib.mfl_expert_sort(p, 9, 16, 4, p, None, None, None, 0, None) == -3
    # the entry point without a workspace: same argument checks, and its fixed maximum
    assert lib.mfl_expert_sort_static(p, _lib.I64, 16, 4, None, None, None, None) == -1
    assert lib.mfl_expert_sort_static(p, _lib.I64, -1, 4, p, None, None, None) == -2
    assert lib.mfl_silu_mul_fwd(None, p, p, 8, BF16, None) == -1
    assert lib.mfl_gather_rows(p, p, 0, None, p, 4, 8, BF16, None) == -2
    # empty problems are accepted and do nothing
    assert lib.mfl_gemm_fwd(None, None, p, I32, None, 0, 8, 8, 2, BF16, BF16, 1.0, 0, None) == 0
    assert lib.mfl_silu_mul_fwd(None, None, None, 0, BF16, None) == 0
    # per-wave and per-workgroup histograms: at least one count per expert, more rows never need less
    assert lib.mfl_expert_sort_workspace(32768, 128) >= 128 * 4
    assert lib.mfl_expert_sort_workspace(65536, 128) >= lib.mfl_expert_sort_workspace(32768, 128)
    assert lib.mfl_expert_sort_workspace(1 << 20, 128) >= lib.mfl_expert_sort_workspace(65536, 128)


def test_python_wrappers_assert_on_cpu_tensors():
    import pytest
    import torch

    from qwen3_moe_fused.grouped_gemm.forward import grouped_gemm_forward
    from qwen3_moe_fused.kernels.silu_mul import silu_mul_forward

    with pytest.raises(AssertionError):
        grouped_gemm_forward(torch.zeros(2, 8), torch.zeros(1, 8, 8), torch.tensor([2]))
    with pytest.raises(AssertionError):
        silu_mul_forward(torch.zeros(4), torch.zeros(4))


def test_naive_trio_runs_on_cpu():
    """The reference's naive functions are plain torch and define the semantics on any device
    (functional.py:7-61): checked here against the oracle on benchmark configuration 1 sizes."""
    import numpy as np
    import torch

    import oracle
    from qwen3_moe_fused.functional import (_moe_fused_linear_naive_bwd_input, _moe_fused_linear_naive_bwd_weight,
                                            _moe_fused_linear_naive_fwd)

    g = torch.Generator().manual_seed(0)
    x = torch.randn((64, 16), generator=g)
    w = torch.randn((4, 12, 16), generator=g) * 0.1
    dy = torch.randn((64, 12), generator=g)
    sel = torch.randint(0, 4, (64,), generator=g)
    np.testing.assert_allclose(_moe_fused_linear_naive_fwd(x, w, sel).numpy(),
                               oracle.linear_fwd(x.numpy(), w.numpy(), sel.numpy()), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(_moe_fused_linear_naive_bwd_input(dy, x, w, sel).numpy(),
                               oracle.linear_bwd_input(dy.numpy(), w.numpy(), sel.numpy()), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(_moe_fused_linear_naive_bwd_weight(dy, x, w, sel).numpy(),
                               oracle.linear_bwd_weight(dy.numpy(), x.numpy(), sel.numpy(), 4), rtol=1e-5, atol=1e-6)
