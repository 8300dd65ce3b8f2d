"""The C-ABI library loads, exports every symbol include/mdy_fp8.h declares, and
rejects bad arguments before touching a device (no compute calls here)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mdy_fp8.h")


@pytest.fixture(scope="module")
def lib():
    from mdy_triton_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from mdy_triton_amd.csrc.build import build
        build()
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mdy_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = declared_functions()
    assert "mdy_act_quant" in names and "mdy_fp8_gemm_nt" in names and len(names) >= 9
    for n in names:
        assert hasattr(lib, n), "missing export %s" % n
    from mdy_triton_amd._lib import SIGNATURES
    assert sorted(SIGNATURES) == names


def test_abi_version(lib):
    text = open(HEADER).read()
    v = int(re.search(r"#define MDY_FP8_ABI_VERSION (\d+)", text).group(1))
    assert lib.mdy_fp8_abi_version() == v


def test_argument_validation_without_device(lib):
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    # PK not a multiple of 128
    assert lib.mdy_act_quant(p, p, p, 4, 100, 100, 4, 100, 1, 1, 0, None) == -2
    assert b"128" in lib.mdy_fp8_last_error()
    # unknown dialect / dtype
    assert lib.mdy_act_quant(p, p, p, 4, 128, 128, 4, 128, 1, 1, 7, None) == -4
    assert lib.mdy_weight_dequant(p, p, p, 128, 128, 9, None) == -4
    # null pointers
    assert lib.mdy_act_quant(None, p, p, 4, 128, 128, 4, 128, 1, 1, 0, None) == -1
    assert lib.mdy_fp8_gemm_nt(p, p, 1, 1, p, None, p, None, 4, 4, 128, 0, None) == -1
    # misaligned output
    assert lib.mdy_act_quant(p, p + 4, p, 4, 128, 128, 4, 128, 1, 1, 0, None) == -3
    # y_t without s_t
    assert lib.mdy_weight_quant(p, p, p, p, None, 128, 128, 128, 1, 128, 128, 1, None) == -1
    # negative / inconsistent sizes
    assert lib.mdy_fp8_gemm_nt(p, p, 1, 1, p, p, p, None, -1, 4, 128, 0, None) == -2
    assert lib.mdy_act_quant(p, p, p, 8, 128, 128, 4, 128, 1, 1, 0, None) == -2
    # empty problems are no-ops that never reach a device
    assert lib.mdy_act_quant(None, None, None, 0, 0, 0, 0, 0, 1, 1, 0, None) == 0
    assert lib.mdy_fp8_gemm_nt(p, p, 1, 1, p, p, p, None, 0, 4, 128, 0, None) == 0
    assert lib.mdy_add_bias(p, p, 0, 16, None) == 0


def test_argument_validation_of_the_later_entry_points(lib):
    buf = ctypes.create_string_buffer(8192)
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    # GEMM with a workspace: negative size, misaligned buffer, empty problem, workspace query of a bad shape
    assert lib.mdy_fp8_gemm_nt_ws(p, p, 1, 1, p, p, p, None, 4, 4, 128, 0, p, -1, None) == -2
    assert lib.mdy_fp8_gemm_nt_ws(p, p, 1, 1, p, p, p, None, 4, 4, 128, 0, p + 4, 64, None) == -3
    assert lib.mdy_fp8_gemm_nt_ws(p, p, 1, 1, p, p, p, None, 0, 4, 128, 0, None, 0, None) == 0
    assert lib.mdy_fp8_gemm_nt_ws(p, p, 1, 1, p, p, p, None, 4, 4, 128, 5, None, 0, None) == -4
    assert lib.mdy_fp8_gemm_workspace_bytes(-1, 4, 128) == 0 and lib.mdy_fp8_gemm_workspace_bytes(4, 4, 0) == 0
    assert lib.mdy_fp8_gemm_workspace_bytes(128, 1536, 4096) >= 2 * 128 * 1536 * 4      # split along K
    assert lib.mdy_fp8_gemm_workspace_bytes(1, 7168, 2048) == 0                          # decode: never
    # grouped GEMM: no group table, a negative group, too many groups, nothing to do
    splits = (ctypes.c_int64 * 3)(4, -1, 4)
    assert lib.mdy_fp8_grouped_gemm_nt(p, p, 1, 1, p, p, p, None, None, 3, 4, 128, 0, None) == -1
    assert lib.mdy_fp8_grouped_gemm_nt(p, p, 1, 1, p, p, p, None, splits, 3, 4, 128, 0, None) == -2
    assert lib.mdy_fp8_grouped_gemm_nt(p, p, 1, 1, p, p, p, None, splits, (1 << 20) + 1, 4, 128, 0, None) == -2
    zero = (ctypes.c_int64 * 2)(0, 0)
    assert lib.mdy_fp8_grouped_gemm_nt(p, p, 1, 1, p, p, p, None, zero, 2, 4, 128, 0, None) == 0
    assert lib.mdy_fp8_grouped_gemm_nt(None, None, 1, 1, None, None, None, None, None, 0, 4, 128, 0, None) == 0
    # training quantizer: unknown transposed-scale mode, unpadded sizes, scale stride shorter than the rows
    assert lib.mdy_quant_transpose(p, p, p, p, p, 128, 128, 128, 1, 128, 128, 128, 7, None) == -4
    assert lib.mdy_quant_transpose(p, p, p, p, p, 100, 128, 128, 1, 100, 128, 128, 0, None) == -2
    assert lib.mdy_quant_transpose(p, p, p, p, p, 128, 128, 128, 1, 128, 128, 64, 0, None) == -2
    assert lib.mdy_quant_transpose(p, p, p, None, p, 128, 128, 128, 1, 128, 128, 128, 0, None) == -1
    # SwiGLU: nothing to write, quantized output without scales, row stride shorter than the row
    assert lib.mdy_swiglu(p, None, None, None, 4, 128, 256, 0, 4, 128, 1, 1, 0, None) == -1
    assert lib.mdy_swiglu(p, None, p, None, 4, 128, 256, 0, 4, 128, 1, 1, 0, None) == -1
    assert lib.mdy_swiglu(p, p, None, None, 4, 128, 200, 0, 0, 0, 1, 1, 0, None) == -2
    assert lib.mdy_swiglu(p, None, p, p, 4, 128, 256, 0, 4, 100, 1, 1, 0, None) == -2
    assert lib.mdy_swiglu(p, p, None, None, 0, 128, 256, 0, 0, 0, 1, 1, 0, None) == 0
    # diagnostics
    assert lib.mdy_quotient_selfcheck(None, 0, 16, 0, None) == -1
    assert lib.mdy_quotient_selfcheck(p, 16, 8, 0, None) == -2
    assert lib.mdy_cast_f32_to_e4m3(p, p, -1, 0, None) == -2 and lib.mdy_cast_f32_to_e4m3(None, None, 0, 0, None) == 0
    assert lib.mdy_fp8_last_error()            # the last message is kept


def test_python_wrappers_keep_reference_preconditions():
    import mdy_triton_amd as m
    x = torch.zeros(4, 130, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        m.act_quant(x)                      # last dim % 128 (offical_kernel.py:23)
    with pytest.raises(AssertionError):
        m.act_quant(torch.zeros(4, 256, dtype=torch.bfloat16)[:, ::2])  # contiguity (:22)
    with pytest.raises(AssertionError):
        m.weight_dequant(torch.zeros(2, 128, 128).to(torch.float8_e4m3fn), torch.zeros(1, 1))  # 2-D (:48)
    with pytest.raises(RuntimeError, match="no CPU path"):
        m.act_quant(torch.zeros(4, 128, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU path"):
        m.DeepLinear(256, 128, dtype=torch.bfloat16)(torch.zeros(4, 256, dtype=torch.bfloat16))


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "mdy_triton_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f


def test_gemm_path_query_needs_no_gpu(lib):
    """mdy_fp8_gemm_path only inspects sizes, strides and pointer alignment."""
    q = lib.mdy_fp8_gemm_path
    assert q(None, None, 56, 1, 4096, 18432, 7168, 1) == 3          # MFMA tiles
    assert q(None, None, 56, 1, 4096, 18432, 7168, 0) == 3
    assert q(None, None, 16, 1, 16, 7168, 2048, 1) == 1             # weight streaming
    assert q(None, None, 2, 1, 300, 200, 200, 1) == 0               # K % 128 != 0: scalar
    assert q(None, None, 1025, 1, 100, 256, 131200, 1) == 0         # K > 65536 and M > 64: scalar
    assert q(8, None, 56, 1, 4096, 1536, 7168, 1) == 0              # misaligned operand: scalar
    assert q(None, None, 32, 1, 128, 1536, 4096, 1) == 4            # split along K with a workspace ...
    assert q(None, None, 32, 1, 128, 1536, 4096, 0) == 3            # ... plain tiles without
    assert q(None, None, 56, 1, 0, 5, 128, 0) == -2
