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
