"""ctypes binding of libmdyfp8.so (the C ABI declared in include/mdy_fp8.h).

The library is the only compute path of this package: if it is missing, or the
tensors are not on a ROCm device, the operators raise - there is no CPU or
PyTorch fallback.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmdyfp8.so")
ABI_VERSION = 15

_lock = threading.Lock()
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p
_int = ctypes.c_int

# name -> argtypes; every function returns int except the two noted below.
SIGNATURES = {
    "mdy_act_quant": [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_act_quant_typed": [_p, _int, _int, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_weight_quant": [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_weight_quant_typed": [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_quant_transpose": [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_quant_transpose_typed": [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_fp8_grouped_gemm_nt": [_p, _p, _i64, _i64, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_act_quant_transpose": [_p, _int, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_fp8_gemm_nt_rowscaled": [_p, _p, _i64, _i64, _p, _p, _i64, _i64, _p, _i64, _i64, _i64, _int, _int, _p],
    "mdy_swiglu": [_p, _p, _p, _p, _i64, _i64, _i64, _int, _i64, _i64, _i64, _i64, _int, _p],
    "mdy_swiglu_bwd": [_p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_weight_dequant": [_p, _p, _p, _i64, _i64, _int, _p],
    "mdy_weight_dequant_block": [_p, _p, _p, _i64, _i64, _int, _int, _p],
    "mdy_fp8_gemm_nt": [_p, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_fp8_gemm_nt_e5m2": [_p, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_fp8_gemm_nt_ws": [_p, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p, _i64, _p],
    "mdy_fp8_gemm_workspace_bytes": [_i64, _i64, _i64],
    "mdy_fp8_gemm_path": [_p, _p, _i64, _i64, _i64, _i64, _i64, _int],
    "mdy_fp8_gemm_nt_static_ws": [_p, _p, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_fp8_gemm_static_workspace_bytes": [],
    "mdy_fp8_gemm_static_workspace_init": [],
    "mdy_group_pad_rows": [_p, _p, _p, _i64, _i64, _i64, _int, _p],
    "mdy_add_grad": [_p, _p, _i64, _int, _int, _p],
    "mdy_add_bias": [_p, _p, _i64, _i64, _p],
    "mdy_add_bias_typed": [_p, _p, _int, _i64, _i64, _p],
    "mdy_cast_f32_to_e4m3": [_p, _p, _i64, _int, _p],
    "mdy_cast_f32_to_e5m2": [_p, _p, _i64, _p],
    "mdy_quotient_selfcheck": [_p, _int, _int, _int, _p],
    "mdy_fp8_abi_version": [],
    "mdy_fp8_last_error": [],
}


class MdyFp8Error(RuntimeError):
    pass


def load():
    """Load (once) and return the ctypes handle; raises if the library is absent."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise MdyFp8Error(
                "%s not found: build it with `python -m mdy_triton_amd.csrc.build` "
                "(needs hipcc; cross-compiles for gfx950 without a GPU)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = (ctypes.c_char_p if name == "mdy_fp8_last_error" else
                          ctypes.c_int64 if name in ("mdy_fp8_gemm_workspace_bytes", "mdy_fp8_gemm_static_workspace_bytes")
                          else ctypes.c_int)
        got = lib.mdy_fp8_abi_version()
        if got != ABI_VERSION:
            raise MdyFp8Error("libmdyfp8.so ABI version %d, expected %d: rebuild" % (got, ABI_VERSION))
        _lib = lib
    return _lib


def check(rc: int, what: str):
    """Turn a non-zero return code into an exception (negative: rejected argument)."""
    if rc == 0:
        return
    msg = load().mdy_fp8_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError("%s rejected its arguments (code %d): %s" % (what, rc, msg))
    raise MdyFp8Error("%s failed (hipError %d): %s" % (what, rc, msg))
