"""Tensor plumbing shared by the operator modules: device checks, raw pointers,
the current HIP stream.  PyTorch is used for memory and streams only."""
import warnings

import torch

from . import _lib

FP8 = torch.float8_e4m3fn
DT_CODE = {torch.bfloat16: 0, torch.float32: 1}
XT_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}      # input types of the activation quantizer


def require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "mdy_triton_amd operators run on a ROCm GPU only (got a %s tensor); there is no CPU path" % t.device)
    return tensors[0].device


def xt_code(x, who):
    try:
        return XT_CODE[x.dtype]
    except KeyError:
        raise TypeError("%s expects a bfloat16, float16 or float32 tensor, got %s" % (who, x.dtype)) from None


def ptr(t):
    return 0 if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """hipStream_t of torch's current stream on `device` (the raw getter skips building a Stream object:
    ~1.5 us per call, which shows in the decode shapes)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    __slots__ = ()

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context that makes `device` current for the launch (kernels go to the current
    device); free when it already is."""
    if torch.cuda.current_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


def out_code(dtype):
    try:
        return DT_CODE[dtype]
    except KeyError:
        raise TypeError("output dtype must be torch.bfloat16 or torch.float32, got %s" % dtype) from None


lib = _lib.load
check = _lib.check


_WS_BYTES = {}


def gemm_workspace(device, M, N, K):
    """Scratch tensor for mdy_fp8_gemm_nt_ws, or None when the shape is never split along K.  It comes
    from torch's caching allocator on the current stream, so it may be dropped as soon as the launch
    has been enqueued: the allocator hands the memory out again in stream order only."""
    key = (M, N, K)
    nbytes = _WS_BYTES.get(key)
    if nbytes is None:                      # one library call per shape, not per GEMM
        if len(_WS_BYTES) > 4096:
            _WS_BYTES.clear()
        nbytes = _WS_BYTES[key] = _lib.load().mdy_fp8_gemm_workspace_bytes(M, N, K)
    if nbytes <= 0:
        return None
    return torch.empty(nbytes, device=device, dtype=torch.uint8)


_SLOW_WARNED = set()


def warn_if_scalar_gemm(a, b, as_rs, as_cs, M, N, K, who):
    """One warning per shape when a LARGE aligned-K GEMM would run on the scalar kernel (one thread per output
    element, ~100x slower than the MFMA kernels).  That kernel is the intended path for K % 128 != 0; a shape
    with K % 128 == 0 reaches it only when K > 65536, when the activation scales span 2^31 bytes or more, or
    when an operand is not 16-byte aligned - none of which should pass silently.  The test that decides is the
    library's own (mdy_fp8_gemm_path); the cheap checks in front of it keep the common case free."""
    if M <= 64 or K % 128 != 0:
        return
    extent = ((M - 1) * as_rs + (K // 128 - 1) * as_cs + 1) * 4
    if K <= 65536 and 0 <= extent < (1 << 31) and as_rs >= 0 and as_cs >= 0 and not ((a.data_ptr() | b.data_ptr()) & 15):
        return
    key = (M, N, K, as_rs, as_cs)
    if key in _SLOW_WARNED:
        return
    if _lib.load().mdy_fp8_gemm_path(a.data_ptr(), b.data_ptr(), as_rs, as_cs, M, N, K, 1) == 0:
        _SLOW_WARNED.add(key)
        warnings.warn("%s: M=%d N=%d K=%d runs on the scalar fallback kernel (K > 65536, activation scales spanning "
                      ">= 2^31 bytes, or an operand that is not 16-byte aligned); expect ~100x the time of the MFMA "
                      "path - split K or the rows into several calls" % (who, M, N, K), RuntimeWarning, stacklevel=3)
