"""Tensor plumbing shared by the operator modules: device checks, raw pointers,
the current HIP stream.  PyTorch is used for memory and streams only."""
import torch

from . import _lib

FP8 = torch.float8_e4m3fn
DT_CODE = {torch.bfloat16: 0, torch.float32: 1}


def require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "mdy_triton_amd operators run on a ROCm GPU only (got a %s tensor); there is no CPU path" % t.device)
    return tensors[0].device


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
