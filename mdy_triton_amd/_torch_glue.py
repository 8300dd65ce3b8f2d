"""Tensor plumbing shared by the operator modules: device checks, raw pointers,
the current HIP stream.  PyTorch is used for memory and streams only."""
import contextlib

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


def stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


@contextlib.contextmanager
def on_device(device):
    """Make `device` current for the launch (kernels go to the current device)."""
    if torch.cuda.current_device() == device.index:
        yield
    else:
        with torch.cuda.device(device):
            yield


def out_code(dtype):
    try:
        return DT_CODE[dtype]
    except KeyError:
        raise TypeError("output dtype must be torch.bfloat16 or torch.float32, got %s" % dtype) from None


lib = _lib.load
check = _lib.check
