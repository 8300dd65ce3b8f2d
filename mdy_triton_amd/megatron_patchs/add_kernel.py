"""Element-wise helpers of the Megatron patch: add_bias and add_grad.

Drop-in for /root/reference/triton_kernels/megatron_patchs/add_kernel.py (add_bias :25-33, add_grad :55-62)."""
import torch

from .._torch_glue import DT_CODE, check, lib, on_device, ptr, require_gpu, stream_ptr
from ..fp8 import add_bias  # noqa: F401  (same operator as dpsk_fp8linear/fp8.py:297-305)


def add_grad(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """In place x += y, added in fp32 and stored in x's dtype (fp32 main_grad += bf16 weight gradient); returns x."""
    assert x.is_contiguous() and y.is_contiguous() and x.shape == y.shape
    if x.dtype not in DT_CODE or y.dtype not in DT_CODE:
        raise TypeError("add_grad expects bfloat16 / float32 tensors, got %s and %s" % (x.dtype, y.dtype))
    dev = require_gpu(x, y)
    with on_device(dev):
        check(lib().mdy_add_grad(ptr(x), ptr(y), x.numel(), DT_CODE[x.dtype], DT_CODE[y.dtype], stream_ptr(dev)), "add_grad")
    return x
