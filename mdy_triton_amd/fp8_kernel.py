"""SwiGLU and block quantizers of the FP8 MLP on MI355X.

Drop-in for the parts of /root/reference/triton_kernels/deepseekv3/fp8_kernel.py that sit
directly before the FP8 linear path: silu_fwd / silu_bwd / triton_silu (fp8_kernel.py:384-434),
weight_quant_block (:124-138), plus silu_act_quant, which fuses the `silu_fwd -> act_quant`
pair of the FP8 MLP (fp8_kernel.py:447-450, 500-515) into one pass over the up/gate tensor.
Only float8_e4m3fn is implemented (the reference defaults to e5m2 but its notebook passes
e4m3fn, deepseekv3/fp8-benchmark.ipynb line 78).
"""
from typing import Optional, Tuple

import torch

from ._torch_glue import FP8, check, lib, on_device, ptr, require_gpu, stream_ptr

_ORDERS = ("up-gate", "gate-up")


def _flatten_up_gate(x: torch.Tensor, order: str, who: str):
    assert order in _ORDERS, "please indicate the order of input, up-gate or gate-up"
    if x.dtype != torch.bfloat16:
        raise TypeError("%s expects a bfloat16 tensor, got %s" % (who, x.dtype))
    if x.size(-1) % 2 != 0:
        raise ValueError("%s: the last dimension holds up and gate and must be even" % who)
    x2 = x.reshape(-1, x.size(-1))
    if x2.numel() > 0 and x2.stride(1) != 1:
        x2 = x2.contiguous()
    return x2, x2.size(0), x2.size(1) // 2


def silu_fwd(x: torch.Tensor, order: str = "up-gate") -> torch.Tensor:
    """act = silu(gate) * up as bf16 [..., N] from x [..., 2N] (fp8_kernel.py:384-402)."""
    x2, M, N = _flatten_up_gate(x, order, "silu_fwd")
    dev = require_gpu(x)
    y = torch.empty(*x.shape[:-1], N, device=dev, dtype=x.dtype)
    if M * N == 0:
        return y
    with on_device(dev):
        check(lib().mdy_swiglu(ptr(x2), ptr(y), None, None, M, N, x2.stride(0) if M else 2 * N, int(order == "gate-up"),
                               0, 0, 0, 0, 0, stream_ptr(dev)), "silu_fwd")
    return y


def silu_bwd(dy: torch.Tensor, x: torch.Tensor, order: str = "up-gate") -> torch.Tensor:
    """Gradient of silu_fwd with respect to x (fp8_kernel.py:404-421); dx has x's shape."""
    x2, M, N = _flatten_up_gate(x, order, "silu_bwd")
    dev = require_gpu(x, dy)
    if dy.dtype != torch.bfloat16 or dy.numel() != M * N:
        raise ValueError("silu_bwd: dy must be bfloat16 with %d elements" % (M * N))
    dy2 = dy.reshape(M, N).contiguous()
    dx = torch.empty(x.shape, device=dev, dtype=x.dtype)
    if M * N == 0:
        return dx
    with on_device(dev):
        check(lib().mdy_swiglu_bwd(ptr(x2), ptr(dy2), ptr(dx), M, N, x2.stride(0) if M else 2 * N,
                                   int(order == "gate-up"), stream_ptr(dev)), "silu_bwd")
    return dx


class _SiluOps(torch.autograd.Function):
    """fp8_kernel.py:423-433."""

    @staticmethod
    def forward(ctx, x, order="up-gate"):
        ctx.x = x
        ctx.order = order
        return silu_fwd(x, order)

    @staticmethod
    def backward(ctx, dy):
        return silu_bwd(dy, ctx.x, ctx.order), None


triton_silu = _SiluOps.apply


def silu_act_quant(x: torch.Tensor, order: str = "up-gate", return_act: bool = False, dialect: str = "official"):
    """One pass: act = silu_fwd(x, order) and its 1x128 quantization.

    dialect "official": (y, s) as offical_kernel.act_quant(act) returns them (N % 128 == 0);
    dialect "deeplinear": (y, s) as fp8.quant_input(act, only_forward=True) returns them (padded,
    column-major scales).  With return_act=True the bf16 act comes back as a third value (the
    backward pass needs it); otherwise it is never written to memory.
    """
    x2, M, N = _flatten_up_gate(x, order, "silu_act_quant")
    dev = require_gpu(x)
    act = torch.empty(*x.shape[:-1], N, device=dev, dtype=x.dtype) if return_act else None
    gate_first = int(order == "gate-up")
    xs = x2.stride(0) if M else 2 * N
    if dialect == "official":
        assert N % 128 == 0
        y = torch.empty(*x.shape[:-1], N, device=dev, dtype=FP8)
        s = torch.empty(*x.shape[:-1], N // 128, device=dev, dtype=torch.float32)
        if M * N > 0:
            with on_device(dev):
                check(lib().mdy_swiglu(ptr(x2), ptr(act), ptr(y), ptr(s), M, N, xs, gate_first, M, N, N // 128, 1, 0,
                                       stream_ptr(dev)), "silu_act_quant")
    elif dialect == "deeplinear":
        PN = (N + 255) // 256 * 256
        PM = (M + 3) // 4 * 4
        y = torch.empty(PM, PN, device=dev, dtype=FP8)
        sbuf = torch.empty(PN // 128, PM, device=dev, dtype=torch.float32)
        if PM * PN > 0:
            with on_device(dev):
                check(lib().mdy_swiglu(ptr(x2), ptr(act), ptr(y), ptr(sbuf), M, N, xs, gate_first, PM, PN, 1, PM, 1,
                                       stream_ptr(dev)), "silu_act_quant")
        s = sbuf.transpose(0, 1)
    else:
        raise ValueError("dialect must be 'official' or 'deeplinear'")
    return (y, s, act) if return_act else (y, s)


def weight_quant_block(x: torch.Tensor, BLOCK_M: int = 128, BLOCK_N: int = 128,
                       dtype: torch.dtype = FP8) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 block quantizer with s = amax / 448 (fp8_kernel.py:124-138, kernel :88-122).

    x [M, N] bf16 with N % 128 == 0 (any strides); returns y [M, N] e4m3fn and s [M//128, N//128].
    """
    assert x.size(-1) % BLOCK_N == 0
    if BLOCK_M != 128 or BLOCK_N != 128:
        raise ValueError("only 128x128 blocks are implemented (the reference default)")
    if dtype != FP8:
        raise TypeError("only torch.float8_e4m3fn is implemented")
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise TypeError("weight_quant_block expects a 2-D bfloat16 tensor")
    dev = require_gpu(x)
    M, N = x.shape
    if M % 128 != 0:
        raise ValueError("weight_quant_block: M must be a multiple of 128 (the reference drops the ragged rows)")
    y = torch.empty(M, N, device=dev, dtype=FP8)
    s = torch.empty(M // 128, N // 128, device=dev, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_weight_quant(ptr(x), ptr(y), ptr(s), None, None, M, N, x.stride(0), x.stride(1), M, N, 0,
                                     stream_ptr(dev)), "weight_quant_block")
    return y, s
