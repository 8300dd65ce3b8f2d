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


def _require_e4m3(fp8_dtype, who: str):
    if fp8_dtype != FP8:
        raise TypeError("%s: only torch.float8_e4m3fn is implemented, got %s (the reference defaults to "
                        "float8_e5m2; pass fp8_dtype=torch.float8_e4m3fn)" % (who, fp8_dtype))


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


class _Fp8MlpCkptOps(torch.autograd.Function):
    """Memory-saving MLP step (fp8_kernel.py:436-494): the forward keeps only x and the two weights; the
    backward recomputes the up/gate projection and the activation, then runs the two weight-gradient and
    the two input-gradient GEMMs on the quantizers' transposed copies."""

    @staticmethod
    def forward(ctx, x, w_up_gate, w_down, fp8_dtype=FP8, order="up-gate", up_gate_cache=None, down_cache=None):
        from . import fp8 as L
        _require_e4m3(fp8_dtype, "fp8_ckpt_mlp")
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        M, H = x2.shape
        N2, inter = w_up_gate.size(0), w_down.size(1)
        q_x, s_x, _, _ = L.quant_input(x2, only_forward=True)
        q_wu, s_wu = (up_gate_cache or L.quant_weight(w_up_gate, only_forward=True))[:2]
        q_wd, s_wd = (down_cache or L.quant_weight(w_down, only_forward=True))[:2]
        up_gate = L.fp8_matmul(q_x[:M], s_x[:M], q_wu[:N2], s_wu[:L._cdiv(N2, 128)])
        q_act, s_act = silu_act_quant(up_gate, order, dialect="deeplinear")      # act itself is never written
        y = L.fp8_matmul(q_act[:M], s_act[:M], q_wd[:w_down.size(0)], s_wd[:L._cdiv(w_down.size(0), 128)])
        ctx.save_for_backward(x2, w_up_gate, w_down)
        ctx.order, ctx.shape, ctx.dims = order, shape, (M, H, N2, inter)
        return y.view(*shape[:-1], w_down.size(0))

    @staticmethod
    def backward(ctx, dy):
        from . import fp8 as L
        x2, w_up_gate, w_down = ctx.saved_tensors
        M, H, N2, inter = ctx.dims
        out_f = w_down.size(0)
        dy2 = dy.reshape(-1, out_f)
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        cd = L._cdiv
        # recompute up_gate and act; the transposed copies feed the weight gradients
        q_x, s_x, q_xt, s_xt = L.quant_input(x2, only_forward=False)
        q_wu, s_wu, q_wut, s_wut = L.quant_weight(w_up_gate, only_forward=False)
        up_gate = L.fp8_matmul(q_x[:M], s_x[:M], q_wu[:N2], s_wu[:cd(N2, 128)])
        act = silu_fwd(up_gate, ctx.order)
        _, _, q_actt, s_actt = L.quant_input(act, only_forward=False)
        _, _, q_wdt, s_wdt = L.quant_weight(w_down, only_forward=False)
        q_dy, s_dy, q_dyt, s_dyt = L.quant_grad_output(dy2)
        dact = L.fp8_matmul(q_dy[:M], s_dy[:M], q_wdt[:inter], s_wdt[:cd(inter, 128)])
        dw_down = L.fp8_matmul(q_dyt[:out_f], s_dyt[:out_f], q_actt[:inter], s_actt[:cd(inter, 128)])
        dup_gate = silu_bwd(dact, up_gate, ctx.order)
        q_du, s_du, q_dut, s_dut = L.quant_grad_output(dup_gate)
        dx = L.fp8_matmul(q_du[:M], s_du[:M], q_wut[:H], s_wut[:cd(H, 128)]).view(ctx.shape)
        dw_up_gate = L.fp8_matmul(q_dut[:N2], s_dut[:N2], q_xt[:H], s_xt[:cd(H, 128)])
        return dx, dw_up_gate, dw_down, None, None, None, None


def fp8_ckpt_mlp(x, w_up_gate, w_down, fp8_dtype=FP8, order="up-gate"):
    """Memory-saving FP8 MLP step with the reference's positional order (fp8_kernel.py:436-494:
    `fp8_ckpt_mlp(h, w1, w2, self.fp8_dtype, self.order)`).  Only float8_e4m3fn is implemented: the reference's
    default, float8_e5m2, raises TypeError here."""
    return _Fp8MlpCkptOps.apply(x, w_up_gate, w_down, fp8_dtype, order)


class Fp8MLP(torch.nn.Module):
    """SwiGLU MLP on the FP8 linear path (fp8_kernel.py:500-515): up/gate projection, silu(gate) * up, down
    projection, both projections block-wise FP8 (`DeepLinear`: e4m3fn, 1x128 activation and 128x128 weight
    scales), no biases.

    Without gradients the activation goes from the up/gate GEMM to the down GEMM through the fused
    SwiGLU + quantizer (one pass, the bf16 activation is never written).  With gradients the default is the
    composition DeepLinear -> triton_silu -> DeepLinear; `low_memory` (attribute or call argument, as in the
    reference) keeps only the input for the backward pass and recomputes up/gate and the activation there.
    """

    def __init__(self, hidden_size, intermediate_size, order="up-gate", fp8_dtype=FP8, low_memory=False,
                 device=None, dtype=torch.bfloat16):
        super().__init__()
        _require_e4m3(fp8_dtype, "Fp8MLP")
        assert order in _ORDERS, "please indicate the order of input, up-gate or gate-up"
        from .fp8 import DeepLinear
        self.up_gate_proj = DeepLinear(hidden_size, intermediate_size * 2, bias=False, device=device, dtype=dtype)
        self.down_proj = DeepLinear(intermediate_size, hidden_size, bias=False, device=device, dtype=dtype)
        self.order = order
        self.fp8_dtype = fp8_dtype
        self.low_memory = low_memory

    def forward(self, hidden_states, low_memory=False):
        up, down = self.up_gate_proj, self.down_proj
        needs_grad = torch.is_grad_enabled() and (hidden_states.requires_grad or up.weight.requires_grad or
                                                  down.weight.requires_grad)
        if not needs_grad or low_memory or self.low_memory:
            # cached quantized weights (re-quantized when a weight changes); the forward needs no transposed copies
            return _Fp8MlpCkptOps.apply(hidden_states, up.weight, down.weight, self.fp8_dtype, self.order,
                                        up._quantized_weight(False) if up.cache_weight else None,
                                        down._quantized_weight(False) if down.cache_weight else None)
        return down(triton_silu(up(hidden_states), self.order))
