"""SwiGLU and block quantizers of the FP8 MLP on MI355X.

Drop-in for the parts of /root/reference/triton_kernels/deepseekv3/fp8_kernel.py that sit
directly before the FP8 linear path: silu_fwd / silu_bwd / triton_silu (fp8_kernel.py:384-434),
weight_quant_block (:124-138), plus silu_act_quant, which fuses the `silu_fwd -> act_quant`
pair of the FP8 MLP (fp8_kernel.py:447-450, 500-515) into one pass over the up/gate tensor; and for
that file's own linear layer in the official dialect (s = amax / finfo.max, no clamp, no eps):
act_quant_block (:62-87), fp8_matmul (:214-252), fp8_matmul_bwd (:254-257), Fp8Linear (:259-313).
Both float8_e4m3fn and float8_e5m2 (the reference's default dtype, fp8_kernel.py:62, 124, 303) are implemented for the
official-dialect functions; e4m3fn runs the tuned kernels, e5m2 the general quantizer kernels and the GEMM with row scales
on both operands (a weight's 128x128 block scales are expanded to one per row for it).  The DeepLinear dialect and the
fused silu_act_quant are e4m3fn only.
"""
from typing import Optional, Tuple

import torch

from ._torch_glue import FP8, check, lib, on_device, ptr, require_gpu, stream_ptr, xt_code

_ORDERS = ("up-gate", "gate-up")


E5M2 = torch.float8_e5m2


def _require_e4m3(fp8_dtype, who: str):
    if fp8_dtype != FP8:
        raise TypeError("%s: only torch.float8_e4m3fn is implemented here, got %s" % (who, fp8_dtype))


def _fp8_mode(fp8_dtype, who: str):
    """(quantizer mode, GEMM operand format) of an fp8 dtype: official dialect with e4m3fn bytes, or with e5m2 bytes."""
    if fp8_dtype == FP8:
        return 0, 0
    if fp8_dtype == E5M2:
        return 2, 1
    raise TypeError("%s: fp8 dtype must be torch.float8_e4m3fn or torch.float8_e5m2, got %s" % (who, fp8_dtype))


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
                       dtype: torch.dtype = E5M2) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 block quantizer with s = amax / finfo(dtype).max (fp8_kernel.py:124-138, kernel :88-122); dtype
    defaults to float8_e5m2 as in the reference.

    x [M, N] (any strides, N % 128 == 0); returns y [M, N] of `dtype` and s [M//128, N//128].
    """
    assert x.size(-1) % BLOCK_N == 0
    if BLOCK_M != 128 or BLOCK_N != 128:
        raise ValueError("only 128x128 blocks are implemented (the reference default)")
    mode, _ = _fp8_mode(dtype, "weight_quant_block")
    if x.dim() != 2:
        raise TypeError("weight_quant_block expects a 2-D tensor")
    xt = xt_code(x, "weight_quant_block")
    dev = require_gpu(x)
    M, N = x.shape
    if M % 128 != 0:
        raise ValueError("weight_quant_block: M must be a multiple of 128 (the reference drops the ragged rows)")
    y = torch.empty(M, N, device=dev, dtype=dtype)
    s = torch.empty(M // 128, N // 128, device=dev, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_weight_quant_typed(ptr(x), xt, ptr(y), ptr(s), None, None, M, N, x.stride(0), x.stride(1), M, N, mode,
                                           stream_ptr(dev)), "weight_quant_block")
    return y, s


def _act_quant_transposed(x2: torch.Tensor, with_rows: bool, who: str, dtype: torch.dtype = FP8):
    """x2 [M, N] (any strides) -> (y, s, y_t_padded, s_t): the official-dialect row-wise quantization (None, None
    unless with_rows) and the quantized transpose y_t [N, PM] with s_t [N, PM/128], PM = cdiv(M, 128) * 128."""
    mode, _ = _fp8_mode(dtype, who)
    xt = xt_code(x2, who)
    dev = require_gpu(x2)
    M, N = x2.shape
    PM = (M + 127) // 128 * 128
    y = torch.empty(PM, N, device=dev, dtype=dtype) if with_rows else None
    s = torch.empty(PM, N // 128, device=dev, dtype=torch.float32) if with_rows else None
    y_t = torch.empty(N, PM, device=dev, dtype=dtype)
    s_t = torch.empty(N, PM // 128, device=dev, dtype=torch.float32)
    if PM * N > 0:
        with on_device(dev):
            check(lib().mdy_act_quant_transpose(ptr(x2), xt, ptr(y), ptr(s), ptr(y_t), ptr(s_t), M, N, x2.stride(0), x2.stride(1),
                                                PM, N, mode, stream_ptr(dev)), who)
    return y, s, y_t, s_t


def act_quant_block(x: torch.Tensor, transpose: bool = False, dtype: torch.dtype = E5M2,
                    BLOCK_N: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1x128 quantizer with s = amax / finfo(dtype).max (fp8_kernel.py:62-87); dtype defaults to float8_e5m2 as in the
    reference.

    transpose=False: (y like x, s [..., N/128]); with float8_e4m3fn the same as offical_kernel.act_quant.
    transpose=True: the flattened [M, N] input is quantized along M: y [N, M], s [N, cdiv(M, 128)] (a last group
    shorter than 128 is completed with zeros, as the reference's masked loads do).
    """
    assert x.size(-1) % BLOCK_N == 0
    if BLOCK_N != 128:
        raise ValueError("only BLOCK_N=128 is implemented (the reference default)")
    mode, _ = _fp8_mode(dtype, "act_quant_block")
    if not transpose:
        xc = x if x.is_contiguous() else x.contiguous()
        if mode == 0:
            from .offical_kernel import act_quant
            return act_quant(xc)
        xt = xt_code(xc, "act_quant_block")
        dev = require_gpu(xc)
        K = xc.size(-1)
        M = xc.numel() // K if K else 0
        y = torch.empty_like(xc, dtype=dtype)
        s = xc.new_empty(*xc.size()[:-1], K // 128, dtype=torch.float32)
        with on_device(dev):
            check(lib().mdy_act_quant_typed(ptr(xc), xt, 128, ptr(y), ptr(s), M, K, K, M, K, K // 128, 1, mode, stream_ptr(dev)),
                  "act_quant_block")
        return y, s
    x2 = x.reshape(-1, x.size(-1))
    M = x2.size(0)
    _, _, y_t, s_t = _act_quant_transposed(x2, False, "act_quant_block", dtype)
    return (y_t if y_t.size(1) == M else y_t[:, :M].contiguous()), s_t


def fp8_matmul(x: torch.Tensor, w: torch.Tensor, scale_x: torch.Tensor, scale_w: torch.Tensor,
               bias: Optional[torch.Tensor] = None, have_w: bool = True) -> torch.Tensor:
    """bf16 y = x . w^T on block-scaled FP8 operands, both float8_e4m3fn or both float8_e5m2 (fp8_kernel.py:214-252).

    have_w=True (forward, input gradient): x [..., K] with scale_x [..., K/128], w [N, K] with 128x128 block scales
    scale_w [N/128, K/128], optional bias [N] added in fp32.  have_w=False (weight gradient): x [M, K] and w [N, K]
    both carry one scale per row and 128 columns, scale_x [M, cdiv(K,128)], scale_w [N, cdiv(K,128)]; a K that is not a
    multiple of 128 is completed with zeros.
    """
    if x.dtype != w.dtype:
        raise TypeError("fp8_matmul expects operands of one fp8 dtype, got %s and %s" % (x.dtype, w.dtype))
    _, fmt = _fp8_mode(x.dtype, "fp8_matmul")
    if have_w:
        assert x.size(-1) % 128 == 0, 'in forward x @ w.T'
        x2 = x.reshape(-1, x.size(-1))
        sx2 = scale_x.reshape(-1, scale_x.size(-1))
        if fmt == 0:
            from .offical_kernel import fp8_gemm
            fused = bias is not None and bias.dtype == torch.bfloat16        # the GEMM epilogue takes a bf16 bias
            y = fp8_gemm(x2 if x2.is_contiguous() else x2.contiguous(), sx2.contiguous(),
                         w if w.is_contiguous() else w.contiguous(), scale_w.contiguous(), out_dtype=torch.bfloat16,
                         bias=bias.contiguous() if fused else None)
        else:
            dev = require_gpu(x, w, scale_x, scale_w)
            M, K = x2.shape
            N = w.size(0)
            x2c, wc = (x2 if x2.is_contiguous() else x2.contiguous()), (w if w.is_contiguous() else w.contiguous())
            sxc, swc = sx2.contiguous(), scale_w.contiguous()
            scales_ok = M == 0 or ((M - 1) * sxc.stride(0) + K // 128) * 4 < (1 << 31)
            if K <= 65536 and scales_ok and x2c.data_ptr() % 16 == 0 and wc.data_ptr() % 16 == 0:
                # e5m2 on the MFMA kernels (operand format bf8): tile kernels, or the weight-streaming / strip kernels
                # for up to 64 rows
                fused = bias is not None and bias.dtype == torch.bfloat16
                y = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
                with on_device(dev):
                    check(lib().mdy_fp8_gemm_nt_e5m2(ptr(x2c), ptr(sxc), sxc.stride(0), 1, ptr(wc), ptr(swc), ptr(y),
                                                     ptr(bias.contiguous()) if fused else None, M, N, K, 0, stream_ptr(dev)),
                          "fp8_matmul")
            else:
                # K beyond 65536, unaligned operands or scales spanning 2^31 bytes: the GEMM with row scales on both
                # operands, the weight's block scales expanded to one per row
                fused = False
                sw_rows = scale_w.repeat_interleave(128, dim=0)[:N].contiguous()
                y = _matmul_rowscaled(x2, sx2, w, sw_rows, M, N, K, dev, fmt)
        if bias is not None and not fused:                               # added in fp32 afterwards
            from .fp8 import add_bias
            add_bias(y, bias.contiguous())
        return y.view(*x.shape[:-1], w.size(0))
    assert x.size(0) % 128 == 0, 'in backward dy.T @ x or dy @ w'
    assert bias is None
    dev = require_gpu(x, w, scale_x, scale_w)
    x2 = x.reshape(-1, x.size(-1))
    M, K = x2.shape
    N = w.size(0)
    if w.size(1) != K or tuple(scale_x.shape[-2:]) != (M, (K + 127) // 128) or tuple(scale_w.shape) != (N, (K + 127) // 128):
        raise ValueError("shape mismatch: x %s scale_x %s w %s scale_w %s" % (tuple(x.shape), tuple(scale_x.shape), tuple(w.shape),
                                                                                tuple(scale_w.shape)))
    return _matmul_rowscaled(x2, scale_x.reshape(M, -1), w, scale_w, M, N, K, dev, fmt)


def _matmul_rowscaled(x2, sx, w, sw, M, N, K, dev, fmt=0):
    """[M, K] . [N, K]^T with per-row scales on both sides; operands may be column slices of K-padded buffers."""
    PK = (K + 127) // 128 * 128

    def k_padded(t):      # a [rows, K] view whose storage already runs to a multiple of 128 columns, zero filled
        if K == PK and t.stride(1) == 1 and t.stride(0) == K and t.data_ptr() % 16 == 0:
            return t
        full = torch.zeros(t.size(0), PK, device=dev, dtype=torch.uint8)
        full[:, :K] = t.view(torch.uint8)
        return full
    a, b = k_padded(x2), k_padded(w)
    out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    if M * N == 0:
        return out
    with on_device(dev):
        check(lib().mdy_fp8_gemm_nt_rowscaled(ptr(a), ptr(sx), sx.stride(0), sx.stride(1), ptr(b), ptr(sw), sw.stride(0),
                                              sw.stride(1), ptr(out), M, N, PK, fmt, 0, stream_ptr(dev)), "fp8_matmul")
    return out


def fp8_matmul_bwd(xt, w, dy, dyt, scale_xt, scale_w, scale_dy, scale_dyt):
    """Input and weight gradient of y = x . w^T from the quantized copies (fp8_kernel.py:254-257)."""
    dx = fp8_matmul(dy, w, scale_dy, scale_w, have_w=True)
    dw = fp8_matmul(dyt, xt, scale_dyt, scale_xt, have_w=False)
    return dx, dw


def _official_linear_backward(x2, w, dy2, need_dx, need_dw, fp8_dtype=FP8):
    """Gradients of y = x2 . w^T in the official dialect (fp8_kernel.py:274-301): dx = dy . w on the row-wise copy of dy
    and the block-quantized w^T, dw = dy^T . x on the transposed copies of dy and x (row scales on both operands).
    One kernel pass over dy gives both of its copies; the transposed copies keep their zero padding to a multiple of
    128 tokens."""
    _, fmt = _fp8_mode(fp8_dtype, "Fp8Linear.backward")
    M, K = x2.shape
    N = w.size(0)
    dev = x2.device
    dx = dw = None
    qdy, sdy, qdyt, sdyt = _act_quant_transposed(dy2, need_dx, "Fp8Linear.backward", fp8_dtype)
    if need_dx:
        qwt, swt = weight_quant_block(w.t(), dtype=fp8_dtype)       # [K, N]: the 128x128 blocks of w, transposed
        dx = fp8_matmul(qdy[:M], qwt, sdy[:M], swt, have_w=True)
    if need_dw:
        _, _, qxt, sxt = _act_quant_transposed(x2, False, "Fp8Linear.backward", fp8_dtype)
        dw = torch.empty(N, K, device=dev, dtype=torch.bfloat16)
        if qdyt.size(1) == 0:
            dw.zero_()                                   # no tokens: an empty sum
        elif N * K > 0:
            with on_device(dev):
                check(lib().mdy_fp8_gemm_nt_rowscaled(ptr(qdyt), ptr(sdyt), sdyt.stride(0), sdyt.stride(1), ptr(qxt), ptr(sxt),
                                                      sxt.stride(0), sxt.stride(1), ptr(dw), N, K, qdyt.size(1), fmt, 0,
                                                      stream_ptr(dev)), "Fp8Linear.backward")
    return dx, dw


class _Fp8LinearFunction(torch.autograd.Function):
    """fp8_kernel.py:259-301.  Forward: act_quant_block(x), weight_quant_block(w), GEMM with the bias in its epilogue.
    Backward: x and dy quantized along the tokens (transposed copies, one kernel pass over dy for both of its copies),
    w^T block-quantized; dx = dy . w through the tile kernels, dw = dy^T . x through the GEMM with row scales on both
    operands.  The transposed copies keep their zero padding to a multiple of 128 tokens, so any token count works."""

    @staticmethod
    def forward(ctx, x, w, bias, fp8_dtype):
        _fp8_mode(fp8_dtype, "Fp8Linear")
        input_shape = x.shape
        x2 = x.reshape(-1, input_shape[-1])
        qx, sx = act_quant_block(x2, dtype=fp8_dtype)
        qw, sw = weight_quant_block(w, dtype=fp8_dtype)
        y = fp8_matmul(qx, qw, sx, sw, bias, have_w=True)
        ctx.save_for_backward(x2, w)
        ctx.bias = bias
        ctx.fp8_dtype = fp8_dtype
        ctx.input_shape = input_shape
        return y.view(*input_shape[:-1], w.size(0))

    @staticmethod
    def backward(ctx, dy):
        dy2 = dy.reshape(-1, dy.size(-1))
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        dbias = dy2.sum(0) if ctx.bias is not None and ctx.needs_input_grad[2] else None
        x2, w = ctx.saved_tensors
        dx, dw = _official_linear_backward(x2, w, dy2, ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.fp8_dtype)
        return (dx.view(ctx.input_shape) if dx is not None else None), dw, dbias, None


fp8_linear_with_quant_ops = _Fp8LinearFunction.apply


class Fp8Linear(torch.nn.Linear):
    """nn.Linear on the official-dialect FP8 path (fp8_kernel.py:303-313); fp8_dtype float8_e5m2 (the reference's
    default) or float8_e4m3fn (what its notebook passes, and the faster one here)."""

    def __init__(self, in_features, out_features, bias=True, device=None, dtype=None, fp8_dtype=E5M2):
        super().__init__(in_features, out_features, bias, device, dtype)
        _fp8_mode(fp8_dtype, "Fp8Linear")
        self.fp8_dtype = fp8_dtype

    def forward(self, x):
        return fp8_linear_with_quant_ops(x, self.weight, self.bias, self.fp8_dtype)


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


class _Fp8MlpCkptOfficial(torch.autograd.Function):
    """The same memory-saving step in the official dialect, as the reference runs it (fp8_kernel.py:436-494):
    act_quant_block / weight_quant_block / fp8_matmul, the activation quantized by the fused SwiGLU kernel in the
    forward (same bytes as silu_fwd + act_quant_block), x the only activation kept."""

    @staticmethod
    def forward(ctx, x, w_up_gate, w_down, fp8_dtype=E5M2, order="up-gate"):
        mode, _ = _fp8_mode(fp8_dtype, "fp8_ckpt_mlp")
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        qx, sx = act_quant_block(x2, dtype=fp8_dtype)
        qwu, swu = weight_quant_block(w_up_gate, dtype=fp8_dtype)
        qwd, swd = weight_quant_block(w_down, dtype=fp8_dtype)
        up_gate = fp8_matmul(qx, qwu, sx, swu)
        if mode == 0:
            qact, sact = silu_act_quant(up_gate, order, dialect="official")       # one pass, e4m3fn
        else:
            qact, sact = act_quant_block(silu_fwd(up_gate, order), dtype=fp8_dtype)
        y = fp8_matmul(qact, qwd, sact, swd)
        ctx.save_for_backward(x2, w_up_gate, w_down)
        ctx.order, ctx.shape, ctx.fp8_dtype = order, shape, fp8_dtype
        return y.view(*shape[:-1], w_down.size(0))

    @staticmethod
    def backward(ctx, dy):
        x2, w_up_gate, w_down = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.size(-1))
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        qx, sx = act_quant_block(x2, dtype=ctx.fp8_dtype)
        qwu, swu = weight_quant_block(w_up_gate, dtype=ctx.fp8_dtype)
        up_gate = fp8_matmul(qx, qwu, sx, swu)
        act = silu_fwd(up_gate, ctx.order)
        dact, dw_down = _official_linear_backward(act, w_down, dy2, True, True, ctx.fp8_dtype)
        dup_gate = silu_bwd(dact, up_gate, ctx.order)
        dx, dw_up_gate = _official_linear_backward(x2, w_up_gate, dup_gate, True, True, ctx.fp8_dtype)
        return dx.view(ctx.shape), dw_up_gate, dw_down, None, None


def fp8_ckpt_mlp(x, w_up_gate, w_down, fp8_dtype=E5M2, order="up-gate", dialect="official"):
    """Memory-saving FP8 MLP step with the reference's positional order and default dtype (fp8_kernel.py:436-494:
    `fp8_ckpt_mlp(h, w1, w2, self.fp8_dtype, self.order)`).  dialect "official" (the reference's: s = amax /
    finfo(fp8_dtype).max, float8_e5m2 or float8_e4m3fn) or "deeplinear" (clamp 1e4 + eps 1e-8, the quantizers of
    dpsk_fp8linear/fp8.py; float8_e4m3fn only)."""
    if dialect == "official":
        return _Fp8MlpCkptOfficial.apply(x, w_up_gate, w_down, fp8_dtype, order)
    if dialect != "deeplinear":
        raise ValueError("dialect must be 'official' or 'deeplinear'")
    return _Fp8MlpCkptOps.apply(x, w_up_gate, w_down, fp8_dtype, order)


class Fp8MLP(torch.nn.Module):
    """SwiGLU MLP on the FP8 linear path (fp8_kernel.py:500-515): up/gate projection, silu(gate) * up, down
    projection, both projections block-wise FP8 (1x128 activation and 128x128 weight scales), no biases.  fp8_dtype
    float8_e5m2 (the reference's default) or float8_e4m3fn.

    dialect "official" (default, what the reference's Fp8MLP computes: its projections are `Fp8Linear`s,
    s = amax / finfo.max) or "deeplinear" (`DeepLinear` projections: clamp 1e4 + eps 1e-8, optional weight cache;
    e4m3fn only).
    Without gradients the activation goes from the up/gate GEMM to the down GEMM through the fused
    SwiGLU + quantizer (one pass, the bf16 activation is never written).  With gradients the default is the
    composition linear -> triton_silu -> linear; `low_memory` (attribute or call argument, as in the
    reference) keeps only the input for the backward pass and recomputes up/gate and the activation there.
    """

    def __init__(self, hidden_size, intermediate_size, order="up-gate", fp8_dtype=E5M2, low_memory=False,
                 device=None, dtype=torch.bfloat16, dialect="official"):
        super().__init__()
        if dialect == "deeplinear":
            _require_e4m3(fp8_dtype, "Fp8MLP(dialect='deeplinear')")
        else:
            _fp8_mode(fp8_dtype, "Fp8MLP")
        assert order in _ORDERS, "please indicate the order of input, up-gate or gate-up"
        if dialect not in ("official", "deeplinear"):
            raise ValueError("dialect must be 'official' or 'deeplinear'")
        if dialect == "official":
            self.up_gate_proj = Fp8Linear(hidden_size, intermediate_size * 2, bias=False, device=device, dtype=dtype,
                                          fp8_dtype=fp8_dtype)
            self.down_proj = Fp8Linear(intermediate_size, hidden_size, bias=False, device=device, dtype=dtype,
                                       fp8_dtype=fp8_dtype)
        else:
            from .fp8 import DeepLinear
            self.up_gate_proj = DeepLinear(hidden_size, intermediate_size * 2, bias=False, device=device, dtype=dtype)
            self.down_proj = DeepLinear(intermediate_size, hidden_size, bias=False, device=device, dtype=dtype)
        self.dialect = dialect
        self.order = order
        self.fp8_dtype = fp8_dtype
        self.low_memory = low_memory

    def forward(self, hidden_states, low_memory=False):
        up, down = self.up_gate_proj, self.down_proj
        needs_grad = torch.is_grad_enabled() and (hidden_states.requires_grad or up.weight.requires_grad or
                                                  down.weight.requires_grad)
        if not needs_grad or low_memory or self.low_memory:
            if self.dialect == "official":
                return _Fp8MlpCkptOfficial.apply(hidden_states, up.weight, down.weight, self.fp8_dtype, self.order)
            # cached quantized weights (when the projections cache); the forward needs no transposed copies
            return _Fp8MlpCkptOps.apply(hidden_states, up.weight, down.weight, self.fp8_dtype, self.order,
                                        up._quantized_weight(False) if up.cache_weight else None,
                                        down._quantized_weight(False) if down.cache_weight else None)
        return down(triton_silu(up(hidden_states), self.order))
