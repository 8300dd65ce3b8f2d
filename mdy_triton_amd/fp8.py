"""DeepLinear: the block-wise FP8 linear layer and its operators on MI355X.

Drop-in for /root/reference/triton_kernels/dpsk_fp8linear/fp8.py: quant_input,
quant_weight, fp8_matmul, add_bias, _DeepLinear, DeepLinear keep their names,
arguments, padding rules and returned layouts.  The GEMM that the reference
delegates to deep_gemm.gemm_fp8_fp8_bf16_nt (fp8.py:310) is this package's own
gfx950 kernel.
"""
from typing import Optional, Tuple

import torch

from ._torch_glue import FP8, check, gemm_workspace, lib, on_device, ptr, require_gpu, stream_ptr, warn_if_scalar_gemm, xt_code


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _quant_transpose(x: torch.Tensor, t_mode: int, who: str):
    """Shared launcher of the two training-time quantizers (row-wise copy + quantized transpose)."""
    if x.dim() != 2:
        raise ValueError("%s expects a 2-D tensor" % who)
    xt = xt_code(x, who)
    dev = require_gpu(x)
    M, K = x.shape
    PM, PN = _cdiv(M, 256) * 256, _cdiv(K, 256) * 256
    A, B = PM // 128, PN // 128
    y = torch.empty(PM, PN, device=dev, dtype=FP8)
    s = torch.empty(B, PM, device=dev, dtype=torch.float32)
    y_t = torch.empty(PN, PM, device=dev, dtype=FP8)
    s_t = torch.empty((A, PN) if t_mode == 0 else (B, A), device=dev, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_quant_transpose_typed(ptr(x), xt, ptr(y), ptr(s), ptr(y_t), ptr(s_t), M, K, x.stride(0), x.stride(1),
                                        PM, PN, PM, t_mode, stream_ptr(dev)), who)
    return y, s.transpose(0, 1), y_t, s_t


def quant_grad_output(x: torch.Tensor):
    """Output-gradient quantizer of the backward pass (fp8.py:46-77).

    x [M, N] bf16, any strides.  Returns (y, s, y_t, s_t) with PM = cdiv(M,256)*256,
    PN = cdiv(N,256)*256: y [PM, PN] quantized along N in groups of 128, s logical
    [PM, PN/128] with strides (1, PM); y_t [PN, PM] quantized along M in groups of
    128, s_t logical [PN, PM/128] with strides (1, PN).
    """
    y, s, y_t, s_t = _quant_transpose(x, 0, "quant_grad_output")
    return y, s, y_t, s_t.transpose(0, 1)


def quant_input(x: torch.Tensor, only_forward: bool = True):
    """1x128 activation quantizer with clamp(amax, 0, 1e4) + 1e-8 (fp8.py:122-161).

    x [M, K] bf16, last dim unit-strided or not (a non-unit column stride is
    copied first in the forward-only case).  Returns (y, s, y_t, s_t):
      y [PM, PN] e4m3fn, PN = cdiv(K,256)*256, PM = cdiv(M,4)*4 (cdiv(M,256)*256 when
      only_forward=False);
      s logical [PM, PN/128] with strides (1, PM) (column-major, as fp8.py:134,161);
      with only_forward=False also y_t [PN, PM], the transposed copy quantized per
      128x128 block, and its scales s_t [PN/128, PM/128]; otherwise None, None.
    """
    if not only_forward:
        return _quant_transpose(x, 1, "quant_input")
    if x.dim() != 2:
        raise ValueError("quant_input expects a 2-D tensor")
    xt = xt_code(x, "quant_input")
    dev = require_gpu(x)
    M, K = x.shape
    if K > 0 and x.stride(1) != 1:
        x = x.contiguous()
    PN = _cdiv(K, 256) * 256
    B = PN // 128
    PM = _cdiv(M, 4) * 4
    y = torch.empty(PM, PN, device=dev, dtype=FP8)
    s = torch.empty(B, PM, device=dev, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_act_quant_typed(ptr(x), xt, 128, ptr(y), ptr(s), M, K, x.stride(0) if M > 0 else K, PM, PN, 1, PM, 1,
                                        stream_ptr(dev)), "quant_input")
    return y, s.transpose(0, 1), None, None


def quant_weight(x: torch.Tensor, only_forward: bool = True):
    """128x128 block weight quantizer with clamp + eps (fp8.py:206-247).

    x [N, K] bf16 (any strides).  Returns (y, s, y_t, s_t): y [PM, PN] e4m3fn with rows
    padded to 128 (256 when only_forward=False) and columns to 256, s [PM/128, PN/128];
    with only_forward=False also the transposed copy y_t [PN, PM], s_t [PN/128, PM/128].
    """
    if x.dim() != 2:
        raise ValueError("quant_weight expects a 2-D tensor")
    xt = xt_code(x, "quant_weight")
    dev = require_gpu(x)
    N, K = x.shape
    BA = 128 if only_forward else 256
    PM, PN = _cdiv(N, BA) * BA, _cdiv(K, 256) * 256
    A, B = PM // 128, PN // 128
    y = torch.empty(PM, PN, device=dev, dtype=FP8)
    s = torch.empty(A, B, device=dev, dtype=torch.float32)
    y_t = s_t = None
    if not only_forward:
        y_t = torch.empty(PN, PM, device=dev, dtype=FP8)
        s_t = torch.empty(B, A, device=dev, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_weight_quant_typed(ptr(x), xt, ptr(y), ptr(s), ptr(y_t), ptr(s_t), N, K, x.stride(0), x.stride(1),
                                     PM, PN, 1, stream_ptr(dev)), "quant_weight")
    return y, s, y_t, s_t


def add_bias(x: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """In-place x[..., :] += b in fp32, stored back as bf16 (fp8.py:297-305)."""
    if x.dtype != torch.bfloat16:
        raise TypeError("add_bias expects a bfloat16 x (the GEMM's output type), got %s" % x.dtype)
    bt = xt_code(b, "add_bias")
    if not x.is_contiguous() or not b.is_contiguous():
        raise ValueError("add_bias expects contiguous tensors")
    dev = require_gpu(x, b)
    N = x.size(-1)
    if b.numel() != N:
        raise ValueError("bias has %d elements, rows have %d" % (b.numel(), N))
    M = x.numel() // N if N else 0
    with on_device(dev):
        check(lib().mdy_add_bias_typed(ptr(x), ptr(b), bt, M, N, stream_ptr(dev)), "add_bias")
    return x


def fp8_matmul(qa: torch.Tensor, sa: torch.Tensor, qb: torch.Tensor, sb: torch.Tensor,
               out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[qa.size(0), qb.size(0)] (bf16) = block-scaled qa . qb^T (fp8.py:307-311).

    sa is the logical [M, K/128] activation scale with arbitrary strides (the
    column-major tensor quant_input returns is used in place); sb [N/128, K/128]
    contiguous.  `bias` (bf16 [N]) is an extension folded into the epilogue.
    """
    if qa.dtype != FP8 or qb.dtype != FP8:
        raise TypeError("fp8_matmul expects float8_e4m3fn operands")
    if not qa.is_contiguous() or not qb.is_contiguous() or not sb.is_contiguous():
        raise ValueError("fp8_matmul expects contiguous qa, qb and sb")
    dev = require_gpu(qa, sa, qb, sb, out, bias)
    M, K = qa.shape
    N = qb.size(0)
    KB = _cdiv(K, 128)
    if qb.size(1) != K or tuple(sa.shape) != (M, KB) or tuple(sb.shape) != (_cdiv(N, 128), KB):
        raise ValueError("shape mismatch: qa %s sa %s qb %s sb %s" % (tuple(qa.shape), tuple(sa.shape),
                                                                       tuple(qb.shape), tuple(sb.shape)))
    if out is None:
        out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (M, N) or not out.is_contiguous():
        raise ValueError("out must be a contiguous bfloat16 [M, N] tensor")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 [N] tensor")
    with on_device(dev):
        warn_if_scalar_gemm(qa, qb, sa.stride(0), sa.stride(1), M, N, K, "fp8_matmul")
        ws = gemm_workspace(dev, M, N, K)      # scratch for shapes that are split along K, else None
        check(lib().mdy_fp8_gemm_nt_ws(ptr(qa), ptr(sa), sa.stride(0), sa.stride(1), ptr(qb), ptr(sb), ptr(out),
                                       ptr(bias), M, N, K, 0, ptr(ws), ws.numel() if ws is not None else 0,
                                       stream_ptr(dev)), "fp8_matmul")
    return out


class _DeepLinear(torch.autograd.Function):
    """fp8.py:313-344: forward = flatten, quantize input and weight, GEMM, bias, view back;
    backward = quantize the output gradient both ways, dgrad = dy . W, wgrad = dy^T . x,
    both as block-scaled FP8 GEMMs on the transposed copies saved by the forward.

    The GEMMs run on the unpadded row counts (the quantizers pad rows to 4/128/256, the
    padding is never multiplied), so shapes that are not multiples of 256 work and no
    result is sliced.  The bias add can be folded into the GEMM epilogue (`fuse_bias`).
    """

    @staticmethod
    def forward(ctx, input, weight, bias, is_grad_enable, weight_cache=None, fuse_bias=False):
        inp_shape = input.shape
        x = input.reshape(-1, input.size(-1))
        M, K = x.shape
        N = weight.size(0)
        need_dgrad = bool(is_grad_enable and input.requires_grad)
        need_wgrad = bool(is_grad_enable and weight.requires_grad)
        # fp8.py:318: the transposed input copy is only needed for wgrad
        q_inp, s_inp, q_inp_t, s_inp_t = quant_input(x, only_forward=not need_wgrad)
        if weight_cache is not None:
            q_weight, s_weight, q_weight_t, s_weight_t = weight_cache
        else:
            q_weight, s_weight, q_weight_t, s_weight_t = quant_weight(weight, only_forward=not need_dgrad)
        if need_dgrad and q_weight_t is None:
            raise RuntimeError("DeepLinear: the cached weight has no transposed copy but dgrad is required")
        if is_grad_enable:
            ctx.inp_shape = inp_shape
            ctx.dims = (M, N, K)
            ctx.quantized = (q_inp_t, s_inp_t, q_weight_t, s_weight_t)
            ctx.has_bias = bias is not None
        fuse_bias = bool(fuse_bias and bias is not None and bias.dtype == torch.bfloat16)    # the epilogue takes a bf16 bias
        out = fp8_matmul(q_inp[:M], s_inp[:M], q_weight[:N], s_weight[:_cdiv(N, 128)],
                         bias=bias if fuse_bias else None)
        if bias is not None and not fuse_bias:
            add_bias(out, bias)
        return out.view(*inp_shape[:-1], N)

    @staticmethod
    def backward(ctx, grad_output):
        q_inp_t, s_inp_t, q_weight_t, s_weight_t = ctx.quantized
        M, N, K = ctx.dims
        dy = grad_output.reshape(-1, N)
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        q_dy, s_dy, q_dy_t, s_dy_t = quant_grad_output(dy)
        dgrad = wgrad = grad_bias = None
        if ctx.needs_input_grad[0]:
            # [M, PN] . [K, PN]^T, contraction over the (zero-padded) output features
            dgrad = fp8_matmul(q_dy[:M], s_dy[:M], q_weight_t[:K], s_weight_t[:_cdiv(K, 128)]).view(*ctx.inp_shape)
        if ctx.needs_input_grad[1]:
            # [N, PM] . [K, PM]^T, contraction over the (zero-padded) tokens
            wgrad = fp8_matmul(q_dy_t[:N], s_dy_t[:N], q_inp_t[:K], s_inp_t[:_cdiv(K, 128)])
        if ctx.has_bias and ctx.needs_input_grad[2]:
            grad_bias = dy.sum(0)
        return dgrad, wgrad, grad_bias, None, None, None


class DeepLinear(torch.nn.Linear):
    """nn.Linear whose forward and backward run the block-wise FP8 path (fp8.py:347-349).

    By default the bf16 master weight is quantized per 128x128 block on every call, as the
    reference does (fp8.py:320).  `cache_weight = True` keeps the quantized copies between
    calls; the owner of the weight then says when it changed:

      * `invalidate_weight_cache()` (or `set_first_micro_batch(True)`, the name the reference's
        Megatron patch uses for the same signal, megatron_patchs/manger.py:77-86) after every
        optimizer step.  It is REQUIRED after updates that go through `weight.data`
        (`weight.data.copy_(main_param)`, `weight.data.mul_(...)`: what Megatron's, apex's and
        DeepSpeed's optimizers do): those do not bump the tensor's version counter, so nothing
        else can see them;
      * in-place updates through the tensor itself (`weight.mul_()`, `optimizer.step()` of
        torch.optim) bump the version counter and a new storage changes the data pointer; both are
        noticed without a call.

    `check_weight_cache = True` (or the environment variable MDY_FP8_CHECK_WEIGHT_CACHE=1)
    verifies every cache hit against a checksum of the weight taken when it was quantized and
    raises if they differ - a debugging aid (one reduction and one host synchronisation per call).
    `fuse_bias = True` adds the bias inside the GEMM epilogue.
    """

    cache_weight = False
    fuse_bias = False
    check_weight_cache = False

    @staticmethod
    def _fingerprint(w: torch.Tensor) -> int:
        """Exact 64-bit sum of the weight's 16-bit patterns (integer arithmetic, so order does not matter)."""
        return int(torch.sum(w.detach().contiguous().view(torch.int16), dtype=torch.int64).item())

    def invalidate_weight_cache(self) -> None:
        """Forget the cached quantized weight: the next forward quantizes the current one."""
        self._wq_cache = None

    def set_first_micro_batch(self, flag: bool = True) -> None:
        """flag=True marks the weight as updated since it was last quantized (the first micro-batch
        of a step in the reference's Megatron patch); False leaves the cache as it is."""
        if flag:
            self.invalidate_weight_cache()

    def _quantized_weight(self, with_transpose: bool):
        import os
        w = self.weight
        key = (w.data_ptr(), w._version, tuple(w.shape), w.device)
        checking = self.check_weight_cache or os.environ.get("MDY_FP8_CHECK_WEIGHT_CACHE", "0") not in ("", "0")
        cached = getattr(self, "_wq_cache", None)
        if cached is not None and cached[0] == key and (cached[1][2] is not None or not with_transpose):
            if checking and cached[2] is not None and cached[2] != self._fingerprint(w):
                raise RuntimeError(
                    "DeepLinear: the weight changed since its quantized copy was cached (an update through "
                    "`.data`, which bumps no version counter); call invalidate_weight_cache() after such updates")
            return cached[1]
        quantized = quant_weight(w.detach(), only_forward=not with_transpose)
        self._wq_cache = (key, quantized, self._fingerprint(w) if checking else None)
        return quantized

    def forward(self, input):
        grad = torch.is_grad_enabled()
        cache = self._quantized_weight(grad and input.requires_grad) if self.cache_weight else None
        return _DeepLinear.apply(input, self.weight, self.bias, grad, cache, self.fuse_bias)
