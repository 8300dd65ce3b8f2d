"""DeepLinear: the block-wise FP8 linear layer and its operators on MI355X.

Drop-in for /root/reference/triton_kernels/dpsk_fp8linear/fp8.py: quant_input,
quant_weight, fp8_matmul, add_bias, _DeepLinear, DeepLinear keep their names,
arguments, padding rules and returned layouts.  The GEMM that the reference
delegates to deep_gemm.gemm_fp8_fp8_bf16_nt (fp8.py:310) is this package's own
gfx950 kernel.
"""
from typing import Optional, Tuple

import torch

from ._torch_glue import FP8, check, lib, on_device, ptr, require_gpu, stream_ptr


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def quant_input(x: torch.Tensor, only_forward: bool = True):
    """1x128 activation quantizer with clamp(amax, 0, 1e4) + 1e-8 (fp8.py:122-161).

    x [M, K] bf16, last dim unit-strided or not (a non-unit column stride is
    copied first).  Returns (y, s, y_t, s_t):
      y [PM, PN] e4m3fn, PN = cdiv(K,256)*256, PM = cdiv(M,4)*4;
      s logical [PM, PN/128] with strides (1, PM) (column-major, as fp8.py:134,161).
    Only only_forward=True is implemented: the transposed outputs belong to the
    backward pass.
    """
    if not only_forward:
        raise NotImplementedError("quant_input(only_forward=False): the backward-pass outputs are not built yet")
    if x.dim() != 2:
        raise ValueError("quant_input expects a 2-D tensor")
    if x.dtype != torch.bfloat16:
        raise TypeError("quant_input expects bfloat16, got %s" % x.dtype)
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
        check(lib().mdy_act_quant(ptr(x), ptr(y), ptr(s), M, K, x.stride(0) if M > 0 else K, PM, PN, 1, PM, 1,
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
    if x.dtype != torch.bfloat16:
        raise TypeError("quant_weight expects bfloat16, got %s" % x.dtype)
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
        check(lib().mdy_weight_quant(ptr(x), ptr(y), ptr(s), ptr(y_t), ptr(s_t), N, K, x.stride(0), x.stride(1),
                                     PM, PN, 1, stream_ptr(dev)), "quant_weight")
    return y, s, y_t, s_t


def add_bias(x: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """In-place x[..., :] += b in fp32, stored back as bf16 (fp8.py:297-305)."""
    if x.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise TypeError("add_bias expects bfloat16 tensors")
    if not x.is_contiguous() or not b.is_contiguous():
        raise ValueError("add_bias expects contiguous tensors")
    dev = require_gpu(x, b)
    N = x.size(-1)
    if b.numel() != N:
        raise ValueError("bias has %d elements, rows have %d" % (b.numel(), N))
    M = x.numel() // N if N else 0
    with on_device(dev):
        check(lib().mdy_add_bias(ptr(x), ptr(b), M, N, stream_ptr(dev)), "add_bias")
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
        check(lib().mdy_fp8_gemm_nt(ptr(qa), ptr(sa), sa.stride(0), sa.stride(1), ptr(qb), ptr(sb), ptr(out),
                                    ptr(bias), M, N, K, 0, stream_ptr(dev)), "fp8_matmul")
    return out


class _DeepLinear(torch.autograd.Function):
    """Forward of fp8.py:313-328: flatten, quantize input and weight, GEMM, bias, view back.

    The bias add is folded into the GEMM epilogue (same fp32 add, one rounding less
    than GEMM->bf16->add->bf16 only when a bias is present; see `fuse_bias`).
    """

    @staticmethod
    def forward(ctx, input, weight, bias, is_grad_enable, weight_cache=None, fuse_bias=False):
        inp_shape = input.shape
        x = input.reshape(-1, input.size(-1))
        q_inp, s_inp, _, _ = quant_input(x, only_forward=True)
        if weight_cache is not None:
            q_weight, s_weight = weight_cache
        else:
            q_weight, s_weight, _, _ = quant_weight(weight, only_forward=True)
        out = fp8_matmul(q_inp, s_inp, q_weight, s_weight, bias=bias if fuse_bias else None)
        if bias is not None and not fuse_bias:
            add_bias(out, bias)
        return out.view(*inp_shape[:-1], -1)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("DeepLinear backward (quant_grad_output + dgrad/wgrad GEMMs) is not built yet")


class DeepLinear(torch.nn.Linear):
    """nn.Linear whose forward runs the block-wise FP8 path (fp8.py:347-349).

    The bf16 master weight is quantized per 128x128 block; the result is cached
    and reused until the weight tensor changes (its version counter or storage),
    which removes the per-call re-quantization the reference notebook subtracts by
    hand.  Set `cache_weight=False` to re-quantize on every call as the reference
    does, `fuse_bias=True` to add the bias inside the GEMM epilogue.
    """

    cache_weight = True
    fuse_bias = False

    def _quantized_weight(self):
        w = self.weight
        key = (w.data_ptr(), w._version, tuple(w.shape), w.device)
        cached = getattr(self, "_wq_cache", None)
        if cached is not None and cached[0] == key:
            return cached[1]
        q, s, _, _ = quant_weight(w.detach(), only_forward=True)
        self._wq_cache = (key, (q, s))
        return q, s

    def forward(self, input):
        cache = self._quantized_weight() if self.cache_weight else None
        return _DeepLinear.apply(input, self.weight, self.bias, torch.is_grad_enabled(), cache, self.fuse_bias)
