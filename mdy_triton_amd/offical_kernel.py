"""DeepSeek-V3 "official" FP8 operators on MI355X: act_quant, weight_dequant, fp8_gemm.

Drop-in for /root/reference/triton_kernels/deepseekv3/offical_kernel.py (same
names, argument meaning, asserts and output shapes); the work is done by
hand-written gfx950 kernels behind the C ABI in include/mdy_fp8.h.
"""
from typing import Optional, Tuple

import torch

from ._torch_glue import FP8, check, gemm_workspace, lib, on_device, out_code, ptr, require_gpu, stream_ptr, warn_if_scalar_gemm, xt_code


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """y = e4m3fn(x / s), s = max|x| / 448 per `block_size` contiguous elements.

    Mirrors act_quant at offical_kernel.py:21-28: x contiguous, last dim a multiple
    of block_size; returns (y like x in float8_e4m3fn, s fp32 [..., K/block_size]).
    """
    assert x.is_contiguous()
    assert x.size(-1) % block_size == 0
    if block_size < 8 or block_size > 512 or block_size & (block_size - 1):
        raise ValueError("block_size must be a power of two from 8 to 512 (128 is the tuned case), got %d" % block_size)
    xt = xt_code(x, "act_quant")      # bf16 with block_size 128 runs the tuned kernel; everything else the general one
    dev = require_gpu(x)
    K = x.size(-1)
    M = x.numel() // K if K else 0
    y = torch.empty_like(x, dtype=FP8)
    s = x.new_empty(*x.size()[:-1], K // block_size, dtype=torch.float32)
    with on_device(dev):
        check(lib().mdy_act_quant_typed(ptr(x), xt, block_size, ptr(y), ptr(s), M, K, K, M, K, K // block_size, 1, 0,
                                        stream_ptr(dev)), "act_quant")
    return y, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y[m, n] = fp32(x[m, n]) * s[m // 128, n // 128] in the default dtype.

    Mirrors weight_dequant at offical_kernel.py:46-53 (2-D contiguous x and s; output
    dtype = torch.get_default_dtype() unless out_dtype is given).
    """
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    if block_size < 8 or block_size & (block_size - 1):
        raise ValueError("block_size must be a power of two >= 8, got %d" % block_size)
    if x.dtype != FP8 or s.dtype != torch.float32:
        raise TypeError("weight_dequant expects float8_e4m3fn weights and float32 scales")
    dev = require_gpu(x, s)
    N, K = x.size()
    if tuple(s.shape) != ((N + block_size - 1) // block_size, (K + block_size - 1) // block_size):
        raise ValueError("scale shape %s does not match weight %s" % (tuple(s.shape), tuple(x.shape)))
    dtype = out_dtype or torch.get_default_dtype()
    y = torch.empty_like(x, dtype=dtype)
    with on_device(dev):
        check(lib().mdy_weight_dequant_block(ptr(x), ptr(s), ptr(y), N, K, block_size, out_code(dtype), stream_ptr(dev)),
              "weight_dequant")
    return y


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor, *,
             out_dtype: Optional[torch.dtype] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """C = A . B^T with per-128-K activation scales and 128x128 weight scales.

    Mirrors fp8_gemm at offical_kernel.py:100-109: a [..., K] e4m3fn, a_s [..., K/128]
    fp32, b [N, K] e4m3fn, b_s [ceil(N/128), ceil(K/128)] fp32, all contiguous; returns
    [..., N] in the default dtype.  `out_dtype` and a bf16 `bias` [N] are extensions.
    """
    assert a.is_contiguous() and b.is_contiguous()
    assert a_s.is_contiguous() and b_s.is_contiguous()
    if a.dtype != FP8 or b.dtype != FP8:
        raise TypeError("fp8_gemm expects float8_e4m3fn operands")
    if a_s.dtype != torch.float32 or b_s.dtype != torch.float32:
        raise TypeError("fp8_gemm expects float32 scales")
    dev = require_gpu(a, a_s, b, b_s, bias)
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0)
    KB = (K + 127) // 128
    if b.dim() != 2 or b.size(1) != K:
        raise ValueError("b must be [N, K] with K=%d, got %s" % (K, tuple(b.shape)))
    if a_s.numel() != M * KB or tuple(b_s.shape) != ((N + 127) // 128, KB):
        raise ValueError("scale shapes do not match: a_s %s, b_s %s" % (tuple(a_s.shape), tuple(b_s.shape)))
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 [N] tensor")
    dtype = out_dtype or torch.get_default_dtype()
    c = a.new_empty(*a.size()[:-1], N, dtype=dtype)
    if K % 128 != 0 and M * N * K >= (1 << 24):
        # A K tail (the masked loads of offical_kernel.py:82-83) would send the whole problem to the one-thread-per-output
        # kernel; zero bytes contribute nothing to any sum, so a problem of any size is completed with zero columns to the
        # next multiple of 128 instead (the scales already have one column for the partial block) and runs on the MFMA kernels.
        PK = KB * 128
        a2 = torch.zeros(M, PK, dtype=torch.uint8, device=dev)
        a2[:, :K] = a.reshape(M, K).view(torch.uint8)
        b2 = torch.zeros(N, PK, dtype=torch.uint8, device=dev)
        b2[:, :K] = b.view(torch.uint8)
        a, b, K = a2.view(FP8), b2.view(FP8), PK
    with on_device(dev):
        warn_if_scalar_gemm(a, b, KB, 1, M, N, K, "fp8_gemm")
        ws = gemm_workspace(dev, M, N, K)      # scratch for shapes that are split along K, else None
        check(lib().mdy_fp8_gemm_nt_ws(ptr(a), ptr(a_s), KB, 1, ptr(b), ptr(b_s), ptr(c), ptr(bias), M, N, K,
                                       out_code(dtype), ptr(ws), ws.numel() if ws is not None else 0,
                                       stream_ptr(dev)), "fp8_gemm")
    return c
