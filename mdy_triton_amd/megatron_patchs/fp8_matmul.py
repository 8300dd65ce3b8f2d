"""Quantizers and GEMMs of the FP8 (grouped) linear layers on MI355X.

Drop-in for the operator functions of /root/reference/triton_kernels/megatron_patchs/fp8_matmul.py:
per_token_cast_to_fp8 (:96-135), group_per_token_cast_to_fp8 (:218-247), per_block_cast_to_fp8
(:334-392), fp8_matmul (:394-398) and fp8_grouped_matmul (:400-413, the DeepGEMM m-grouped
contiguous GEMM).  Same names, arguments, padding rules and returned layouts; the Megatron /
TransformerEngine module classes that call them are not part of this package.
"""
import ctypes
from typing import List, Optional, Sequence

import torch

from .._torch_glue import FP8, check, lib, on_device, ptr, require_gpu, stream_ptr, xt_code
from ..fp8 import _cdiv, fp8_matmul, quant_input  # noqa: F401  (fp8_matmul is re-exported under the reference's name)


def _check_2d(x, who):
    """2-D bf16 / fp16 / fp32 input; returns its type code for the typed entry points."""
    if x.dim() != 2:
        raise TypeError("%s expects a 2-D tensor" % who)
    return xt_code(x, who)


def per_token_cast_to_fp8(x: torch.Tensor, output_transpose: bool = False):
    """1x128 quantizer with clamp + eps; with output_transpose also the 128x1 column-wise
    quantization of the transpose (fp8_matmul.py:96-135).

    Returns (y, s, y_t, s_t): y [PM, PN], s logical [PM, PN/128] (strides (1, PM)); PM = cdiv(M,4)*4 and
    y_t = s_t = None without output_transpose, else PM = cdiv(M,128)*128, y_t [PN, PM],
    s_t logical [PN, PM/128] (strides (1, PN)).  PN = cdiv(N,256)*256.
    """
    if not output_transpose:
        return quant_input(x, only_forward=True)
    xt = _check_2d(x, "per_token_cast_to_fp8")
    dev = require_gpu(x)
    M, N = x.shape
    PM, PN = _cdiv(M, 128) * 128, _cdiv(N, 256) * 256
    y = torch.empty(PM, PN, device=dev, dtype=FP8)
    s = torch.empty(PN // 128, PM, device=dev, dtype=torch.float32)
    y_t = torch.empty(PN, PM, device=dev, dtype=FP8)
    s_t = torch.empty(PM // 128, PN, device=dev, dtype=torch.float32)
    if PM * PN > 0:
        with on_device(dev):
            check(lib().mdy_quant_transpose_typed(ptr(x), xt, ptr(y), ptr(s), ptr(y_t), ptr(s_t), M, N, x.stride(0), x.stride(1), PM, PN,
                                            PM, 0, stream_ptr(dev)), "per_token_cast_to_fp8")
    return y, s.transpose(0, 1), y_t, s_t.transpose(0, 1)


def group_per_token_cast_to_fp8(x_all: torch.Tensor, m_splits: Sequence[int]):
    """Row-wise quantization of all rows plus, per expert group, the column-wise quantized transpose
    (fp8_matmul.py:218-247).  Every group size and N must be multiples of 256 (asserted there at :227).

    Returns (y_all [M, N], s_all logical [M, N/128] with strides (1, M), [y_t of group g: [N, m_g]],
    [s_t of group g: logical [N, m_g/128]]).
    """
    xt = _check_2d(x_all, "group_per_token_cast_to_fp8")
    dev = require_gpu(x_all)
    Mtot, N = x_all.shape
    if sum(m_splits) != Mtot:
        raise ValueError("m_splits sum to %d, x_all has %d rows" % (sum(m_splits), Mtot))
    y_all = torch.empty(Mtot, N, device=dev, dtype=FP8)
    s_all = torch.empty(N // 128, Mtot, device=dev, dtype=torch.float32)
    yt_all, st_all = [], []
    row = 0
    with on_device(dev):
        for mg in m_splits:
            assert mg % 256 == 0 and N % 256 == 0
            y_t = torch.empty(N, mg, device=dev, dtype=FP8)
            s_t = torch.empty(mg // 128, N, device=dev, dtype=torch.float32)
            if mg > 0:
                x = x_all[row:row + mg]
                check(lib().mdy_quant_transpose_typed(ptr(x), xt, ptr(y_all[row:]), s_all.data_ptr() + 4 * row, ptr(y_t), ptr(s_t), mg, N,
                                                x.stride(0), x.stride(1), mg, N, Mtot, 0, stream_ptr(dev)),
                      "group_per_token_cast_to_fp8")
            yt_all.append(y_t)
            st_all.append(s_t.transpose(0, 1))
            row += mg
    return y_all, s_all.transpose(0, 1), yt_all, st_all


def per_block_cast_to_fp8(x, output_normal: bool = True, output_transpose: bool = False):
    """128x128 block quantizer with clamp + eps for one weight or a list of equally shaped weights
    (fp8_matmul.py:334-392): rows padded to 128 (256 with output_transpose), columns to 128 (256 with
    output_normal).  Returns (y, s) and/or (y_t, s_t) in that order, with a leading group dimension
    when a list of more than one weight is given.
    """
    xs: List[torch.Tensor] = list(x) if isinstance(x, (list, tuple)) else [x]
    for w in xs:
        xt = _check_2d(w, "per_block_cast_to_fp8")
        if w.shape != xs[0].shape or w.dtype != xs[0].dtype:
            raise ValueError("per_block_cast_to_fp8: all weights must have the same shape")
    dev = require_gpu(*xs)
    G = len(xs)
    M, N = xs[0].shape
    BA, BB = (256 if output_transpose else 128), (256 if output_normal else 128)
    PM, PN = _cdiv(M, BA) * BA, _cdiv(N, BB) * BB
    A, B = PM // 128, PN // 128
    if not (output_normal or output_transpose):
        return ()
    # a copy that is not asked for is neither allocated nor written (the kernel takes NULL for it)
    y = torch.empty(G, PM, PN, device=dev, dtype=FP8) if output_normal else None
    s = torch.empty(G, A, B, device=dev, dtype=torch.float32) if output_normal else None
    y_t = torch.empty(G, PN, PM, device=dev, dtype=FP8) if output_transpose else None
    s_t = torch.empty(G, B, A, device=dev, dtype=torch.float32) if output_transpose else None
    if PM * PN > 0:
        with on_device(dev):
            for g, w in enumerate(xs):
                check(lib().mdy_weight_quant_typed(ptr(w), xt, ptr(y[g]) if output_normal else None, ptr(s[g]) if output_normal else None,
                                             ptr(y_t[g]) if output_transpose else None,
                                             ptr(s_t[g]) if output_transpose else None, M, N, w.stride(0), w.stride(1), PM, PN, 1,
                                             stream_ptr(dev)), "per_block_cast_to_fp8")
    post = (lambda t: t.squeeze(0)) if G == 1 else (lambda t: t)
    out = ()
    if output_normal:
        out += (post(y), post(s))
    if output_transpose:
        out += (post(y_t), post(s_t))
    return out


def fp8_grouped_matmul(qa: torch.Tensor, sa: torch.Tensor, qb: torch.Tensor, sb: torch.Tensor, m_splits: Sequence[int],
                       out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[rows of group g] = block-scaled qa[rows of group g] . qb[g]^T, bf16 (fp8_matmul.py:400-413).

    qa [M, K] e4m3fn with M = sum(m_splits); sa logical [M, K/128] (any strides); qb [G, N, K]; sb
    [G, N/128, K/128]; group sizes need no alignment.  `bias` (bf16 [G, N]) is an extension folded into
    the epilogue.
    """
    if qa.dtype != FP8 or qb.dtype != FP8:
        raise TypeError("fp8_grouped_matmul expects float8_e4m3fn operands")
    if qb.dim() != 3 or not qa.is_contiguous() or not qb.is_contiguous() or not sb.is_contiguous():
        raise ValueError("fp8_grouped_matmul expects contiguous qa [M, K], qb [G, N, K] and sb")
    dev = require_gpu(qa, sa, qb, sb, out, bias)
    M, K = qa.shape
    G, N, _ = qb.shape
    KB = _cdiv(K, 128)
    if len(m_splits) != G or sum(m_splits) != M or any(m < 0 for m in m_splits):
        raise ValueError("m_splits %s does not describe %d groups over %d rows" % (list(m_splits), G, M))
    if qb.size(2) != K or tuple(sa.shape) != (M, KB) or tuple(sb.shape) != (G, _cdiv(N, 128), KB):
        raise ValueError("shape mismatch: qa %s sa %s qb %s sb %s" % (tuple(qa.shape), tuple(sa.shape), tuple(qb.shape),
                                                                       tuple(sb.shape)))
    if out is None:
        out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (M, N) or not out.is_contiguous():
        raise ValueError("out must be a contiguous bfloat16 [M, N] tensor")
    if bias is not None and (bias.dtype != torch.bfloat16 or tuple(bias.shape) != (G, N) or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 [G, N] tensor")
    if M * N == 0:
        return out
    splits = (ctypes.c_int64 * G)(*[int(m) for m in m_splits])
    with on_device(dev):
        check(lib().mdy_fp8_grouped_gemm_nt(ptr(qa), ptr(sa), sa.stride(0), sa.stride(1), ptr(qb), ptr(sb), ptr(out), ptr(bias),
                                            ctypes.cast(splits, ctypes.c_void_p), G, N, K, 0, stream_ptr(dev)),
              "fp8_grouped_matmul")
    return out
