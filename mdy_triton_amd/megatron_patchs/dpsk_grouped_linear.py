"""Padding of grouped (mixture-of-experts) activations to the row multiples the FP8 grouped path wants.

Drop-in for Fp8Padding / Fp8Unpadding of
/root/reference/triton_kernels/megatron_patchs/dpsk_grouped_linear.py:690-902 (module names, constructor and
`forward(inp, m_splits)` as there): every expert's rows are moved to a slot of cdiv(m, 256) * 256 rows, the rest of
the slot zero-filled, and back.  The reference does the copy with TransformerEngine's multi_padding_fused and the way
back with torch.split / torch.cat; here both directions are one HIP kernel (mdy_group_pad_rows) and each is the
other's gradient.  The grouped GEMM of this package needs no padding (its tiles follow the group boundaries); the
grouped quantizer that also emits the transposed copies (group_per_token_cast_to_fp8) does, as in the reference
(megatron_patchs/fp8_matmul.py:227), and this is how a ragged batch reaches it.

The GroupedLinear module of the same reference file wraps TransformerEngine's module machinery around the operators
of megatron_patchs/fp8_matmul.py and is not part of this package.
"""
import ctypes
from typing import List, Sequence, Tuple

import torch

from .._torch_glue import check, lib, on_device, ptr, require_gpu, stream_ptr

PAD_MULTIPLE = 256


def padded_splits(m_splits: Sequence[int], multiple: int = PAD_MULTIPLE) -> List[int]:
    return [(int(m) + multiple - 1) // multiple * multiple for m in m_splits]


def _move_rows(inp: torch.Tensor, m_splits: Sequence[int], unpad: bool, multiple: int) -> torch.Tensor:
    if any(int(m) < 0 for m in m_splits):
        raise ValueError("m_splits must be non-negative, got %s" % list(m_splits))
    dev = require_gpu(inp)
    x = inp.reshape(-1, inp.shape[-1])
    if not x.is_contiguous():
        x = x.contiguous()
    pads = padded_splits(m_splits, multiple)
    rows_in, rows_out = (sum(pads), sum(int(m) for m in m_splits)) if unpad else (sum(int(m) for m in m_splits), sum(pads))
    if x.size(0) != rows_in:
        raise ValueError("%s expects %d rows for m_splits %s, got %d" % ("unpadding" if unpad else "padding", rows_in,
                                                                        list(m_splits), x.size(0)))
    out = torch.empty(rows_out, x.size(1), dtype=x.dtype, device=dev)
    G = len(m_splits)
    if rows_out * x.size(1) == 0 or G == 0:
        return out
    splits = (ctypes.c_int64 * G)(*[int(m) for m in m_splits])
    with on_device(dev):
        check(lib().mdy_group_pad_rows(ptr(x), ptr(out), ctypes.cast(splits, ctypes.c_void_p), G,
                                       x.size(1) * x.element_size(), multiple, int(unpad), stream_ptr(dev)),
              "Fp8Unpadding" if unpad else "Fp8Padding")
    return out


def pad_groups(inp: torch.Tensor, m_splits: Sequence[int], multiple: int = PAD_MULTIPLE) -> torch.Tensor:
    """[sum m, H] -> [sum pad(m), H]: group g's rows at the start of its slot, zeros behind them."""
    return _move_rows(inp, m_splits, False, multiple)


def unpad_groups(inp: torch.Tensor, m_splits: Sequence[int], multiple: int = PAD_MULTIPLE) -> torch.Tensor:
    """[sum pad(m), H] -> [sum m, H]: the first m rows of every slot."""
    return _move_rows(inp, m_splits, True, multiple)


class _Fp8Padding(torch.autograd.Function):
    """dpsk_grouped_linear.py:798-846: forward pads, backward unpads the gradient."""

    @staticmethod
    def forward(ctx, inp, m_splits, padded_m_splits, is_grad_enabled):
        if is_grad_enabled:
            ctx.m_splits = list(m_splits)
            ctx.requires_dgrad = inp.requires_grad
        return pad_groups(inp, m_splits)

    @staticmethod
    def backward(ctx, grad_output):
        grad_input = unpad_groups(grad_output, ctx.m_splits) if ctx.requires_dgrad else None
        return grad_input, None, None, None


class _Fp8Unpadding(torch.autograd.Function):
    """dpsk_grouped_linear.py:690-739: forward unpads, backward pads the gradient (zeros in the padding rows)."""

    @staticmethod
    def forward(ctx, inp, m_splits, padded_m_splits, is_grad_enabled):
        if is_grad_enabled:
            ctx.m_splits = list(m_splits)
            ctx.requires_dgrad = inp.requires_grad
        return unpad_groups(inp, m_splits)

    @staticmethod
    def backward(ctx, grad_output):
        grad_input = pad_groups(grad_output, ctx.m_splits) if ctx.requires_dgrad else None
        return grad_input, None, None, None


class Fp8Padding(torch.nn.Module):
    """Pads every expert's rows to a multiple of 256; forward returns (padded tensor, padded_m_splits)
    (dpsk_grouped_linear.py:849-902)."""

    def __init__(self, num_gemms) -> None:
        super().__init__()
        self.num_gemms = num_gemms

    def forward(self, inp: torch.Tensor, m_splits: List[int]) -> Tuple[torch.Tensor, List[int]]:
        assert len(m_splits) == self.num_gemms, "Number of splits should match number of GEMMs."
        pads = padded_splits(m_splits)
        if torch.is_grad_enabled():
            out = _Fp8Padding.apply(inp, m_splits, pads, True)
        else:
            out = pad_groups(inp, m_splits)
        return out, pads


class Fp8Unpadding(torch.nn.Module):
    """Inverse of Fp8Padding: forward(inp, m_splits) takes the padded tensor and the UNPADDED splits
    (dpsk_grouped_linear.py:742-793)."""

    def __init__(self, num_gemms) -> None:
        super().__init__()
        self.num_gemms = num_gemms

    def forward(self, inp: torch.Tensor, m_splits: List[int]) -> torch.Tensor:
        assert len(m_splits) == self.num_gemms, "Number of splits should match number of GEMMs."
        pads = padded_splits(m_splits)
        if torch.is_grad_enabled():
            return _Fp8Unpadding.apply(inp, m_splits, pads, True)
        return unpad_groups(inp, m_splits)
