"""mdy_triton_amd: the DeepSeek-V3-style block-wise FP8 linear path of
mdy666/mdy_triton, rebuilt for AMD MI355X (gfx950) as hand-written HIP kernels
behind a C ABI.  Importing the package does not load the library; the first
operator call does, and raises if it has not been built."""
from .offical_kernel import act_quant, fp8_gemm, weight_dequant  # noqa: F401
from .fp8 import DeepLinear, add_bias, fp8_matmul, quant_grad_output, quant_input, quant_weight  # noqa: F401

from .fp8_kernel import (Fp8Linear, Fp8MLP, act_quant_block, fp8_ckpt_mlp, silu_act_quant, silu_bwd, silu_fwd, triton_silu,  # noqa: F401
                         weight_quant_block)

from .megatron_patchs.fp8_matmul import (fp8_grouped_matmul, group_per_token_cast_to_fp8, per_block_cast_to_fp8,  # noqa: F401
                         per_token_cast_to_fp8)

from .megatron_patchs.dpsk_grouped_linear import Fp8Padding, Fp8Unpadding  # noqa: F401

__all__ = ["Fp8Linear", "act_quant_block", "Fp8Padding", "Fp8Unpadding", "Fp8MLP", "fp8_ckpt_mlp", "per_token_cast_to_fp8", "group_per_token_cast_to_fp8", "per_block_cast_to_fp8", "fp8_grouped_matmul", "silu_fwd", "silu_bwd", "triton_silu", "silu_act_quant", "weight_quant_block", "act_quant", "weight_dequant", "fp8_gemm", "quant_input", "quant_weight", "quant_grad_output", "fp8_matmul", "add_bias",
           "DeepLinear"]
