"""SwiGLU of the Megatron patch: act = silu(gate) * up on the un-split [.., 2D] output of the first MLP projection.

Drop-in for /root/reference/triton_kernels/megatron_patchs/swiglu.py (`_FusedSiLUNoSplit` :76-134, `swiglu_impl` :137-138,
which Megatron calls with the gate in the first half: order 'gate-up').  The kernels are the package's mdy_swiglu /
mdy_swiglu_bwd (the same arithmetic as deepseekv3/fp8_kernel.py's silu_fwd / silu_bwd)."""
from ..fp8_kernel import _SiluOps, silu_bwd, silu_fwd  # noqa: F401

_FusedSiLUNoSplit = _SiluOps


def fused_up_gate_silu_no_split(x, order="up-gate"):
    """y [.., D] = up * silu(gate) from x [.., 2D] holding up and gate side by side in the given order."""
    return _SiluOps.apply(x, order)


def swiglu_impl(x, bias, fp8_input_store=False):
    """Megatron's bias_swiglu_impl replacement (swiglu.py:137-138): the bias and the fp8 flag are ignored there too."""
    return _SiluOps.apply(x, "gate-up")
