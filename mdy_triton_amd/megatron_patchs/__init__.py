"""Operator functions of /root/reference/triton_kernels/megatron_patchs (fp8_matmul.py) on MI355X.
Only the quantizers, the GEMMs and the CustomManger funnel with its quantized-weight cache (manger.py) are
mirrored; the Megatron / TransformerEngine module patches that call them are outside this package."""
