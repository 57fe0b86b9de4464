"""`sgl_kernel.gemm` (sgl-kernel/python/sgl_kernel/gemm.py:13-42,100-145): the same names."""

from sglang_amd.sgl_kernel.gemm import (  # noqa: F401
    fp8_blockwise_scaled_mm,
    fp8_scaled_mm,
    int8_scaled_mm,
    sgl_per_tensor_quant_fp8,
    sgl_per_token_group_quant_fp8,
    sgl_per_token_group_quant_int8,
    sgl_per_token_quant_fp8,
)
