"""Stand-in for the part of the reference's ``sgl_kernel`` package that serves the
W8A8 quantized-linear path and its grouped (MoE) GEMM (sgl-kernel/python/sgl_kernel/__init__.py)."""

from .gemm import (
    fp8_blockwise_scaled_mm,
    fp8_scaled_mm,
    int8_mm_i32,
    int8_scaled_mm,
    sgl_per_token_group_quant_fp8,
    sgl_per_token_group_quant_int8,
    sgl_per_tensor_quant_fp8,
    sgl_per_token_quant_fp8,
)
from .moe import apply_shuffle_mul_sum, fp8_blockwise_scaled_grouped_mm, prepare_moe_input, shuffle_rows, silu_and_mul

__all__ = [
    "apply_shuffle_mul_sum",
    "fp8_blockwise_scaled_grouped_mm",
    "prepare_moe_input",
    "shuffle_rows",
    "silu_and_mul",
    "fp8_blockwise_scaled_mm",
    "fp8_scaled_mm",
    "int8_mm_i32",
    "int8_scaled_mm",
    "sgl_per_token_group_quant_fp8",
    "sgl_per_token_group_quant_int8",
    "sgl_per_tensor_quant_fp8",
    "sgl_per_token_quant_fp8",
]
