"""`sgl_kernel.moe` names of the grouped block-FP8 GEMM and the data movement around it."""

from sglang_amd.sgl_kernel.moe import (  # noqa: F401
    apply_shuffle_mul_sum,
    fp8_blockwise_scaled_grouped_mm,
    prepare_moe_input,
    shuffle_rows,
)
