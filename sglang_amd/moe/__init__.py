"""MoE expert layer on the grouped block-scaled FP8 GEMM
(python/sglang/srt/layers/moe/cutlass_moe.py)."""

from .cutlass_moe import cutlass_fused_experts_fp8

__all__ = ["cutlass_fused_experts_fp8"]
