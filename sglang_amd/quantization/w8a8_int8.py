"""INT8 linear glue (python/sglang/srt/layers/quantization/w8a8_int8.py:329-391)."""

from __future__ import annotations

from typing import Optional

import torch

from ..sgl_kernel import int8_scaled_mm
from ..sgl_kernel.gemm import int8_linear
from .int8_kernel import per_token_quant_int8

# Rows up to which quantization and GEMM go to one operator (sglq_w8a8_int8_linear: a single kernel on the
# shapes of the decode kernel without split-K, bit-identical to the two calls); above it the two calls below.
FUSED_QUANT_MAX_ROWS = 2


def _fusable(x: torch.Tensor, weight: torch.Tensor) -> bool:
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    return (0 < rows <= FUSED_QUANT_MAX_ROWS and x.is_cuda and x.dtype in (torch.bfloat16, torch.float16)
            and x.shape[-1] % 128 == 0 and x.is_contiguous() and weight.dim() == 2 and weight.stride(0) == 1)


def process_weights_after_loading(weight: torch.Tensor, weight_scale: torch.Tensor):
    """Stored [N, K] int8 weight -> the [K, N] transposed view the GEMM takes, and the
    [N, 1] fp32 scales unchanged (w8a8_int8.py:337-338)."""
    return weight.t(), weight_scale


def apply_w8a8_int8_linear(
    x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """W8A8Int8LinearMethod.apply (w8a8_int8.py:371-391): per-token INT8 quantization
    of x followed by int8_scaled_mm with the transposed weight view; decode rows take both steps in one
    operator with the same result."""
    if _fusable(x, weight):
        return int8_linear(x.view(-1, x.shape[-1]), weight, weight_scale, bias).view(*x.shape[:-1], weight.shape[1])
    x_q, x_scale = per_token_quant_int8(x)
    return int8_scaled_mm(x_q, weight, x_scale, weight_scale, out_dtype=x.dtype, bias=bias)


class W8A8Int8LinearMethod:
    """process_weights_after_loading and apply of W8A8Int8LinearMethod (w8a8_int8.py:329-338,
    371-391) on any object with `weight` ([N, K] int8) and `weight_scale` ([N, 1] fp32)."""

    def __init__(self, quantization_config=None):
        self.quantization_config = quantization_config

    def process_weights_after_loading(self, layer) -> None:
        weight, weight_scale = process_weights_after_loading(layer.weight, layer.weight_scale.data)
        layer.weight = torch.nn.Parameter(weight, requires_grad=False)
        layer.weight_scale = torch.nn.Parameter(weight_scale, requires_grad=False)

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        return apply_w8a8_int8_linear(x, layer.weight, layer.weight_scale, bias)
