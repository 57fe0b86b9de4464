"""INT8 linear glue (python/sglang/srt/layers/quantization/w8a8_int8.py:329-391)."""

from __future__ import annotations

from typing import Optional

import torch

from ..sgl_kernel import int8_scaled_mm
from .int8_kernel import per_token_quant_int8


def process_weights_after_loading(weight: torch.Tensor, weight_scale: torch.Tensor):
    """Stored [N, K] int8 weight -> the [K, N] transposed view the GEMM takes, and the
    [N, 1] fp32 scales unchanged (w8a8_int8.py:337-338)."""
    return weight.t(), weight_scale


def apply_w8a8_int8_linear(
    x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """W8A8Int8LinearMethod.apply (w8a8_int8.py:371-391): per-token INT8 quantization
    of x followed by int8_scaled_mm with the transposed weight view."""
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
        x_q, x_scale = per_token_quant_int8(x)
        return int8_scaled_mm(x_q, layer.weight, x_scale, layer.weight_scale, out_dtype=x.dtype, bias=bias)
