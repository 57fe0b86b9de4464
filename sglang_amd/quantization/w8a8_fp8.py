"""The W8A8-FP8 linear method's tensor flow: per-channel FP8 weights, per-token dynamic FP8
activations (python/sglang/srt/layers/quantization/w8a8_fp8.py:97-189).

A `layer` here is any object with `weight` ([N, K]) and, for an FP8 checkpoint, `weight_scale`
([N, 1] fp32) attributes: an nn.Module or a plain namespace.  Weight creation and loading
belong to the model loader and are not mirrored."""

from __future__ import annotations

from typing import Optional

import torch
from torch.nn import Parameter

from .fp8 import quantize_weight_per_channel
from .fp8_utils import apply_fp8_linear, cutlass_fp8_supported


class W8A8Fp8Config:
    """The one field of W8A8Fp8Config (w8a8_fp8.py:47-77) that the linear method reads."""

    def __init__(self, is_checkpoint_fp8_serialized: bool = False):
        self.is_checkpoint_fp8_serialized = is_checkpoint_fp8_serialized

    @classmethod
    def from_config(cls, config: dict) -> "W8A8Fp8Config":
        quant_method = config.get("quant_method", "")
        return cls("compressed-tensors" in quant_method or "w8a8_fp8" in quant_method)


class W8A8Fp8LinearMethod:
    """process_weights_after_loading and apply of W8A8Fp8LinearMethod (w8a8_fp8.py:97-189)."""

    def __init__(self, quantization_config: W8A8Fp8Config):
        self.cutlass_fp8_supported = cutlass_fp8_supported()
        self.quantization_config = quantization_config

    def process_weights_after_loading(self, layer) -> None:
        if self.quantization_config.is_checkpoint_fp8_serialized:
            # codes and per-channel scales come from the checkpoint: only the [K, N] view is taken (:110-111)
            weight_scale = layer.weight_scale.detach()
            layer.weight = Parameter(layer.weight.t(), requires_grad=False)
            layer.weight_scale = Parameter(weight_scale, requires_grad=False)
            return
        # a 16-bit checkpoint: every output channel is one quantization group (:114-121); the
        # reference's other branch, one scale per tensor for torch._scaled_mm, has no use here
        qweight, weight_scale = quantize_weight_per_channel(layer.weight)
        layer.weight = Parameter(qweight.t(), requires_grad=False)
        layer.weight_scale = Parameter(weight_scale.contiguous(), requires_grad=False)
        layer.input_scale = None

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        return apply_fp8_linear(
            x,
            layer.weight,
            layer.weight_scale,
            bias=bias,
            cutlass_fp8_supported=self.cutlass_fp8_supported,
        )
