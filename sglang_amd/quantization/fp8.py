"""What Fp8LinearMethod does with a layer's tensors after loading, for the branches that end in
this library's GEMMs (python/sglang/srt/layers/quantization/fp8.py:333-439), as a function of
tensors instead of a method of a layer object."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .fp8_kernel import fp8_max
from .utils import convert_to_channelwise


def quantize_weight_per_channel(weight: torch.Tensor, eps: float = 1e-10) -> Tuple[torch.Tensor, torch.Tensor]:
    """per_token_group_quant_fp8(weight, weight.shape[-1]) (fp8.py:366-369): every output channel is
    one group: scale = max(amax, eps) / 448, codes = weight / scale.  Done in torch on the weight's
    device: it runs once per layer at load time, and a row-long group is no size the activation
    kernel is built for."""
    w = weight.float()
    scale = w.abs().amax(dim=-1, keepdim=True).clamp(min=eps) / fp8_max
    q = (w / scale).clamp(min=-fp8_max, max=fp8_max).to(torch.float8_e4m3fn)
    return q, scale


def process_weights_after_loading(
    weight: torch.Tensor,
    weight_scale: Optional[torch.Tensor] = None,
    logical_widths: Optional[List[int]] = None,
    input_scale: Optional[torch.Tensor] = None,
    block_quant: bool = False,
    is_checkpoint_fp8_serialized: bool = True,
    static_activations: bool = False,
):
    """Returns (weight, weight_scale, input_scale) as apply_fp8_linear / w8a8_block_fp8_linear take them.

    * block_quant: the [N, K] weight and its [N/128, K/128] scales unchanged (fp8.py:335-358).
    * a 16-bit checkpoint: per-channel quantization, the [K, N] transposed view of the codes and
      [N, 1] scales, no input scale (fp8.py:362-378).
    * an FP8 checkpoint with one scale per fused shard: the scales spread to one per channel, the
      transposed view, and for static activations the largest input scale (fp8.py:382-433)."""
    if block_quant:
        return weight, weight_scale, None
    if not is_checkpoint_fp8_serialized:
        qweight, scale = quantize_weight_per_channel(weight)
        return qweight.t(), scale.contiguous(), None
    assert weight_scale is not None and logical_widths is not None
    scale = convert_to_channelwise(weight_scale, logical_widths)
    in_scale = input_scale.max() if (static_activations and input_scale is not None) else None
    return weight.t(), scale, in_scale


class Fp8Config:
    """The fields of Fp8Config (fp8.py:96-190) that the linear method reads."""

    def __init__(
        self,
        is_checkpoint_fp8_serialized: bool = False,
        activation_scheme: str = "dynamic",
        weight_block_size: Optional[List[int]] = None,
    ):
        if activation_scheme not in ("static", "dynamic"):
            raise ValueError(f"Unsupported activation scheme {activation_scheme}")
        if weight_block_size is not None:
            if not is_checkpoint_fp8_serialized:
                raise ValueError("block-wise quantization needs an FP8 checkpoint")
            if len(weight_block_size) != 2:
                raise ValueError(f"weight_block_size must have two entries, got {len(weight_block_size)}")
            if activation_scheme != "dynamic":
                raise ValueError("block-wise quantization takes dynamic activation scales only")
        self.is_checkpoint_fp8_serialized = is_checkpoint_fp8_serialized
        self.activation_scheme = activation_scheme
        self.weight_block_size = weight_block_size


class Fp8LinearMethod:
    """process_weights_after_loading and apply of Fp8LinearMethod (fp8.py:204-223,333-488) for
    the branches that end in this library's GEMMs, on any object with `weight` and, per branch,
    `weight_scale_inv` (block quantization), `weight_scale` + `logical_widths` (FP8 checkpoint)
    and `input_scale` (static activations)."""

    def __init__(self, quant_config: Fp8Config):
        from .fp8_utils import cutlass_fp8_supported, dispatch_w8a8_block_fp8_linear

        self.quant_config = quant_config
        self.cutlass_fp8_supported = cutlass_fp8_supported()
        self.block_quant = quant_config.weight_block_size is not None
        self.w8a8_block_fp8_linear = dispatch_w8a8_block_fp8_linear()

    def process_weights_after_loading(self, layer) -> None:
        cfg = self.quant_config
        static = cfg.activation_scheme == "static"
        if self.block_quant:
            layer.weight = torch.nn.Parameter(layer.weight.data, requires_grad=False)
            layer.weight_scale_inv = torch.nn.Parameter(layer.weight_scale_inv.data, requires_grad=False)
            return
        weight, weight_scale, input_scale = process_weights_after_loading(
            layer.weight.data,
            getattr(layer, "weight_scale", None),
            getattr(layer, "logical_widths", None),
            getattr(layer, "input_scale", None),
            block_quant=False,
            is_checkpoint_fp8_serialized=cfg.is_checkpoint_fp8_serialized,
            static_activations=static,
        )
        layer.weight = torch.nn.Parameter(weight, requires_grad=False)
        layer.weight_scale = torch.nn.Parameter(weight_scale, requires_grad=False)
        layer.input_scale = torch.nn.Parameter(input_scale, requires_grad=False) if input_scale is not None else None

    def apply(self, layer, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        from .fp8_utils import apply_fp8_linear

        if self.block_quant:
            return self.w8a8_block_fp8_linear(
                input=x,
                weight=layer.weight,
                block_size=self.quant_config.weight_block_size,
                weight_scale=layer.weight_scale_inv,
                input_scale=None,
                bias=bias,
            )
        return apply_fp8_linear(
            input=x,
            weight=layer.weight,
            weight_scale=layer.weight_scale,
            input_scale=layer.input_scale,
            bias=bias,
            cutlass_fp8_supported=self.cutlass_fp8_supported,
            use_per_token_if_dynamic=False,
        )
