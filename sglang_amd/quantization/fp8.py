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
