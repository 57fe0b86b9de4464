"""Scale bookkeeping of fused FP8 modules at load time
(python/sglang/srt/layers/quantization/utils.py:59-121).  Plain torch, not timed."""

from __future__ import annotations

from typing import List, Tuple, Union

import torch


def per_tensor_dequantize(tensor: torch.Tensor, inv_scale: Union[float, torch.Tensor]) -> torch.Tensor:
    """Codes times their scale, in half precision (utils.py:59-64)."""
    return tensor.to(torch.float16) * inv_scale


def all_close_1d(x: torch.Tensor) -> bool:
    """Whether all entries of a vector are (nearly) the same (utils.py:67-69)."""
    assert x.dim() == 1
    return bool(torch.allclose(x, x[0].expand_as(x)))


def convert_to_channelwise(weight_scale: torch.Tensor, logical_widths: List[int]) -> torch.Tensor:
    """One scale per fused shard (or a single scalar) spread to one per output channel, [sum, 1]
    fp32: what fp8_scaled_mm takes (utils.py:72-92)."""
    total = sum(logical_widths)
    if weight_scale.dim() == 0:
        return weight_scale.to(torch.float32).reshape(1, 1).expand(total, 1).contiguous()
    widths = torch.tensor(logical_widths, device=weight_scale.device)
    per_shard = weight_scale.reshape(-1)[: len(logical_widths)].to(torch.float32)
    return per_shard.repeat_interleave(widths).reshape(total, 1)


def requantize_with_max_scale(
    weight: torch.Tensor, weight_scale: torch.Tensor, logical_widths: List[int]
) -> Tuple[torch.Tensor, torch.Tensor]:
    """The shards of a fused module re-quantized in place with the largest of their scales, so
    that one per-tensor scale serves the module (utils.py:95-121).  A checkpoint that stored the
    module fused has loaded one scale and left the others at their initial value (the most
    negative FP8 number): then the weight already has that single scale and is left alone."""
    from .fp8_kernel import scaled_fp8_quant

    max_w_scale = weight_scale.max()
    unfused = bool(weight_scale[-1] > torch.finfo(torch.float8_e4m3fn).min)
    if unfused:
        start = 0
        for idx, width in enumerate(logical_widths):
            shard = per_tensor_dequantize(weight[start : start + width, :], weight_scale[idx])
            weight[start : start + width, :], _ = scaled_fp8_quant(shard, max_w_scale)
            start += width
    return max_w_scale, weight
