"""apply_w8a8_block_int8_linear with the reference's call sequence
(python/sglang/srt/layers/quantization/int8_utils.py:11-33)."""

from __future__ import annotations

from typing import List, Optional

import torch

from .int8_kernel import per_token_group_quant_int8, w8a8_block_int8_matmul


def apply_w8a8_block_int8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    block_size: List[int],
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    assert input_scale is None
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    q_input, x_scale = per_token_group_quant_int8(input_2d, block_size[1])
    if bias is not None and bias.dtype == input.dtype and bias.is_contiguous() and bias.numel() == weight.shape[0]:
        # the matmul and `output + bias` (int8_utils.py:26-32) in one kernel, same two roundings
        output = w8a8_block_int8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input.dtype, bias=bias)
    else:
        output = w8a8_block_int8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input.dtype)
        if bias is not None:
            output = output + bias
    return output.to(dtype=input.dtype).view(*output_shape)


# Weight preparation at load time (plain torch; not timed).


def input_to_int8(x: torch.Tensor, dtype: torch.dtype = torch.int8):
    """Per-tensor INT8 quantization in torch (int8_utils.py:34-44): amax clamped at 1e-12,
    q = clamp(x * (127 / amax)) converted to `dtype` (the conversion truncates toward zero);
    returns q and 1 / (127 / amax)."""
    info = torch.iinfo(dtype)
    lo, hi = x.aminmax()
    amax = torch.maximum(lo.abs(), hi.abs()).clamp(min=1e-12)
    scale = info.max / amax
    q = (x * scale).clamp(min=info.min, max=info.max).to(dtype).contiguous()
    return q, scale.float().reciprocal()


def block_dequant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size: List[int]) -> torch.Tensor:
    """Block-quantized [n, k] codes times their block scales, fp32 (int8_utils.py:47-73)."""
    n, k = x_q_block.shape
    assert x_s.shape[0] == (n + block_size[0] - 1) // block_size[0]
    assert x_s.shape[1] == (k + block_size[1] - 1) // block_size[1]
    expanded = x_s.repeat_interleave(block_size[0], dim=0).repeat_interleave(block_size[1], dim=1)[:n, :k]
    return x_q_block.to(torch.float32) * expanded
