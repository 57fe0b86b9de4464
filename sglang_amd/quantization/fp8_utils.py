"""Linear-layer glue of the FP8 paths: view to 2-D, quantize, GEMM, bias, reshape
(python/sglang/srt/layers/quantization/fp8_utils.py:182-212 and :539-778)."""

from __future__ import annotations

from typing import List, Optional

import torch

from ..sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm
from ..sgl_kernel.gemm import fp8_blockwise_scaled_mm_bias
from .fp8_kernel import per_token_group_quant_fp8, sglang_per_token_quant_fp8, static_quant_fp8, w8a8_block_fp8_matmul


def w8a8_block_fp8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    block_size: List[int],
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Block-FP8 linear: the call sequence of
    cutlass_w8a8_block_fp8_linear_with_fallback (fp8_utils.py:182-212).

    weight [N, K] e4m3fn, weight_scale [ceil(N/128), ceil(K/128)] fp32.  Shapes
    with N or K not a multiple of 128 run on the same kernel (the reference
    diverts them to its Triton kernel, :193-199)."""
    assert input_scale is None
    assert list(block_size) == [128, 128], "only 128x128 weight blocks are built"
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    q_input, x_scale = per_token_group_quant_fp8(input_2d, block_size[1], column_major_scales=True)
    if bias is not None and bias.dtype == input_2d.dtype and bias.is_contiguous() and bias.numel() == weight.shape[0]:
        # the GEMM and `output += bias` (fp8_utils.py:207-211) in one kernel, same two roundings
        output = fp8_blockwise_scaled_mm_bias(q_input, weight.T, x_scale, weight_scale.T, input_2d.dtype, bias)
    else:
        output = fp8_blockwise_scaled_mm(q_input, weight.T, x_scale, weight_scale.T, out_dtype=input_2d.dtype)
        if bias is not None:
            output += bias
    return output.to(dtype=input_2d.dtype).view(*output_shape)


def triton_w8a8_block_fp8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    block_size: List[int],
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The call sequence of triton_w8a8_block_fp8_linear (fp8_utils.py:289-309): row-major
    activation scales, the weight and its scales as stored, any N and K."""
    assert input_scale is None
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    q_input, x_scale = per_token_group_quant_fp8(input_2d, block_size[1], column_major_scales=False)
    if bias is not None and bias.dtype == input_2d.dtype and bias.is_contiguous() and bias.numel() == weight.shape[0]:
        output = w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input_2d.dtype, bias=bias)
    else:
        output = w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input_2d.dtype)
        if bias is not None:
            output += bias
    return output.to(dtype=input_2d.dtype).view(*output_shape)


def apply_fp8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Per-token activation / per-channel weight FP8 linear: the dynamic branch of
    apply_fp8_linear that ends in fp8_scaled_mm (fp8_utils.py:693,720-733).

    weight is the [K, N] transposed view, weight_scale one fp32 per output channel."""
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[1]]
    if input_scale is not None:
        # static per-tensor activation scale, broadcast to one scale per token because the GEMM
        # takes per-token scales (fp8_utils.py:684-689)
        assert input_scale.numel() == 1
        qinput, x_scale = static_quant_fp8(input_2d.contiguous(), input_scale, repeat_scale=True)
    else:
        qinput, x_scale = sglang_per_token_quant_fp8(input_2d)
    assert weight_scale.numel() == weight.shape[1], "cutlass w8a8 fp8 sgl-kernel only supports per-channel scale"
    output = fp8_scaled_mm(qinput, weight, x_scale, weight_scale, out_dtype=input.dtype, bias=bias)
    return output.view(*output_shape)
