"""Linear-layer glue of the FP8 paths: view to 2-D, quantize, GEMM, bias, reshape
(python/sglang/srt/layers/quantization/fp8_utils.py:182-212 and :539-778)."""

from __future__ import annotations

import os
from typing import List, Optional

import torch

from ..sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm
from ..sgl_kernel.gemm import block_fp8_linear, fp8_blockwise_scaled_mm_bias, fp8_linear
from .fp8_kernel import (
    per_token_group_quant_fp8,
    per_token_group_quant_fp8_pow2,
    w8a8_block_fp8_matmul_deepgemm,
    scaled_fp8_quant,
    sglang_per_token_quant_fp8,
    static_quant_fp8,
    w8a8_block_fp8_matmul,
)


# Rows up to which w8a8_block_fp8_linear hands quantization and GEMM to one operator: the single
# fused decode kernel is chosen for up to 4 rows (measured; beyond that two launches are faster).
FUSED_QUANT_MAX_ROWS = 4
# ... and up to which apply_fp8_linear's dynamic per-token branch does (sglq_w8a8_fp8_linear: every block of
# the fused kernel reads the rows once more for their maxima, which pays for one or two rows)
FUSED_TOKEN_QUANT_MAX_ROWS = 2


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
    fusable_bias = bias is None or (bias.dtype == input_2d.dtype and bias.is_contiguous() and bias.numel() == weight.shape[0])
    if (input_2d.shape[0] <= FUSED_QUANT_MAX_ROWS and fusable_bias and input_2d.dtype in (torch.bfloat16, torch.float16)
            and input_2d.is_contiguous() and weight.shape[1] % 128 == 0 and weight.is_contiguous()):
        # decode-sized batches: quantization and GEMM (and bias) as one operator, a single kernel on the
        # shapes of the decode kernel without split-K; bit-identical to the calls below
        return block_fp8_linear(input_2d, weight.T, weight_scale.T, bias).view(*output_shape)
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
    input_scale_ub: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    cutlass_fp8_supported: bool = True,
    use_per_token_if_dynamic: bool = False,
    pad_output: Optional[bool] = None,
    compressed_tensor_quant: bool = False,
) -> torch.Tensor:
    """FP8 linear with per-token or per-tensor activation scales and per-channel or per-tensor
    weight scales: apply_fp8_linear (fp8_utils.py:539-778), same parameters in the same order,
    every branch ending in this library's fp8_scaled_mm.

    weight is the [K, N] transposed view of the stored [N, K] codes; weight_scale has one fp32
    per output channel ([N, 1] or [N]) or a single element.

    * default branch (:684-733): a static `input_scale` quantizes through static_quant_fp8 with
      the scale repeated per token; otherwise the activations are quantized per token.
    * `compressed_tensor_quant` (:567-596): scaled_fp8_quant(input, input_scale,
      use_per_token_if_dynamic=...), i.e. static per-tensor, dynamic per-tensor or dynamic
      per-token activation scales.
    * A per-tensor activation scale is repeated per token and a per-tensor weight scale per
      channel before the GEMM, which takes [M] and [N] scales; the reference sends those cases
      to torch._scaled_mm (:644-655,735-748), whose result is the same product.
    * `input_scale_ub` is accepted and unused, as in the reference's body.  `pad_output` only
      pads rows for torch._scaled_mm there and has no effect here.  `cutlass_fp8_supported`
      chooses between the sgl_kernel GEMM and torch._scaled_mm in the reference; this library has
      one GEMM and uses it for either value."""
    del input_scale_ub, pad_output, cutlass_fp8_supported
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[1]]
    if compressed_tensor_quant:
        qinput, x_scale = scaled_fp8_quant(input_2d.contiguous(), input_scale, use_per_token_if_dynamic=use_per_token_if_dynamic)
    elif input_scale is not None:
        # static per-tensor activation scale, broadcast to one scale per token because the GEMM
        # takes per-token scales (fp8_utils.py:684-689)
        assert input_scale.numel() == 1
        qinput, x_scale = static_quant_fp8(input_2d.contiguous(), input_scale, repeat_scale=True)
    else:
        rows = input_2d.shape[0]
        if (0 < rows <= FUSED_TOKEN_QUANT_MAX_ROWS and input.is_cuda and input.dtype in (torch.bfloat16, torch.float16)
                and input_2d.shape[1] % 128 == 0 and weight.stride(0) == 1 and weight_scale.numel() == weight.shape[1] and weight.shape[1] > 1):
            # decode rows: quantization and GEMM in one operator (a single kernel on the decode kernel's shapes),
            # bit-identical to the two calls below
            ws = weight_scale if weight_scale.dtype == torch.float32 and weight_scale.is_contiguous() else weight_scale.to(torch.float32).contiguous()
            return fp8_linear(input_2d.contiguous(), weight, ws, bias).view(*output_shape)
        qinput, x_scale = sglang_per_token_quant_fp8(input_2d.contiguous())
    m, n = qinput.shape[0], weight.shape[1]
    if x_scale.numel() == 1 and m != 1:
        x_scale = x_scale.reshape(1, 1).expand(m, 1).contiguous()
    if weight_scale.numel() == 1 and n != 1:
        weight_scale = weight_scale.to(torch.float32).reshape(1, 1).expand(n, 1).contiguous()
    assert weight_scale.numel() == n, "fp8_scaled_mm takes one weight scale per output channel (or a single one)"
    output = fp8_scaled_mm(qinput, weight, x_scale, weight_scale, out_dtype=input.dtype, bias=bias)
    return output.view(*output_shape)


# ---------------------------------------------------------------------------------------------
# The names the reference's linear methods import for this path (fp8_utils.py:79-147,182-258).

cutlass_w8a8_block_fp8_linear_with_fallback = w8a8_block_fp8_linear


# The reference's deep_gemm_wrapper.DEEPGEMM_SCALE_UE8M0 (true on the hardware whose DeepGEMM wants power-of-two
# scales): when set, deepgemm_w8a8_block_fp8_linear_with_fallback quantizes with power-of-two scales and runs the
# GEMM whose matrix instructions apply them; the weights must then have been through requant_weight_ue8m0_inplace,
# as the reference's loaders do under that flag.  Off by default (SGLANG_AMD_SCALE_UE8M0=1 or assignment turns it on).
DEEPGEMM_SCALE_UE8M0 = os.environ.get("SGLANG_AMD_SCALE_UE8M0", "0").lower() in ("1", "true", "yes")


def deepgemm_w8a8_block_fp8_linear_with_fallback(
    input: torch.Tensor,
    weight: torch.Tensor,
    block_size: List[int],
    weight_scale: torch.Tensor,
    input_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The call sequence of deepgemm_w8a8_block_fp8_linear_with_fallback (fp8_utils.py:215-258): column-major
    activation scales, the GEMM that is DeepGEMM's there, `output += bias`; outputs other than bfloat16 and
    weights whose N is not a multiple of 64 take the row-major path, as in the reference (:227-234).
    With DEEPGEMM_SCALE_UE8M0 (:245): power-of-two activation scales (kept as fp32 rather than packed four
    to an int32: per_token_group_quant_fp8_pow2) and w8a8_block_fp8_matmul_deepgemm, which lets the matrix
    instructions apply the scales; the weight's block scales must be powers of two (requant_weight_ue8m0_inplace).
    Without: fp32 scales with the row count padded to a multiple of four (`scale_tma_aligned=True`) and this
    library's block-scaled kernel, which takes the scales' strides as they are."""
    assert input_scale is None
    if not (input.dtype == torch.bfloat16 and weight.shape[0] % 64 == 0 and weight.shape[1] % 128 == 0):
        return triton_w8a8_block_fp8_linear(input, weight, block_size, weight_scale, input_scale, bias)
    input_2d = input.view(-1, input.shape[-1])
    output_shape = [*input.shape[:-1], weight.shape[0]]
    if DEEPGEMM_SCALE_UE8M0:
        q_input, x_scale = per_token_group_quant_fp8_pow2(input_2d, block_size[1], column_major_scales=True)
        output = w8a8_block_fp8_matmul_deepgemm(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input.dtype)
    else:
        q_input, x_scale = per_token_group_quant_fp8(input_2d, block_size[1], column_major_scales=True, scale_tma_aligned=True)
        output = w8a8_block_fp8_matmul(q_input, weight, x_scale, weight_scale, block_size, output_dtype=input.dtype)
    if bias is not None:
        output += bias
    return output.to(dtype=input.dtype).view(*output_shape)


def cutlass_fp8_supported() -> bool:
    """True where fp8_scaled_mm can run (fp8_utils.py:79-88 asks for an SM89+ CUDA build): here,
    where the HIP library loads and a GPU is present."""
    from .. import _lib

    try:
        _lib.load()
    except Exception:
        return False
    return torch.cuda.is_available()


def cutlass_block_fp8_supported() -> bool:
    """True where fp8_blockwise_scaled_mm can run (fp8_utils.py:115-128).  The reference also
    wants SGLANG_SUPPORT_CUTLASS_BLOCK_FP8 set; this library has no slower path to prefer."""
    return cutlass_fp8_supported()


def dispatch_w8a8_block_fp8_linear():
    """The block-FP8 linear the layers call (fp8_utils.py:137-147)."""
    return cutlass_w8a8_block_fp8_linear_with_fallback


# ---------------------------------------------------------------------------------------------
# Weight preparation at load time (plain torch on whatever device the weights are on; not timed).


def input_to_float8(x: torch.Tensor, dtype: torch.dtype = torch.float8_e4m3fn):
    """Per-tensor quantization in torch (fp8_utils.py:339-355): amax clamped at 1e-12,
    q = clamp(x * (fp_max / amax)) rounded to `dtype`; returns q and 1 / (fp_max / amax)."""
    fp_max = torch.finfo(dtype).max
    lo, hi = x.aminmax()
    amax = torch.maximum(lo.abs(), hi.abs()).float().clamp(min=1e-12)
    scale = fp_max / amax
    q = (x.float() * scale).clamp(min=-fp_max, max=fp_max).to(dtype).contiguous()
    return q, scale.float().reciprocal()


def _expand_block_scales(x_s: torch.Tensor, block_size: List[int], n: int, k: int) -> torch.Tensor:
    return x_s.repeat_interleave(block_size[0], dim=-2).repeat_interleave(block_size[1], dim=-1)[..., :n, :k]


def block_quant_dequant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size: List[int], dtype: torch.dtype) -> torch.Tensor:
    """Block-quantized weight [..., n, k] with scales [..., ceil(n/bn), ceil(k/bk)] back to `dtype`
    (fp8_utils.py:401-421)."""
    *_, n, k = x_q_block.shape
    return (x_q_block.to(torch.float32) * _expand_block_scales(x_s, block_size, n, k)).to(dtype)


def _tensor_quant_fp8(x: torch.Tensor, dtype: torch.dtype):
    # the reference quantizes with its CUDA operator where it has one and in torch elsewhere
    # (fp8_utils.py:392-396); the operator here is scaled_fp8_quant on GPU tensors
    if x.is_cuda:
        from .fp8_kernel import scaled_fp8_quant

        return scaled_fp8_quant(x)
    return input_to_float8(x, dtype=dtype)


def block_quant_to_tensor_quant(x_q_block: torch.Tensor, x_s: torch.Tensor, block_size: List[int]):
    """Block-wise FP8 quantization re-quantized with one scale for the tensor (fp8_utils.py:358-398)."""
    n, k = x_q_block.shape
    assert x_s.shape[0] == (n + block_size[0] - 1) // block_size[0]
    assert x_s.shape[1] == (k + block_size[1] - 1) // block_size[1]
    return _tensor_quant_fp8(block_quant_dequant(x_q_block, x_s, block_size, torch.float32), x_q_block.dtype)


def channel_quant_to_tensor_quant(x_q_channel: torch.Tensor, x_s: torch.Tensor):
    """Per-channel FP8 quantization re-quantized with one scale for the tensor (fp8_utils.py:489-499)."""
    return _tensor_quant_fp8(x_q_channel.to(torch.float32) * x_s, x_q_channel.dtype)


def ceil_to_ue8m0(x: torch.Tensor) -> torch.Tensor:
    """The next power of two at or above abs(x) (fp8_utils.py:485-486)."""
    return torch.pow(2.0, torch.ceil(torch.log2(x.abs())))


def _requant_weight_ue8m0(weight: torch.Tensor, weight_scale_inv: torch.Tensor, weight_block_size: List[int]):
    """fp8_utils.py:432-463 up to the scale layout: the weight dequantized to bf16 and block-quantized again with
    power-of-two scales.  The scales stay fp32 [N/128, K/128] (the reference goes on to expand and pack them into
    DeepGEMM's column-major int32 layout, :453-461, which the GEMM here does not use)."""
    assert list(weight_block_size) == [128, 128]
    *_, n, k = weight.shape
    dequant = block_quant_dequant(weight, weight_scale_inv, weight_block_size, torch.bfloat16)
    out_w, out_s = per_block_cast_to_fp8(dequant.view((-1, k)))
    return out_w.view(weight.shape), out_s.view(weight_scale_inv.shape)


def requant_weight_ue8m0_inplace(weight, weight_scale_inv, weight_block_size):
    """fp8_utils.py:424-429."""
    assert isinstance(weight, torch.nn.Parameter)
    assert isinstance(weight_scale_inv, torch.nn.Parameter)
    weight.data, weight_scale_inv.data = _requant_weight_ue8m0(weight, weight_scale_inv, weight_block_size)


def per_block_cast_to_fp8(x: torch.Tensor):
    """128 x 128 block quantization of a 2-D weight with power-of-two scales (fp8_utils.py:468-481):
    block amax clamped at 1e-4, scale = ceil_to_ue8m0(amax / 448), q = x * (1 / scale)."""
    assert x.dim() == 2
    m, n = x.shape
    mp, np_ = (m + 127) // 128 * 128, (n + 127) // 128 * 128
    padded = torch.zeros((mp, np_), dtype=x.dtype, device=x.device)
    padded[:m, :n] = x
    blocks = padded.view(mp // 128, 128, np_ // 128, 128)
    amax = blocks.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = ceil_to_ue8m0(amax / 448.0)
    q = (blocks * (1.0 / sf)).to(torch.float8_e4m3fn)
    return q.view(mp, np_)[:m, :n].contiguous(), sf.view(mp // 128, np_ // 128)
