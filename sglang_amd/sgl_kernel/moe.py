"""Grouped (MoE) block-scaled FP8 GEMM and the data-movement operators around it, behind the
reference's operator names and argument lists (sgl-kernel/python/sgl_kernel/moe.py:131-205,
sgl-kernel/python/sgl_kernel/gemm.py:281-288, sgl-kernel/python/sgl_kernel/elementwise.py:171-183;
checks of sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:606-641 and
sgl-kernel/csrc/moe/prepare_moe_input.cu)."""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from .._lib import DTYPE_CODE

FP8 = torch.float8_e4m3fn


def _check(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def fp8_blockwise_scaled_grouped_mm(
    output,
    a_ptrs,
    b_ptrs,
    out_ptrs,
    a_scales_ptrs,
    b_scales_ptrs,
    a,
    b,
    scales_a,
    scales_b,
    stride_a,
    stride_b,
    stride_c,
    layout_sfa,
    layout_sfb,
    problem_sizes,
    expert_offsets,
    workspace,
):
    """output[rows of expert e] = a[rows of expert e] @ b[e], block-scaled, for every expert.

    a [total_m, K] e4m3fn row-major; b [E, K, N] e4m3fn with every b[e] column-major (the
    transposed view of the [E, N, K] weight); scales_a [total_m, K/128] fp32 row-major (the
    reference's K-major convention, fp8_blockwise_moe_kernel.cu:96-97, i.e. what
    sglang_per_token_group_quant_fp8 and shuffle_rows produce, cutlass_moe.py:156-158, without
    per_group_transpose); scales_b [E, K/128, N/128] fp32 with any strides; problem_sizes
    [E, 3] int32 rows (M_e, N, K) and expert_offsets [E] int32 on the device.

    The pointer arrays (a_ptrs ... b_scales_ptrs), stride_a/b/c and layout_sfa/sfb are the
    scratch that the reference's pre-kernel fills for CUTLASS (fp8_blockwise_moe_kernel.cu:56-77);
    this implementation plans its tiles from problem_sizes and expert_offsets and leaves them
    untouched.  `workspace` receives the tile plan."""
    _check(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor")
    _check(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)")
    _check(problem_sizes.size(0) == expert_offsets.size(0), "Number of experts in problem_sizes must match expert_offsets")
    _check(problem_sizes.dtype == torch.int32, "problem_sizes must be int32")
    _check(a.dtype == FP8, "a must be kFloat8_e4m3fn")
    _check(b.dtype == FP8, "b must be kFloat8_e4m3fn")
    _check(output.dtype in (torch.bfloat16, torch.half), "output must be bfloat16 or half")
    _check(scales_a.dtype == torch.float32, "scales_a must be float32")
    _check(scales_b.dtype == torch.float32, "scales_b must be float32")
    _check(expert_offsets.dtype == torch.int32, "expert_offsets must be int32")
    _check(output.dim() == 2, "output must be 2D tensor")
    _check(a.dim() == 2, "a must be 2D tensor")
    _check(b.dim() == 3, "b must be 3D tensor")
    _check(scales_a.dim() == 2, "scales_a must be 2D tensor")
    _check(scales_b.dim() == 3, "scales_b must be 3D tensor")
    _check(expert_offsets.dim() == 1, "expert_offsets must be 1D tensor")
    _check(workspace.dim() == 1, "workspace must be 1D tensor")
    for name, t in (("output", output), ("a", a), ("b", b), ("scales_a", scales_a), ("scales_b", scales_b),
                    ("problem_sizes", problem_sizes), ("expert_offsets", expert_offsets), ("workspace", workspace)):
        _check(t.is_cuda, f"{name} must be a CUDA tensor")
    num_experts, k, n = b.shape
    total_m = a.size(0)
    _check(a.size(1) == k, "a and b shapes cannot be multiplied")
    _check(problem_sizes.size(0) == num_experts, "problem_sizes must have one row per expert of b")
    _check(tuple(output.shape) == (total_m, n), "output must have shape (a.size(0), b.size(2))")
    _check(problem_sizes.is_contiguous() and expert_offsets.is_contiguous(), "problem_sizes and expert_offsets must be contiguous")
    _check(total_m <= 1 or a.stride(1) == 1, "a must be a row major tensor")
    _check(num_experts == 0 or k <= 1 or b.stride(1) == 1, "every b[e] must be a column major tensor")
    _check(n <= 1 or output.stride(1) == 1, "output must be a row major tensor")
    kb, nb = (k + 127) // 128, (n + 127) // 128
    _check(tuple(scales_a.shape) == (total_m, kb), "scales_a must have shape (a.size(0), ceil(K / 128))")
    _check(tuple(scales_b.shape) == (num_experts, kb, nb), "scales_b must have shape (E, ceil(K / 128), ceil(N / 128))")
    if total_m == 0 or n == 0 or num_experts == 0:
        return
    lib = _lib.load()
    rc = lib.sglq_fp8_blockwise_scaled_grouped_mm(
        a.data_ptr(), a.stride(0) if total_m > 1 else k,
        b.data_ptr(), b.stride(2) if n > 1 else k, b.stride(0) if num_experts > 1 else n * k,
        scales_a.data_ptr(), scales_a.stride(0), scales_a.stride(1),
        scales_b.data_ptr(), scales_b.stride(0), scales_b.stride(1), scales_b.stride(2),
        output.data_ptr(), output.stride(0), DTYPE_CODE[output.dtype],
        problem_sizes.data_ptr(), expert_offsets.data_ptr(), num_experts, total_m, n, k,
        workspace.data_ptr(), workspace.numel() * workspace.element_size(), _lib.stream_ptr(a.device))
    _lib.check(rc, "fp8_blockwise_scaled_grouped_mm")


def _cuda_int32(name, t):
    _check(t.is_cuda, f"{name} must be a CUDA tensor")
    _check(t.dtype == torch.int32, f"{name} must be int32")
    _check(t.is_contiguous(), f"{name} must be contiguous")


def prepare_moe_input(
    topk_ids,
    expert_offsets,
    problem_sizes1,
    problem_sizes2,
    input_permutation,
    output_permutation,
    num_experts,
    n,
    k,
    blockscale_offsets: Optional[torch.Tensor] = None,
):
    """Routing tables from the top-k expert ids (sgl-kernel/python/sgl_kernel/moe.py:173-196):
    fills expert_offsets [E + 1], problem_sizes1/2 [E, 3], input_permutation (a_map) and
    output_permutation (c_map), both [m * topk], and blockscale_offsets [E + 1] if given."""
    _check(topk_ids.dtype == torch.int32, "topk_ids must be int32")  # prepare_moe_input.cu:153
    for name, t in (("topk_ids", topk_ids), ("expert_offsets", expert_offsets), ("problem_sizes1", problem_sizes1),
                    ("problem_sizes2", problem_sizes2), ("input_permutation", input_permutation),
                    ("output_permutation", output_permutation)):
        _cuda_int32(name, t)
    _check(topk_ids.dim() == 2, "topk_ids must be a [num_tokens, topk] tensor")
    _check(expert_offsets.numel() >= num_experts + 1, "expert_offsets must hold num_experts + 1 entries")
    _check(problem_sizes1.numel() >= 3 * num_experts and problem_sizes2.numel() >= 3 * num_experts,
           "problem_sizes must have shape (num_experts, 3)")
    _check(input_permutation.numel() >= topk_ids.numel() and output_permutation.numel() >= topk_ids.numel(),
           "the permutations must hold one entry per element of topk_ids")
    if blockscale_offsets is not None:
        _cuda_int32("blockscale_offsets", blockscale_offsets)
        _check(blockscale_offsets.numel() >= num_experts + 1, "blockscale_offsets must hold num_experts + 1 entries")
    rc = _lib.load().sglq_prepare_moe_input(
        topk_ids.data_ptr(), expert_offsets.data_ptr(), None if blockscale_offsets is None else blockscale_offsets.data_ptr(),
        problem_sizes1.data_ptr(), problem_sizes2.data_ptr(), input_permutation.data_ptr(), output_permutation.data_ptr(),
        topk_ids.numel(), max(topk_ids.size(1), 1), int(num_experts), int(n), int(k), _lib.stream_ptr(topk_ids.device))
    _lib.check(rc, "prepare_moe_input")


def shuffle_rows(input_tensor, dst2src_map, output_tensor_shape):
    """output[d] = input[dst2src_map[d]] (sgl-kernel/python/sgl_kernel/gemm.py:281-288)."""
    _check(input_tensor.is_cuda and dst2src_map.is_cuda, "input and dst2src_map must be CUDA tensors")
    _check(input_tensor.dim() == 2 and input_tensor.is_contiguous(), "input must be a contiguous 2D tensor")
    _check(dst2src_map.dtype == torch.int32 and dst2src_map.is_contiguous(), "dst2src_map must be a contiguous int32 tensor")
    output_tensor = torch.empty(output_tensor_shape, device=input_tensor.device, dtype=input_tensor.dtype)
    _check(output_tensor.dim() == 2 and output_tensor.size(1) == input_tensor.size(1), "output rows must have the input's length")
    _check(dst2src_map.numel() >= output_tensor.size(0), "dst2src_map must hold one entry per output row")
    rc = _lib.load().sglq_shuffle_rows(
        input_tensor.data_ptr(), dst2src_map.data_ptr(), output_tensor.data_ptr(), input_tensor.size(0), output_tensor.size(0),
        input_tensor.size(1) * input_tensor.element_size(), _lib.stream_ptr(input_tensor.device))
    _lib.check(rc, "shuffle_rows")
    return output_tensor


def apply_shuffle_mul_sum(input, output, permutation, factors):
    """output[i] = sum_j factors[i, j] * input[permutation[i * topk + j]]
    (sgl-kernel/python/sgl_kernel/moe.py:199-207; checks of prepare_moe_input.cu:320-345)."""
    _check(input.dim() == 2, "input_tensor must be 2D [m * topk, row_stride]")
    _check(output.dim() == 2, "output_tensor must be 2D [m, row_stride]")
    _check(permutation.dim() == 1, "permutation must be 1D [m * topk]")
    _check(input.is_cuda and output.is_cuda and permutation.is_cuda, "tensors must be CUDA tensors")
    _check(input.is_contiguous() and output.is_contiguous() and permutation.is_contiguous(), "tensors must be contiguous")
    _check(output.dtype in (torch.bfloat16, torch.float16) and input.dtype == output.dtype, "input and output must be Half or BFloat16")
    _check(permutation.dtype == torch.int32, "permutation must be int32")
    m, row = output.shape
    _check(input.size(1) == row, "input and output rows must have the same length")
    if m == 0:
        return
    topk = permutation.size(0) // m
    _check(permutation.size(0) == m * topk and topk > 0, "permutation size must match m * topk")
    f_ptr = None
    if factors is not None:
        _check(factors.dtype == output.dtype, "Factors must match output dtype")
        _check(factors.numel() == m * topk, "Factors must have shape [m * topk]")
        _check(factors.is_cuda and factors.is_contiguous(), "factors must be a contiguous CUDA tensor")
        f_ptr = factors.data_ptr()
    rc = _lib.load().sglq_apply_shuffle_mul_sum(
        input.data_ptr(), output.data_ptr(), permutation.data_ptr(), f_ptr, DTYPE_CODE[output.dtype], m, topk, row, input.size(0),
        _lib.stream_ptr(input.device))
    _lib.check(rc, "apply_shuffle_mul_sum")


def silu_and_mul(input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """out = silu(input[..., :d]) * input[..., d:] (sgl-kernel/python/sgl_kernel/elementwise.py:171-183)."""
    if input.shape[-1] * input.element_size() % 16 != 0:
        raise ValueError("The pointers must be multiple of 16 bytes.")
    d = input.shape[-1] // 2
    if out is not None:
        assert input.ndim == out.ndim and input.shape[:-1] == out.shape[:-1] and input.shape[-1] == 2 * out.shape[-1]
    else:
        out = torch.empty(input.shape[:-1] + (d,), device=input.device, dtype=input.dtype)
    _check(input.is_cuda and out.is_cuda, "input and out must be CUDA tensors")
    _check(input.is_contiguous() and out.is_contiguous(), "input and out must be contiguous")
    if input.dtype not in (torch.bfloat16, torch.float16) or out.dtype != input.dtype:
        raise NotImplementedError("silu_and_mul: Half and BFloat16 are built")
    tokens = input.numel() // input.shape[-1] if input.numel() else 0
    rc = _lib.load().sglq_silu_and_mul(input.data_ptr(), DTYPE_CODE[input.dtype], out.data_ptr(), tokens, d, _lib.stream_ptr(input.device))
    _lib.check(rc, "silu_and_mul")
    return out


def silu_and_mul_per_token_group_quant_fp8(input: torch.Tensor, group_size: int = 128, eps: float = 1e-10):
    """silu_and_mul(input) followed by sglang_per_token_group_quant_fp8(., 128) in one kernel
    (the two calls of python/sglang/srt/layers/moe/cutlass_moe.py:187-194); the intermediate
    is not materialised.  input [..., 2 d] Half / BFloat16, d a multiple of 128; returns
    (codes [..., d] e4m3fn, scales [..., d / 128] fp32 row-major), bit-identical to the two calls."""
    if group_size != 128:
        raise NotImplementedError("silu_and_mul_per_token_group_quant_fp8: group size 128 is built")
    _check(input.is_cuda and input.is_contiguous(), "input must be a contiguous CUDA tensor")
    if input.dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError("silu_and_mul_per_token_group_quant_fp8: Half and BFloat16 are built")
    d = input.shape[-1] // 2
    _check(input.shape[-1] == 2 * d and d % 128 == 0, "the last dimension must be 2 d with d a multiple of 128")
    out_q = torch.empty(input.shape[:-1] + (d,), device=input.device, dtype=FP8)
    out_s = torch.empty(input.shape[:-1] + (d // 128,), device=input.device, dtype=torch.float32)
    tokens = input.numel() // input.shape[-1] if input.numel() else 0
    rc = _lib.load().sglq_silu_and_mul_group_quant_fp8(input.data_ptr(), DTYPE_CODE[input.dtype], out_q.data_ptr(), out_s.data_ptr(),
                                                       tokens, d, eps, _lib.stream_ptr(input.device))
    _lib.check(rc, "silu_and_mul_per_token_group_quant_fp8")
    return out_q, out_s


def per_token_group_quant_fp8_to_expert_rows(x: torch.Tensor, slot_map: torch.Tensor, topk: int, group_size: int = 128,
                                             eps: float = 1e-10):
    """sglang_per_token_group_quant_fp8(x, 128) followed by shuffle_rows of codes and scales with
    a_map (python/sglang/srt/layers/moe/cutlass_moe.py:156-158) in one kernel: token t is quantized
    once and written to the rows slot_map[t * topk + j], j < topk (slot_map = prepare_moe_input's
    output_permutation; entries outside [0, m * topk) are skipped and rows that no slot names stay
    uninitialised).  x [m, k] Half / BFloat16 / Float; returns (codes [m * topk, k] e4m3fn, scales
    [m * topk, k / 128] fp32 row-major), bit-identical to the three calls on every row a slot names."""
    if group_size != 128:
        raise NotImplementedError("per_token_group_quant_fp8_to_expert_rows: group size 128 is built")
    _check(x.is_cuda and x.dim() == 2 and x.is_contiguous(), "x must be a contiguous 2D CUDA tensor")
    _check(x.dtype in DTYPE_CODE, "x must be Float, Half or BFloat16")
    _check(x.size(1) % 128 == 0, "the last dimension must be divisible by group_size")
    _cuda_int32("slot_map", slot_map)
    m, k = x.shape
    _check(topk > 0 and slot_map.numel() >= m * topk, "slot_map must hold m * topk entries")
    out_q = torch.empty((m * topk, k), device=x.device, dtype=FP8)
    out_s = torch.empty((m * topk, k // 128), device=x.device, dtype=torch.float32)
    rc = _lib.load().sglq_per_token_group_quant_fp8_scatter(x.data_ptr(), DTYPE_CODE[x.dtype], out_q.data_ptr(), out_s.data_ptr(),
                                                            slot_map.data_ptr(), m, k, int(topk), m * topk, eps,
                                                            _lib.stream_ptr(x.device))
    _lib.check(rc, "per_token_group_quant_fp8_to_expert_rows")
    return out_q, out_s
