"""Grouped (MoE) block-scaled FP8 GEMM behind the reference's operator name and argument list
(sgl-kernel/python/sgl_kernel/moe.py:131-170, checks of
sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:606-641)."""

from __future__ import annotations

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
