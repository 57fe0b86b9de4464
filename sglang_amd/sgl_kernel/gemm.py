"""Operators of the W8A8 path under their ``sgl_kernel`` names and signatures
(sgl-kernel/python/sgl_kernel/gemm.py:13-42,100-145).

Each public function forwards positionally to ``torch.ops.sgl_kernel.<op>``,
as the reference wrappers do; the op implementations registered here validate
their arguments the way the reference's C++ entry points do (same conditions,
``RuntimeError`` on violation), allocate the output with torch and enqueue the
HIP kernel on the current stream through the C ABI.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _lib
from .._lib import DTYPE_CODE

FP8 = torch.float8_e4m3fn


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


# ---------------------------------------------------------------------------
# argument validation (device-independent so that it can be exercised on CPU tensors)
# ---------------------------------------------------------------------------
def check_mm_common(mat_a, mat_b, out_dtype, elem_dtype, elem_name, require_cuda=True):
    """Checks shared by the three GEMM entry points
    (int8_gemm_kernel.cu:670-683, fp8_gemm_kernel.cu:1078-1094,
    fp8_blockwise_gemm_kernel.cu:351-365)."""
    if require_cuda:
        _check(mat_a.is_cuda, "mat_a must be a CUDA tensor")
        _check(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _check(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _check(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _check(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _check(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _check(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _check((mat_a.size(1) * mat_a.element_size()) % 16 == 0, "mat_a must be multiple of 16 bytes for memory alignment")
    _check((mat_b.size(0) * mat_b.element_size()) % 16 == 0, "mat_b must be multiple of 16 bytes for memory alignment")
    _check(mat_a.dtype == elem_dtype, f"mat_a must be {elem_name}")
    _check(mat_b.dtype == elem_dtype, f"mat_b must be {elem_name}")
    _check(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")
    # kernel-side requirements on strides that the reference leaves to its GEMM library
    _check(mat_a.size(0) <= 1 or mat_a.stride(0) % 16 == 0, "mat_a row stride must be a multiple of 16 bytes")
    _check(mat_b.size(1) <= 1 or mat_b.stride(1) % 16 == 0, "mat_b column stride must be a multiple of 16 bytes")


def check_rowcol_scales(mat_a, mat_b, scales_a, scales_b, out_dtype, bias):
    """int8_gemm_kernel.cu:685-696 / fp8_gemm_kernel.cu:1096-1105."""
    _check(scales_a.numel() == mat_a.size(0), "size of scales_a is not matched")
    _check(scales_b.numel() == mat_b.size(1), "size of scales_b is not matched")
    _check(scales_a.is_contiguous(), "scales_a must be contiguous")
    _check(scales_b.is_contiguous(), "scales_b msut be contiguous")
    _check(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _check(scales_b.dtype == torch.float32, "scales_b must be Float32")
    if bias is not None:
        _check(bias.numel() == mat_b.size(1), "size of bias is not matched")
        _check(bias.is_contiguous(), "bias must be contiguous")
        _check(bias.dtype == out_dtype, "bias dtype must match output dtype")


def _is_contiguous_vector(t: torch.Tensor) -> bool:
    return t.is_contiguous() and (t.dim() == 1 or (t.dim() == 2 and min(t.shape) == 1))


def check_blockwise_scales(mat_a, mat_b, scales_a, scales_b):
    """fp8_blockwise_gemm_kernel.cu:367-380.  Scale extents use ceil division so
    that N (or K) that is not a multiple of 128 is accepted with the scale shapes
    the callers allocate (fp8.py:276-306); for multiples of 128 this is the
    reference's condition."""
    m, k = mat_a.shape
    n = mat_b.size(1)
    _check(scales_a.dim() == 2 and scales_b.dim() == 2, "scales must be 2D tensors")
    _check(m == scales_a.size(0), "size of scales_a is not matched")
    _check((k + 127) // 128 == scales_a.size(1), "size of scales_a is not matched")
    _check(scales_a.stride(0) == 1 or _is_contiguous_vector(scales_a), "scales_a must be M major")
    _check((k + 127) // 128 == scales_b.size(0), "size of scales_b is not matched")
    _check((n + 127) // 128 == scales_b.size(1), "size of scales_b is not matched")
    _check(scales_b.stride(0) == 1 or _is_contiguous_vector(scales_b), "scales_b must be K major")
    _check(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _check(scales_b.dtype == torch.float32, "scales_b must be Float32")


def check_group_quant(input, output_q, output_s, group_size, q_dtype, require_cuda=True):
    """per_token_group_quant_8bit.cu:125-131 (+ CHECK_INPUT = CUDA and contiguous)."""
    for name, t in (("input", input), ("output_q", output_q)):
        if require_cuda:
            _check(t.is_cuda, f"{name} must be a CUDA tensor")
        _check(t.is_contiguous(), f"{name} must be contiguous")
    if require_cuda:
        _check(output_s.is_cuda, "output_s must be a CUDA tensor")
    _check(input.dtype in DTYPE_CODE, "input must be Float, Half or BFloat16")
    _check(output_q.dtype == q_dtype, f"output_q must be {q_dtype}")
    _check(output_q.shape == input.shape, "output_q must have the shape of input")
    _check(group_size > 0 and input.numel() % group_size == 0, "input.numel() must be divisible by group_size")
    _check(input.dim() >= 1 and input.shape[-1] % group_size == 0, "the last dimension must be divisible by group_size")
    _check(output_s.dim() == 2, "output_s must be a 2D tensor")
    _check(output_s.dtype == torch.float32, "output_s must be Float32")
    rows = input.numel() // input.shape[-1] if input.numel() else 0
    _check(tuple(output_s.shape) == (rows, input.shape[-1] // group_size), "output_s has the wrong shape")


def check_token_quant_fp8(input, output_q, output_s, require_cuda=True):
    """per_token_quant_fp8.cu:166-173."""
    for name, t in (("input", input), ("output_q", output_q), ("output_s", output_s)):
        if require_cuda:
            _check(t.is_cuda, f"{name} must be a CUDA tensor")
        _check(t.is_contiguous(), f"{name} must be contiguous")
    _check(input.dim() == 2, "input must be a 2D tensor")
    _check(input.dtype in DTYPE_CODE, "input must be Float, Half or BFloat16")
    _check(output_q.dtype == FP8 and output_q.shape == input.shape, "output_q must be Float8_e4m3fn with input's shape")
    _check(output_s.dtype == torch.float32 and output_s.numel() == input.size(0), "output_s must hold one Float32 per token")
    _check(input.size(1) % 8 == 0, f"Hidden dimension must be divisible by 8, but got {input.size(1)}")


def check_tensor_quant_fp8(input, output_q, output_s, require_cuda=True):
    """per_tensor_quant_fp8.cu:96-99 (CHECK_INPUT: CUDA and contiguous) plus what the kernels assume."""
    for name, t in (("input", input), ("output_q", output_q), ("output_s", output_s)):
        if require_cuda:
            _check(t.is_cuda, f"{name} must be a CUDA tensor")
        _check(t.is_contiguous(), f"{name} must be contiguous")
    _check(input.dtype in DTYPE_CODE, "input must be Float, Half or BFloat16")
    _check(output_q.dtype == FP8 and output_q.numel() == input.numel(), "output_q must be Float8_e4m3fn with input's element count")
    _check(output_s.dtype == torch.float32 and output_s.numel() >= 1, "output_s must hold one Float32")


# ---------------------------------------------------------------------------
# op implementations (CUDA dispatch key = ROCm device tensors)
# ---------------------------------------------------------------------------
def _int8_scaled_mm_impl(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    check_mm_common(mat_a, mat_b, out_dtype, torch.int8, "Int8")
    _check(mat_a.size(1) % 16 == 0, "mat_a.size(1) must be multiple of 16 for memory alignment")
    _check(mat_b.size(0) % 16 == 0, "mat_b.size(0) must be multiple of 16 for memory alignment")
    _check(mat_b.size(1) % 8 == 0, "mat_b.size(1) must be multiple of 8 for memory alignment")
    check_rowcol_scales(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)
    m, k = mat_a.shape
    n = mat_b.size(1)
    out = torch.empty((m, n), dtype=out_dtype, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_int8_scaled_mm(
        mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_a.data_ptr(), scales_b.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, *_lib.workspace(mat_a.device),
        _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "int8_scaled_mm")
    return out


def _fp8_scaled_mm_impl(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    check_mm_common(mat_a, mat_b, out_dtype, FP8, "Float8_e4m3fn")
    check_rowcol_scales(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)
    m, k = mat_a.shape
    n = mat_b.size(1)
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((m, n), dtype=out_dtype, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_fp8_scaled_mm(
        mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_a.data_ptr(), scales_b.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, *_lib.workspace(mat_a.device),
        _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "fp8_scaled_mm")
    return out


def _fp8_blockwise_scaled_mm_impl(mat_a, mat_b, scales_a, scales_b, out_dtype):
    check_mm_common(mat_a, mat_b, out_dtype, FP8, "Float8_e4m3fn")
    check_blockwise_scales(mat_a, mat_b, scales_a, scales_b)
    m, k = mat_a.shape
    n = mat_b.size(1)
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((m, n), dtype=out_dtype, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_fp8_blockwise_scaled_mm(
        mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_a.data_ptr(), scales_a.stride(0), scales_a.stride(1),
        scales_b.data_ptr(), scales_b.stride(0), scales_b.stride(1),
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, *_lib.workspace(mat_a.device),
        _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "fp8_blockwise_scaled_mm")
    return out


def fp8_blockwise_scaled_mm_ue8m0(mat_a, mat_b, scales_a, scales_b, out_dtype):
    """fp8_blockwise_scaled_mm for scales that are all powers of two (UE8M0 values as fp32, what
    ceil_to_ue8m0 of fp8_utils.py:485-486 produces): same arguments and result.  For bf16 outputs of more
    than 128 rows the matrix instruction applies the scales itself and accumulates in place, reading only
    their exponent bits; the caller guarantees that they are powers of two.  No counterpart among the
    reference's ops: there this GEMM is DeepGEMM's (w8a8_block_fp8_matmul_deepgemm, fp8_kernel.py)."""
    check_mm_common(mat_a, mat_b, out_dtype, FP8, "Float8_e4m3fn")
    check_blockwise_scales(mat_a, mat_b, scales_a, scales_b)
    m, k = mat_a.shape
    n = mat_b.size(1)
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    out = torch.empty((m, n), dtype=out_dtype, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_fp8_blockwise_scaled_mm_ue8m0(
        mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_a.data_ptr(), scales_a.stride(0), scales_a.stride(1),
        scales_b.data_ptr(), scales_b.stride(0), scales_b.stride(1),
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, *_lib.workspace(mat_a.device),
        _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "fp8_blockwise_scaled_mm_ue8m0")
    return out


def fp8_blockwise_scaled_mm_bias(mat_a, mat_b, scales_a, scales_b, out_dtype, bias):
    """fp8_blockwise_scaled_mm followed by the caller's `output += bias`
    (fp8_utils.py:207-211) in one kernel; no counterpart among the reference's ops."""
    check_mm_common(mat_a, mat_b, out_dtype, FP8, "Float8_e4m3fn")
    check_blockwise_scales(mat_a, mat_b, scales_a, scales_b)
    m, k = mat_a.shape
    n = mat_b.size(1)
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    _check(bias.is_cuda and bias.is_contiguous() and bias.numel() == n and bias.dtype == out_dtype,
           "bias must be a contiguous CUDA tensor of N elements in out_dtype")
    out = torch.empty((m, n), dtype=out_dtype, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_fp8_blockwise_scaled_mm_bias(
        mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_a.data_ptr(), scales_a.stride(0), scales_a.stride(1),
        scales_b.data_ptr(), scales_b.stride(0), scales_b.stride(1), bias.data_ptr(),
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, *_lib.workspace(mat_a.device),
        _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "fp8_blockwise_scaled_mm_bias")
    return out


def block_fp8_linear(input_2d, mat_b, scales_b, bias=None, eps=1e-10):
    """per_token_group_quant_fp8(input_2d, 128) followed by fp8_blockwise_scaled_mm and the caller's
    bias add (fp8_utils.py:204-211) as one operator; for M <= 4 on the shapes that the decode kernel
    without split-K takes with one to 2.5 blocks per compute unit it is a single launch (for M <= 8 only
    when a 16- or 32-row block is forced through the test hook), otherwise the two kernels in turn.  input_2d [M, K] contiguous, 16- or 32-bit float;
    mat_b [K, N] column-major e4m3fn; scales_b [K/128, N/128] fp32; the output has input_2d's dtype
    (bfloat16 or half).  Bit-identical to the operators called in turn."""
    _check(input_2d.is_cuda and mat_b.is_cuda and scales_b.is_cuda, "tensors must be CUDA tensors")
    _check(input_2d.dim() == 2 and input_2d.is_contiguous(), "input must be a contiguous 2D tensor")
    _check(mat_b.dim() == 2 and mat_b.stride(0) == 1 and mat_b.dtype == FP8, "mat_b must be a column major Float8_e4m3fn tensor")
    _check(input_2d.dtype in (torch.bfloat16, torch.float16), "input must be BFloat16 or Half (the output takes its dtype)")
    m, k = input_2d.shape
    n = mat_b.size(1)
    _check(mat_b.size(0) == k, "input and mat_b shapes cannot be multiplied")
    _check(k % 128 == 0, "K must be a multiple of the quantization group, 128")
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    _check(scales_b.dtype == torch.float32 and scales_b.dim() == 2 and scales_b.shape == (k // 128, (n + 127) // 128),
           "scales_b must be a Float32 [K/128, ceil(N/128)] tensor")
    out_dtype = input_2d.dtype
    if bias is not None:
        _check(bias.is_cuda and bias.is_contiguous() and bias.numel() == n and bias.dtype == out_dtype,
               "bias must be a contiguous CUDA tensor of N elements in the output dtype")
    out = torch.empty((m, n), dtype=out_dtype, device=input_2d.device)
    if m == 0 or n == 0:
        return out
    rc = _lib.load().sglq_w8a8_block_fp8_linear(
        input_2d.data_ptr(), DTYPE_CODE[input_2d.dtype], mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_b.data_ptr(), scales_b.stride(0), scales_b.stride(1), None if bias is None else bias.data_ptr(),
        out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype], m, n, k, eps, *_lib.workspace(input_2d.device),
        _lib.stream_ptr(input_2d.device))
    _lib.check(rc, "w8a8_block_fp8_linear")
    return out


def _token_quant_linear(fn_name, elem_dtype, elem_name, input_2d, mat_b, scales_b, bias):
    _check(input_2d.is_cuda and mat_b.is_cuda and scales_b.is_cuda, "tensors must be CUDA tensors")
    _check(input_2d.dim() == 2 and input_2d.is_contiguous(), "input must be a contiguous 2D tensor")
    _check(mat_b.dim() == 2 and mat_b.stride(0) == 1 and mat_b.dtype == elem_dtype, f"mat_b must be a column major {elem_name} tensor")
    _check(input_2d.dtype in (torch.bfloat16, torch.float16), "input must be BFloat16 or Half (the output takes its dtype)")
    m, k = input_2d.shape
    n = mat_b.size(1)
    _check(mat_b.size(0) == k, "input and mat_b shapes cannot be multiplied")
    _check(k % 16 == 0, "mat_b must be multiple of 16 bytes for memory alignment")
    _check((n * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    _check(n <= 1 or mat_b.stride(1) % 16 == 0, "mat_b column stride must be a multiple of 16 bytes")
    _check(scales_b.dtype == torch.float32 and scales_b.is_contiguous() and scales_b.numel() == n, "scales_b must be a contiguous Float32 tensor of N elements")
    out_dtype = input_2d.dtype
    if bias is not None:
        _check(bias.is_cuda and bias.is_contiguous() and bias.numel() == n and bias.dtype == out_dtype,
               "bias must be a contiguous CUDA tensor of N elements in the output dtype")
    out = torch.empty((m, n), dtype=out_dtype, device=input_2d.device)
    if m == 0 or n == 0:
        return out
    rc = getattr(_lib.load(), fn_name)(
        input_2d.data_ptr(), DTYPE_CODE[input_2d.dtype], mat_b.data_ptr(), mat_b.stride(1) if n > 1 else k,
        scales_b.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(), out.stride(0), DTYPE_CODE[out_dtype],
        m, n, k, *_lib.workspace(input_2d.device), _lib.stream_ptr(input_2d.device))
    _lib.check(rc, fn_name[5:])
    return out


def int8_linear(input_2d, mat_b, scales_b, bias=None):
    """per_token_quant_int8(input_2d) followed by int8_scaled_mm (the pair of calls of
    W8A8Int8LinearMethod.apply, w8a8_int8.py:387-391) as one operator, the fused form of the reference's
    CPU backend (int8_scaled_mm_with_quant, sgl-kernel/csrc/cpu/gemm_int8.cpp:423-489).  For decode rows on
    the shapes of the decode kernel without split-K it is a single launch, otherwise the two kernels run one
    after the other.  input_2d [M, K] contiguous bfloat16 or half; mat_b [K, N] column-major int8; scales_b
    [N] or [N, 1] fp32; the output has input_2d's dtype.  Bit-identical to the operators called in turn."""
    return _token_quant_linear("sglq_w8a8_int8_linear", torch.int8, "Int8", input_2d, mat_b, scales_b, bias)


def fp8_linear(input_2d, mat_b, scales_b, bias=None):
    """sgl_per_token_quant_fp8(input_2d) followed by fp8_scaled_mm (apply_fp8_linear's dynamic per-token
    branch, fp8_utils.py:693,725-732) as one operator; see int8_linear.  mat_b [K, N] column-major e4m3fn."""
    return _token_quant_linear("sglq_w8a8_fp8_linear", FP8, "Float8_e4m3fn", input_2d, mat_b, scales_b, bias)


def _group_quant_impl(fn_name, q_dtype, input, output_q, output_s, group_size, eps, qmin, qmax):
    check_group_quant(input, output_q, output_s, group_size, q_dtype)
    if input.numel() == 0:
        return
    hidden = input.shape[-1]
    rows = input.numel() // hidden
    lib = _lib.load()
    rc = getattr(lib, fn_name)(
        input.data_ptr(), DTYPE_CODE[input.dtype], output_q.data_ptr(), output_s.data_ptr(), rows, hidden,
        int(group_size), output_s.stride(0), output_s.stride(1), float(eps), float(qmin), float(qmax),
        _lib.stream_ptr(input.device))
    _lib.check(rc, fn_name)


def _sgl_per_token_group_quant_fp8_impl(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0):
    if scale_ue8m0:
        # power-of-two scales packed four exponent bytes to an int32 word, column-major
        # (per_token_group_quant_8bit.cu:50-65,86-105; the reference asserts a column-major buffer, :190-191)
        for name, t in (("input", input), ("output_q", output_q)):
            _check(t.is_cuda, f"{name} must be a CUDA tensor")
            _check(t.is_contiguous(), f"{name} must be contiguous")
        _check(output_s.is_cuda, "output_s must be a CUDA tensor")
        _check(input.dtype in DTYPE_CODE, "input must be Float, Half or BFloat16")
        _check(output_q.dtype == FP8 and output_q.shape == input.shape, "output_q must be Float8_e4m3fn with the shape of input")
        if group_size != 128:
            raise NotImplementedError("sgl_per_token_group_quant_fp8: scale_ue8m0=True is built for group_size 128 only")
        _check(input.dim() >= 1 and input.shape[-1] % 128 == 0, "the last dimension must be divisible by group_size")
        _check(output_s.dim() == 2, "output_s must be a 2D tensor")
        _check(output_s.dtype == torch.int32, "output_s must be Int32 (four UE8M0 scales per element)")
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        groups = input.shape[-1] // 128
        _check(output_s.size(0) == rows and output_s.size(1) * 4 >= groups, "output_s has the wrong shape")
        if rows == 0:
            return
        _check(output_s.stride(0) == 1 and output_s.stride(1) >= rows, "output_s must be column major (scale_ue8m0)")
        rc = _lib.load().sglq_per_token_group_quant_fp8_ue8m0(
            input.data_ptr(), DTYPE_CODE[input.dtype], output_q.data_ptr(), output_s.data_ptr(), rows, input.shape[-1],
            output_s.stride(1), float(eps), float(fp8_min), float(fp8_max), _lib.stream_ptr(input.device))
        _lib.check(rc, "sgl_per_token_group_quant_fp8")
        return
    _group_quant_impl("sglq_per_token_group_quant_fp8", FP8, input, output_q, output_s, group_size, eps, fp8_min, fp8_max)


def _sgl_per_token_group_quant_int8_impl(input, output_q, output_s, group_size, eps, int8_min, int8_max):
    _group_quant_impl("sglq_per_token_group_quant_int8", torch.int8, input, output_q, output_s, group_size, eps, int8_min, int8_max)


def _sgl_per_token_quant_fp8_impl(input, output_q, output_s):
    check_token_quant_fp8(input, output_q, output_s)
    if input.numel() == 0:
        return
    lib = _lib.load()
    rc = lib.sglq_per_token_quant_fp8(
        input.data_ptr(), DTYPE_CODE[input.dtype], output_q.data_ptr(), output_s.data_ptr(),
        input.size(0), input.size(1), _lib.stream_ptr(input.device))
    _lib.check(rc, "sgl_per_token_quant_fp8")


def _sgl_per_tensor_quant_fp8_impl(input, output_q, output_s, is_static):
    check_tensor_quant_fp8(input, output_q, output_s)
    if input.numel() == 0:
        return
    lib = _lib.load()
    rc = lib.sglq_per_tensor_quant_fp8(
        input.data_ptr(), DTYPE_CODE[input.dtype], output_q.data_ptr(), output_s.data_ptr(), input.numel(),
        1 if is_static else 0, _lib.stream_ptr(input.device))
    _lib.check(rc, "sgl_per_tensor_quant_fp8")


_SCHEMAS = {
    # sgl-kernel/csrc/common_extension.cc:101-130
    "int8_scaled_mm": "(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? bias) -> Tensor",
    "fp8_scaled_mm": "(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? bias) -> Tensor",
    "fp8_blockwise_scaled_mm": "(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype) -> Tensor",
    "sgl_per_token_group_quant_fp8": "(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s, int group_size, float eps, float fp8_min, float fp8_max, bool scale_ue8m0) -> ()",
    "sgl_per_token_group_quant_int8": "(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s, int group_size, float eps, float int8_min, float int8_max) -> ()",
    "sgl_per_token_quant_fp8": "(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s) -> ()",
    "sgl_per_tensor_quant_fp8": "(Tensor input, Tensor(a!) output_q, Tensor(b!) output_s, bool is_static) -> ()",
}
_IMPLS = {
    "int8_scaled_mm": _int8_scaled_mm_impl,
    "fp8_scaled_mm": _fp8_scaled_mm_impl,
    "fp8_blockwise_scaled_mm": _fp8_blockwise_scaled_mm_impl,
    "sgl_per_token_group_quant_fp8": _sgl_per_token_group_quant_fp8_impl,
    "sgl_per_token_group_quant_int8": _sgl_per_token_group_quant_int8_impl,
    "sgl_per_token_quant_fp8": _sgl_per_token_quant_fp8_impl,
    "sgl_per_tensor_quant_fp8": _sgl_per_tensor_quant_fp8_impl,
}

_library = torch.library.Library("sgl_kernel", "FRAGMENT")
for _name, _schema in _SCHEMAS.items():
    _library.define(_name + _schema)
    _library.impl(_name, _IMPLS[_name], "CUDA")


# ---------------------------------------------------------------------------
# public wrappers: same names, argument order and forwarding as the reference
# ---------------------------------------------------------------------------
def int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    return torch.ops.sgl_kernel.int8_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    return torch.ops.sgl_kernel.fp8_blockwise_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype)


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    return torch.ops.sgl_kernel.fp8_scaled_mm.default(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def sgl_per_token_group_quant_fp8(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    fp8_min: float,
    fp8_max: float,
    scale_ue8m0: bool,
) -> None:
    torch.ops.sgl_kernel.sgl_per_token_group_quant_fp8.default(
        input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0
    )


def sgl_per_token_group_quant_int8(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    int8_min: float,
    int8_max: float,
) -> None:
    torch.ops.sgl_kernel.sgl_per_token_group_quant_int8.default(
        input, output_q, output_s, group_size, eps, int8_min, int8_max
    )


def sgl_per_token_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor) -> None:
    torch.ops.sgl_kernel.sgl_per_token_quant_fp8.default(input, output_q, output_s)


def sgl_per_tensor_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor, is_static: bool) -> None:
    """sgl-kernel/python/sgl_kernel/gemm.py:129-137."""
    torch.ops.sgl_kernel.sgl_per_tensor_quant_fp8.default(input, output_q, output_s, is_static)


def int8_mm_i32(mat_a: torch.Tensor, mat_b: torch.Tensor) -> torch.Tensor:
    """INT32 accumulators of ``int8_scaled_mm`` before its epilogue (no reference
    counterpart; used to compare the accumulators bit for bit)."""
    check_mm_common(mat_a, mat_b, torch.bfloat16, torch.int8, "Int8")
    m, k = mat_a.shape
    n = mat_b.size(1)
    out = torch.empty((m, n), dtype=torch.int32, device=mat_a.device)
    lib = _lib.load()
    rc = lib.sglq_int8_mm_i32(mat_a.data_ptr(), mat_a.stride(0) if m > 1 else k, mat_b.data_ptr(),
                              mat_b.stride(1) if n > 1 else k, out.data_ptr(), out.stride(0), m, n, k,
                              *_lib.workspace(mat_a.device), _lib.stream_ptr(mat_a.device))
    _lib.check(rc, "int8_mm_i32")
    return out
