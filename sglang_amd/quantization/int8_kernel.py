"""The INT8 helpers of python/sglang/srt/layers/quantization/int8_kernel.py with the
reference's Python signatures, on the HIP kernels: per_token_quant_int8 (:51-81),
per_token_group_quant_int8 / sglang_per_token_group_quant_int8 (:127-205) and
w8a8_block_int8_matmul (:339-425)."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import _lib
from .._lib import DTYPE_CODE


def per_token_quant_int8(x, scale_dtype=torch.float32, cal_sum=False):
    assert x.is_contiguous()
    if not x.is_cuda:
        raise RuntimeError("per_token_quant_int8: x must be a CUDA tensor")
    if x.dtype not in DTYPE_CODE:
        raise RuntimeError("per_token_quant_int8: x must be Float, Half or BFloat16")
    hidden = x.shape[-1]
    rows = x.numel() // hidden if hidden else 0
    x_q = torch.empty_like(x, device=x.device, dtype=torch.int8)
    scales = torch.empty(x.shape[:-1] + (1,), device=x.device, dtype=torch.float32)
    x_sum = torch.empty(x.shape[:-1], device=x.device, dtype=x.dtype) if cal_sum else None
    if rows > 0:
        lib = _lib.load()
        rc = lib.sglq_per_token_quant_int8(
            x.data_ptr(), DTYPE_CODE[x.dtype], x_q.data_ptr(), scales.data_ptr(),
            x_sum.data_ptr() if cal_sum else None, rows, hidden, _lib.stream_ptr(x.device))
        _lib.check(rc, "per_token_quant_int8")
    if scale_dtype != torch.float32:
        scales = scales.to(scale_dtype)
    if cal_sum:
        return x_q, scales, x_sum
    return x_q, scales


def sglang_per_token_group_quant_int8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = torch.int8,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """int8_kernel.py:186-205: row-major fp32 scales [..., K / group_size]."""
    from ..sgl_kernel import sgl_per_token_group_quant_int8

    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    iinfo = torch.iinfo(dtype)
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), device=x.device, dtype=torch.float32)
    x2 = x.view(-1, x.shape[-1])
    sgl_per_token_group_quant_int8(x2, x_q.view(x2.shape), x_s.view(x2.shape[0], -1), group_size, eps, iinfo.min, iinfo.max)
    return x_q, x_s


# the Triton twin (:127-183) has the same arithmetic (divide, clamp, truncating cast)
per_token_group_quant_int8 = sglang_per_token_group_quant_int8


def w8a8_block_int8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float16,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """int8_kernel.py:339-425: A int8 [..., K] contiguous, B int8 [N, K] contiguous (the
    weight as stored), As fp32 [..., K/128], Bs fp32 [N/128, K/128].  `bias` (not an argument of
    the reference's function): the caller's `output + bias` (int8_utils.py:31-32) fused, [N] in
    output_dtype, same two roundings."""
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]
    if block_n != 128 or block_k != 128:
        raise NotImplementedError("w8a8_block_int8_matmul: only 128 x 128 weight blocks are built")
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1] and A.is_contiguous()
    assert -(-A.shape[-1] // block_k) == As.shape[-1]
    M = A.numel() // A.shape[-1]
    assert B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    N, K = B.shape
    assert -(-N // block_n) == Bs.shape[0]
    assert -(-K // block_k) == Bs.shape[1]
    if not (A.is_cuda and B.is_cuda and As.is_cuda and Bs.is_cuda):
        raise RuntimeError("w8a8_block_int8_matmul: tensors must be CUDA tensors")
    if A.dtype != torch.int8 or B.dtype != torch.int8:
        raise RuntimeError("w8a8_block_int8_matmul: A and B must be Int8")
    if As.dtype != torch.float32 or Bs.dtype != torch.float32:
        raise RuntimeError("w8a8_block_int8_matmul: scales must be Float32")
    if output_dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("w8a8_block_int8_matmul: output_dtype must be Half or BFloat16")
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    if M == 0 or N == 0:
        return C
    As2 = As.reshape(M, As.shape[-1])
    if not Bs.is_contiguous():
        Bs = Bs.contiguous()
    lib = _lib.load()
    if bias is not None:
        if not (bias.is_cuda and bias.is_contiguous() and bias.numel() == N and bias.dtype == output_dtype):
            raise RuntimeError("w8a8_block_int8_matmul: bias must be a contiguous CUDA tensor of N elements in output_dtype")
        rc = lib.sglq_int8_blockwise_scaled_mm_bias(
            A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
            Bs.data_ptr(), Bs.stride(1), Bs.stride(0), bias.data_ptr(), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
            *_lib.workspace(A.device), _lib.stream_ptr(A.device))
        _lib.check(rc, "w8a8_block_int8_matmul")
        return C
    rc = lib.sglq_int8_blockwise_scaled_mm(
        A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
        Bs.data_ptr(), Bs.stride(1), Bs.stride(0), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
        *_lib.workspace(A.device), _lib.stream_ptr(A.device))
    _lib.check(rc, "w8a8_block_int8_matmul")
    return C
