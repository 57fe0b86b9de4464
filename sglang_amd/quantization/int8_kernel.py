"""per_token_quant_int8 with the reference's Python signature
(python/sglang/srt/layers/quantization/int8_kernel.py:51-81), on the HIP kernel."""

from __future__ import annotations

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
