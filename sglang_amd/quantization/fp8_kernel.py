"""Host-side quantization helpers of the FP8 path, mirroring the callers in
python/sglang/srt/layers/quantization/fp8_kernel.py (names, arguments, returned
layouts), on top of the HIP operators."""

from __future__ import annotations

import torch

from typing import Optional, Tuple

from .. import _lib
from .._lib import DTYPE_CODE
from ..sgl_kernel import sgl_per_tensor_quant_fp8, sgl_per_token_group_quant_fp8, sgl_per_token_quant_fp8

# gfx950 implements the OCP formats: e4m3fn with maximum 448 (fp8_kernel.py:71-85
# selects the fnuz/224 variant only for gfx94x).
fp8_dtype = torch.float8_e4m3fn
fp8_max = torch.finfo(fp8_dtype).max
fp8_min = -fp8_max


def create_per_token_group_quant_fp8_output_scale(
    x_shape,
    device,
    group_size,
    column_major_scales: bool,
    scale_tma_aligned: bool,
    scale_ue8m0: bool,
):
    """Scale buffer in the layout the consumer GEMM wants (fp8_kernel.py:300-341)."""
    if scale_ue8m0:
        # int32 words of four exponent bytes, [ceil4(K/128)/4, ceil4(M)] transposed; zero-filled as in the
        # reference (:319-323), so that the bytes of groups beyond K/128 are defined
        assert column_major_scales and scale_tma_aligned
        x_q_mn, x_q_k = x_shape
        x_s_mn, x_s_k = x_q_mn, x_q_k // 128
        aligned_mn = (x_s_mn + 3) // 4 * 4
        aligned_k = (x_s_k + 3) // 4 * 4
        return torch.zeros((aligned_k // 4, aligned_mn), device=device, dtype=torch.int).transpose(0, 1)[:x_s_mn, :]
    if column_major_scales:
        if scale_tma_aligned:
            aligned_size = (x_shape[-2] + 3) // 4 * 4
            return torch.empty(
                x_shape[:-2] + (x_shape[-1] // group_size, aligned_size), device=device, dtype=torch.float32
            ).permute(-1, -2)[: x_shape[-2], :]
        return torch.empty(
            (x_shape[-1] // group_size,) + x_shape[:-1], device=device, dtype=torch.float32
        ).permute(-1, -2)
    return torch.empty(x_shape[:-1] + (x_shape[-1] // group_size,), device=device, dtype=torch.float32)


def sglang_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
):
    """fp8_kernel.py:344-372."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = torch.empty_like(x, device=x.device, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(
        x_shape=tuple(x.shape),
        device=x.device,
        group_size=group_size,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
    )
    if x.shape[0] > 0:
        sgl_per_token_group_quant_fp8(x, x_q, x_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0)
    return x_q, x_s


# The reference's `per_token_group_quant_fp8` (fp8_kernel.py:217-297) is the Triton
# twin with the same signature; here both names run the HIP kernel.
per_token_group_quant_fp8 = sglang_per_token_group_quant_fp8


def sglang_per_token_quant_fp8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype):
    """fp8_kernel.py:375-391."""
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[0], 1, device=x.device, dtype=torch.float32)
    sgl_per_token_quant_fp8(x, x_q, x_s)
    return x_q, x_s


def static_quant_fp8(
    x: torch.Tensor,
    x_s: torch.Tensor,
    repeat_scale: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:437-490: quantize `x` (ndim >= 2, contiguous) with the given per-tensor
    scale; with repeat_scale the returned scale is that value once per token, shape [M, 1]."""
    assert x.is_contiguous(), "`x` is not contiguous"
    assert x_s.numel() == 1, "only supports per-tensor scale"
    if not x.is_cuda:
        raise RuntimeError("static_quant_fp8: input must be a CUDA tensor")
    if x.dtype not in DTYPE_CODE:
        raise NotImplementedError(f"static_quant_fp8: unsupported input dtype {x.dtype}")
    x_q = torch.empty_like(x, device=x.device, dtype=fp8_dtype)
    n = x.shape[-1]
    m = x.numel() // n if n > 0 else 0
    scale = x_s if x_s.dtype == torch.float32 and x_s.device == x.device else x_s.to(device=x.device, dtype=torch.float32)
    x_s_repeat = torch.empty((m, 1), device=x.device, dtype=torch.float32) if repeat_scale else None
    rc = _lib.load().sglq_static_quant_fp8(
        x.data_ptr(), DTYPE_CODE[x.dtype], x_q.data_ptr(), scale.data_ptr(),
        x_s_repeat.data_ptr() if repeat_scale else None, m, n, _lib.stream_ptr(x.device))
    _lib.check(rc, "static_quant_fp8")
    return x_q, (x_s_repeat if repeat_scale else x_s)


def scaled_fp8_quant(
    input: torch.Tensor,
    scale: Optional[torch.Tensor] = None,
    num_token_padding: Optional[int] = None,
    use_per_token_if_dynamic: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """fp8_kernel.py:1233-1266 (the sgl_kernel branch): per-token dynamic, per-tensor
    dynamic (scale starts at zero, the op merges max|x| / 448 into it) or per-tensor
    static quantization of a 2-D tensor; rows past input's are left unwritten."""
    assert input.ndim == 2, f"Expected 2D input tensor, got {input.ndim}D"
    shape = input.shape
    if num_token_padding:
        shape = (max(num_token_padding, input.shape[0]), shape[1])
    output = torch.empty(shape, device=input.device, dtype=fp8_dtype)
    q = output[: input.shape[0]]
    if scale is None:
        if use_per_token_if_dynamic:
            scale = torch.empty((shape[0], 1), device=input.device, dtype=torch.float32)
            sgl_per_token_quant_fp8(input, q, scale[: input.shape[0]])
        else:
            scale = torch.zeros(1, device=input.device, dtype=torch.float32)
            sgl_per_tensor_quant_fp8(input, q, scale, is_static=False)
    else:
        assert scale.numel() == 1, f"Expected scalar scale, got numel={scale.numel()}"
        sgl_per_tensor_quant_fp8(input, q, scale, is_static=True)
    return output, scale


def w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size,
    output_dtype: torch.dtype = torch.float16,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """fp8_kernel.py:801-846,870-967 (w8a8_block_fp8_matmul and its Triton twin): A e4m3fn
    [..., K] contiguous, B e4m3fn [N, K] contiguous (the weight as stored), As fp32 [..., K/128]
    (row-major, as per_token_group_quant_fp8 returns it without column_major_scales), Bs fp32
    [N/128, K/128]; N and K need not be multiples of 128 (K of 16 and N of 4).  `bias` (not an argument of the
    reference's function): the caller's `output += bias` (fp8_utils.py:307-308) fused, [N] in
    output_dtype, same two roundings.  UE8M0-packed (int32) scales are not accepted."""
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]
    if block_n != 128 or block_k != 128:
        raise NotImplementedError("w8a8_block_fp8_matmul: only 128 x 128 weight blocks are built")
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1]
    assert A.is_contiguous()
    if As.dtype != torch.float32 or Bs.dtype != torch.float32:
        raise NotImplementedError("w8a8_block_fp8_matmul: scales must be Float32")
    assert -(-A.shape[-1] // block_k) == As.shape[-1]
    M = A.numel() // A.shape[-1]
    assert B.ndim == 2
    assert B.is_contiguous()
    assert Bs.ndim == 2
    N, K = B.shape
    assert -(-N // block_n) == Bs.shape[0]
    assert -(-K // block_k) == Bs.shape[1]
    if not (A.is_cuda and B.is_cuda and As.is_cuda and Bs.is_cuda):
        raise RuntimeError("w8a8_block_fp8_matmul: tensors must be CUDA tensors")
    if A.dtype != fp8_dtype or B.dtype != fp8_dtype:
        raise RuntimeError("w8a8_block_fp8_matmul: A and B must be Float8_e4m3fn")
    if output_dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("w8a8_block_fp8_matmul: output_dtype must be Half or BFloat16")
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    if M == 0 or N == 0:
        return C
    As2 = As.reshape(M, As.shape[-1])
    if not Bs.is_contiguous():
        Bs = Bs.contiguous()
    lib = _lib.load()
    if bias is not None:
        if not (bias.is_cuda and bias.is_contiguous() and bias.numel() == N and bias.dtype == output_dtype):
            raise RuntimeError("w8a8_block_fp8_matmul: bias must be a contiguous CUDA tensor of N elements in output_dtype")
        rc = lib.sglq_fp8_blockwise_scaled_mm_bias(
            A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
            Bs.data_ptr(), Bs.stride(1), Bs.stride(0), bias.data_ptr(), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
            *_lib.workspace(A.device), _lib.stream_ptr(A.device))
    else:
        rc = lib.sglq_fp8_blockwise_scaled_mm(
            A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
            Bs.data_ptr(), Bs.stride(1), Bs.stride(0), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
            *_lib.workspace(A.device), _lib.stream_ptr(A.device))
    _lib.check(rc, "w8a8_block_fp8_matmul")
    return C


# the Triton kernel behind it (:870-948) computes the same sums
w8a8_block_fp8_matmul_triton = w8a8_block_fp8_matmul


def per_token_group_quant_fp8_pow2(x: torch.Tensor, group_size: int = 128, eps: float = 1e-10,
                                   column_major_scales: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """sglang_per_token_group_quant_fp8(..., scale_ue8m0=True) (fp8_kernel.py:344-372) with the scales as fp32
    instead of four exponent bytes per int32: each group's scale is the smallest power of two >=
    max(amax / 448, 1e-10), the codes are the same.  The input of w8a8_block_fp8_matmul_deepgemm here."""
    assert group_size == 128, "power-of-two scales are built for groups of 128"
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    if not x.is_cuda:
        raise RuntimeError("per_token_group_quant_fp8_pow2: input must be a CUDA tensor")
    if x.dtype not in DTYPE_CODE:
        raise RuntimeError("per_token_group_quant_fp8_pow2: input must be Half, BFloat16 or Float")
    x_q = torch.empty_like(x, device=x.device, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(tuple(x.shape), x.device, group_size, column_major_scales, False, False)
    hidden = x.shape[-1]
    tokens = x.numel() // hidden
    if tokens > 0:
        s2 = x_s.reshape(tokens, hidden // group_size) if x_s.ndim != 2 else x_s
        rc = _lib.load().sglq_per_token_group_quant_fp8_pow2(
            x.data_ptr(), DTYPE_CODE[x.dtype], x_q.data_ptr(), s2.data_ptr(), tokens, hidden, s2.stride(0), s2.stride(1),
            eps, fp8_min, fp8_max, _lib.stream_ptr(x.device))
        _lib.check(rc, "per_token_group_quant_fp8_pow2")
    return x_q, x_s


def unpack_ue8m0_scales(x_s: torch.Tensor, num_groups: int) -> torch.Tensor:
    """The fp32 powers of two [M, num_groups] of packed UE8M0 scales [M, ceil(num_groups / 4)] int32 (byte g % 4 of
    word [row, g / 4] is the biased exponent of group g: per_token_group_quant_8bit.cu:57-64,94)."""
    assert x_s.dtype == torch.int32 and x_s.ndim == 2
    shifts = torch.tensor([0, 8, 16, 24], device=x_s.device, dtype=torch.int32)
    e = (x_s.unsqueeze(-1) >> shifts) & 0xFF
    return (e.reshape(x_s.shape[0], -1)[:, :num_groups] << 23).contiguous().view(torch.float32)


# weights whose block scales have been checked to be powers of two: (data_ptr, shape, version counter)
_pow2_checked = set()


def check_pow2_scales(Bs: torch.Tensor, what: str = "Bs") -> None:
    """Raise unless every fp32 scale is a power of two (no mantissa bits, positive): the kernels behind
    w8a8_block_fp8_matmul_deepgemm read only the exponent of a scale on the shapes where the matrix instruction
    applies it, so other values would be rounded down there and used in full elsewhere, with no error.  Checked
    once per tensor (address, shape and version counter; one device round trip), not under stream capture."""
    key = (Bs.device.type, Bs.data_ptr(), tuple(Bs.shape), Bs._version)
    if key in _pow2_checked:
        return
    if Bs.is_cuda and torch.cuda.is_current_stream_capturing():
        return
    bits = Bs.contiguous().view(torch.int32)
    if bool(((bits & 0x7FFFFF) != 0).any()) or bool((bits <= 0).any()):
        raise ValueError(f"w8a8_block_fp8_matmul_deepgemm: {what} holds scales that are not powers of two; the weight must go "
                         "through requant_weight_ue8m0_inplace (or per_block_cast_to_fp8) first")
    if len(_pow2_checked) > 4096:
        _pow2_checked.clear()
    _pow2_checked.add(key)


def w8a8_block_fp8_matmul_deepgemm(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size,
    output_dtype: torch.dtype,
) -> torch.Tensor:
    """fp8_kernel.py:849-867: the block-scaled FP8 GEMM for scales that are powers of two, DeepGEMM's
    gemm_nt_f8f8bf16 in the reference, here sglq_fp8_blockwise_scaled_mm_ue8m0 (the matrix instruction applies
    the scales and accumulates in place).  A e4m3fn [..., K] contiguous; B e4m3fn [N, K] contiguous; As fp32
    powers of two [..., K/128] in any layout (per_token_group_quant_fp8_pow2), or the packed int32 form of
    sglang_per_token_group_quant_fp8(scale_ue8m0=True), which the library reads as it is
    (sglq_fp8_blockwise_scaled_mm_ue8m0_packed); Bs fp32 powers of two
    [N/128, K/128] (per_block_cast_to_fp8 / requant_weight_ue8m0_inplace).  bf16 output only, as there (:859-860)."""
    assert len(block_size) == 2
    if block_size[0] != 128 or block_size[1] != 128:
        raise NotImplementedError("w8a8_block_fp8_matmul_deepgemm: only 128 x 128 weight blocks are built")
    assert output_dtype == torch.bfloat16, "only BFloat16 outputs (fp8_kernel.py:859-860)"
    assert A.shape[-1] == B.shape[-1]
    assert A.is_contiguous() and B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    N, K = B.shape
    assert K % 128 == 0, "K must be a multiple of 128 (fp8_utils.py:228)"
    M = A.numel() // K
    if not (A.is_cuda and B.is_cuda and As.is_cuda and Bs.is_cuda):
        raise RuntimeError("w8a8_block_fp8_matmul_deepgemm: tensors must be CUDA tensors")
    if A.dtype != fp8_dtype or B.dtype != fp8_dtype:
        raise RuntimeError("w8a8_block_fp8_matmul_deepgemm: A and B must be Float8_e4m3fn")
    assert -(-N // 128) == Bs.shape[0] and K // 128 == Bs.shape[1]
    if Bs.dtype != torch.float32:
        raise NotImplementedError("w8a8_block_fp8_matmul_deepgemm: Bs must be Float32 powers of two [N/128, K/128]")
    check_pow2_scales(Bs)
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    if M == 0 or N == 0:
        return C
    if As.dtype == torch.int32:
        As2 = As.reshape(M, As.shape[-1]) if As.ndim != 2 else As
        assert As2.shape == (M, -(-(K // 128) // 4)), "packed scales: one int32 word per row and four K blocks"
        ws_ptr, ws_bytes = _lib.workspace(A.device)
        if 4 * M * (K // 128) + 256 > ws_bytes // 2:
            # (more rows than the cached workspace has room for beside split-K partial sums: expand here)
            return w8a8_block_fp8_matmul_deepgemm(A, B, unpack_ue8m0_scales(As2, K // 128), Bs, block_size, output_dtype)
        rc = _lib.load().sglq_fp8_blockwise_scaled_mm_ue8m0_packed(
            A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
            Bs.data_ptr(), Bs.stride(1), Bs.stride(0), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
            ws_ptr, ws_bytes, _lib.stream_ptr(A.device))
        _lib.check(rc, "w8a8_block_fp8_matmul_deepgemm")
        return C
    elif As.dtype == torch.float32:
        assert As.shape[-1] == K // 128 and As.numel() == M * (K // 128)
        As2 = As.reshape(M, K // 128) if As.ndim != 2 else As
    else:
        raise NotImplementedError("w8a8_block_fp8_matmul_deepgemm: As must be Float32 or packed Int32")
    rc = _lib.load().sglq_fp8_blockwise_scaled_mm_ue8m0(
        A.data_ptr(), K, B.data_ptr(), K, As2.data_ptr(), As2.stride(0), As2.stride(1),
        Bs.data_ptr(), Bs.stride(1), Bs.stride(0), C.data_ptr(), N, DTYPE_CODE[output_dtype], M, N, K,
        *_lib.workspace(A.device), _lib.stream_ptr(A.device))
    _lib.check(rc, "w8a8_block_fp8_matmul_deepgemm")
    return C
