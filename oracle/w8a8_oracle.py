"""CPU oracle for the W8A8 quantized-linear path.  TEST INFRASTRUCTURE ONLY.

This module restates, in IEEE-754 binary32 arithmetic on the CPU (torch CPU
tensors, no GPU, no compiled extension), what each operator on the path
computes in the reference.  Only tests, the smoke check and the benchmark's
CPU-baseline leg may import it; the shipped operators never do.

Every function cites the reference lines it follows.  Parity status:

* per_token_group_quant_fp8 / per_token_quant_fp8 / per_token_quant_int8:
  pinned by closed-form constructions (x = code * scale), by an independent
  bit-level e4m3fn encoder (``e4m3fn_encode_rne``), by the scalar C restatement
  in ``w8a8_oracle.c`` and by torch's CPU float8 cast (tests/test_oracle.py).
* int8 accumulators: pinned exactly by float64 matmul and int64 brute force.
* fp8_blockwise_scaled_mm / fp8_scaled_mm / int8_scaled_mm outputs: pinned by
  special cases that reduce to plain matmul, one-hot rows and float64 brute
  force on tiny shapes; compared at rtol/atol 1e-2 because the reference's
  summation order inside its GEMM library is not defined by its sources.

The reference keeps no golden vectors for this path, so none are checked.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

FP8_E4M3_MAX = 448.0
FP8 = torch.float8_e4m3fn


# ---------------------------------------------------------------------------
# e4m3fn encoder written from the format definition (1-4-3, bias 7, no inf,
# S.1111.111 = NaN, max finite 448).  Independent of torch's cast; used to pin it.
# ---------------------------------------------------------------------------
def e4m3fn_encode_rne(x: torch.Tensor) -> torch.Tensor:
    """Round-to-nearest-even fp32 -> e4m3fn bit patterns (uint8).

    Inputs must already be clamped to [-448, 448] (NaN maps to 0x7f)."""
    x = x.to(torch.float32)
    bits = x.view(torch.int32)
    sign = ((bits >> 24) & 0x80).to(torch.int32)
    ax = x.abs().to(torch.float64)
    out = torch.zeros_like(bits)
    # subnormal range of e4m3: multiples of 2^-9 below 2^-6
    # normal: exponent e in [-6, 8], 3 mantissa bits
    e = torch.floor(torch.log2(torch.clamp(ax, min=2.0**-30)))
    e = torch.clamp(e, min=-6.0)
    # guard against log2 rounding at exact powers of two
    e = torch.where(ax >= torch.pow(2.0, e + 1), e + 1, e)
    e = torch.where((ax < torch.pow(2.0, e)) & (e > -6), e - 1, e)
    quantum = torch.pow(2.0, e - 3)
    scaled = ax / quantum  # exact: power-of-two scaling in float64
    fl = torch.floor(scaled)
    frac = scaled - fl
    up = (frac > 0.5) | ((frac == 0.5) & (torch.remainder(fl, 2.0) == 1.0))
    n = (fl + up.to(torch.float64)).to(torch.int64)  # in units of quantum
    # n in [0, 16]; n == 16 means carry into next binade
    eb = (e + 7).to(torch.int64)  # biased exponent for normals
    is_sub = ax < 2.0**-6
    # subnormals: code = n (n up to 8 -> 8 is the smallest normal, encodes naturally)
    code_sub = n
    code_norm = (eb << 3) + (n - 8)  # n-8 in [0, 8]; 8 carries into exponent
    code = torch.where(is_sub, code_sub, code_norm).to(torch.int32)
    code = torch.where(torch.isnan(x), torch.full_like(code, 0x7F), code)
    out = (code | sign).to(torch.uint8)
    return out


def e4m3fn_decode(codes: torch.Tensor) -> torch.Tensor:
    """uint8 e4m3fn bit patterns -> fp32 values, from the format definition."""
    c = codes.to(torch.int32)
    s = torch.where((c & 0x80) != 0, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = (c & 0x7).to(torch.float32)
    sub = m * 2.0**-9
    nor = (1.0 + m / 8.0) * torch.pow(2.0, (e - 7).to(torch.float32))
    v = torch.where(e == 0, sub, nor)
    v = torch.where((c & 0x7F) == 0x7F, torch.full_like(v, float("nan")), v)
    return (s * v).to(torch.float32)


def _to_fp8(x_clamped: torch.Tensor) -> torch.Tensor:
    return x_clamped.to(FP8)


def round_half_away(x: torch.Tensor) -> torch.Tensor:
    """Round to nearest integer, ties away from zero (C ``roundf``), exactly.

    ``x - trunc(x)`` is exact in binary floating point, so no double rounding."""
    t = torch.trunc(x)
    frac = x - t
    step = torch.where(frac.abs() >= 0.5, torch.sign(x), torch.zeros_like(x))
    return t + step


# ---------------------------------------------------------------------------
# a1  per-token-group FP8 quantization
# ---------------------------------------------------------------------------
def make_group_scale_buffer(
    m: int, k: int, group_size: int, column_major_scales: bool, scale_tma_aligned: bool
) -> torch.Tensor:
    """Scale buffer layouts accepted by the op
    (python/sglang/srt/layers/quantization/fp8_kernel.py:300-341)."""
    g = k // group_size
    if column_major_scales:
        if scale_tma_aligned:
            aligned = (m + 3) // 4 * 4
            return torch.zeros((g, aligned), dtype=torch.float32).permute(1, 0)[:m, :]
        return torch.zeros((g, m), dtype=torch.float32).permute(1, 0)
    return torch.zeros((m, g), dtype=torch.float32)


def per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    eps: float,
    min_8bit: float,
    max_8bit: float,
    dst: torch.dtype,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:45,72-113.

    absmax starts at eps (:45,80); y_s = absmax / max_8bit (:86, fp32 divide);
    q = clamp(x / y_s, min, max) (:110, fp32 divide) cast to dst (:111)."""
    assert x.shape[-1] % group_size == 0
    xf = x.to(torch.float32).reshape(-1, group_size)
    amax = torch.clamp(xf.abs().amax(dim=1, keepdim=True), min=torch.tensor(eps, dtype=torch.float32))
    y_s = amax / torch.tensor(max_8bit, dtype=torch.float32)
    q = torch.clamp(xf / y_s, min_8bit, max_8bit)
    if dst == torch.int8:
        # static_cast<int8_t>(float) truncates toward zero
        qd = torch.trunc(q).to(torch.int8)
    else:
        qd = q.to(dst)
    return qd.reshape(x.shape), y_s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))


def per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int = 128,
    eps: float = 1e-10,
    fp8_min: float = -FP8_E4M3_MAX,
    fp8_max: float = FP8_E4M3_MAX,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Wrapper with the caller's defaults (fp8_kernel.py:83-85,344-372).
    Returns codes [.., K] (e4m3fn) and row-major fp32 scales [.., K/group]."""
    return per_token_group_quant_8bit(x, group_size, eps, fp8_min, fp8_max, FP8)


# ---------------------------------------------------------------------------
# a2  per-token INT8 quantization
# ---------------------------------------------------------------------------
def per_token_quant_int8(x: torch.Tensor, cal_sum: bool = False):
    """python/sglang/srt/layers/quantization/int8_kernel.py:38-48.

    absmax = max(max|x|, 1e-10) (:39); scale = absmax / 127 (:40);
    q = round_half_away(x * (127 / absmax)) (:41-42) -> int8."""
    xf = x.to(torch.float32)
    amax = torch.clamp(xf.abs().amax(dim=-1, keepdim=True), min=torch.tensor(1e-10, dtype=torch.float32))
    c127 = torch.tensor(127.0, dtype=torch.float32)
    scale = amax / c127
    r = c127 / amax
    q = round_half_away(xf * r)
    q = torch.clamp(q, -128, 127).to(torch.int8)
    if cal_sum:
        return q, scale, xf.sum(dim=-1).to(x.dtype)
    return q, scale


# ---------------------------------------------------------------------------
# a3  per-token FP8 quantization
# ---------------------------------------------------------------------------
def per_token_quant_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:35-71.

    max = max|x| from 0 (:35-47); scale = max / 448 (:52);
    inv = scale == 0 ? 0 : 1 / scale (:57); q = clamp(x * inv, +-448) (:68-69)."""
    assert x.dim() == 2
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=1, keepdim=True)
    scale = amax / torch.tensor(FP8_E4M3_MAX, dtype=torch.float32)
    inv = torch.where(scale == 0, torch.zeros_like(scale), 1.0 / scale)
    q = torch.clamp(xf * inv, -FP8_E4M3_MAX, FP8_E4M3_MAX)
    return q.to(FP8), scale


def per_token_group_quant_fp8_ue8m0(x: torch.Tensor, eps: float = 1e-10) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """sgl_per_token_group_quant_fp8 with scale_ue8m0 = true, groups of 128
    (sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:45,72-113).

    amax = max(eps, max|x|) per group (:45,72-84); y_s = amax / 448 (:86);
    y_s = exp2(ceil(log2(max(y_s, 1e-10)))) (:87-89), taken here as the smallest power of two
    that is >= its argument, read off the float's exponent and mantissa bits; the stored byte
    is log2(y_s) + 127 (:94-99); q = clamp(x / y_s, -448, 448) -> e4m3fn RNE (:108-111).
    Where log2f's own rounding could cross an integer (a quotient within a few units in the
    last place above a power of two, fp32 inputs only) the reference's result depends on its
    log2f and is not pinned.

    Returns (q, exponent bytes [M, K/128] uint8, packed int32 [M, ceil4(K/128)/4] laid out as
    python/sglang/srt/layers/quantization/fp8_kernel.py:308-320: zero-filled words of four
    bytes, column-major with the column stride rounded up to 4 rows)."""
    m, k = x.shape
    assert k % 128 == 0
    xf = x.to(torch.float32).reshape(m, k // 128, 128)
    amax = torch.clamp(xf.abs().amax(dim=2), min=eps)
    y = torch.clamp(amax / torch.tensor(FP8_E4M3_MAX, dtype=torch.float32), min=1e-10)
    bits = y.view(torch.int32)
    biased = (bits >> 23) + ((bits & 0x7FFFFF) != 0).to(torch.int32)
    scale = ((biased << 23).to(torch.int32)).view(torch.float32)
    q = torch.clamp(xf / scale.unsqueeze(2), -FP8_E4M3_MAX, FP8_E4M3_MAX).to(FP8).reshape(m, k)
    groups = k // 128
    words = (groups + 3) // 4
    padded = torch.zeros((m, words * 4), dtype=torch.int32)
    padded[:, :groups] = biased
    packed_vals = padded[:, 0::4] | (padded[:, 1::4] << 8) | (padded[:, 2::4] << 16) | (padded[:, 3::4] << 24)
    aligned_m = (m + 3) // 4 * 4
    packed = torch.zeros((words, aligned_m), dtype=torch.int32).transpose(0, 1)[:m, :]
    packed.copy_(packed_vals)
    return q, biased.to(torch.uint8), packed


def per_tensor_quant_fp8(x: torch.Tensor, scale: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """sgl-kernel/csrc/gemm/per_tensor_quant_fp8.cu:10-123.

    Dynamic (scale is None): scale = max|x| / 448 (:44, the maximum over the blocks'
    `max / 448` equals the divide of the overall maximum: the divide is monotonic).
    Then, for both modes: inv = 1 / scale (:56); q = max(min(x * inv, 448), -448)
    (:70,:88) -> e4m3fn RNE.  fminf / fmaxf return their non-NaN operand, so the
    NaN of 0 * inf (all-zero tensor, dynamic) becomes +448."""
    xf = x.to(torch.float32)
    if scale is None:
        scale = (xf.abs().amax() / torch.tensor(FP8_E4M3_MAX, dtype=torch.float32)).reshape(1)
    else:
        scale = scale.to(torch.float32).reshape(1)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale
    v = xf * inv
    v = torch.where(torch.isnan(v), torch.full_like(v, FP8_E4M3_MAX), torch.minimum(v, torch.tensor(FP8_E4M3_MAX)))
    v = torch.maximum(v, torch.tensor(-FP8_E4M3_MAX))
    return v.to(FP8), scale


def static_quant_fp8(x: torch.Tensor, x_s: torch.Tensor, repeat_scale: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """python/sglang/srt/layers/quantization/fp8_kernel.py:395-490.

    Per row (:424-430): y widened to fp32, y_s widened to fp32, y_s_inv = 1 / y_s,
    q = clamp(y * y_s_inv, -448, 448) -> e4m3fn RNE.  With repeat_scale the scale is
    returned once per row, shape [M, 1] fp32 (:431-432,458-465), otherwise x_s itself (:488).
    NaN inputs are not pinned: the reference leaves tl.clamp's NaN behaviour open."""
    assert x.is_contiguous(), "`x` is not contiguous"
    assert x_s.numel() == 1, "only supports per-tensor scale"
    s = x_s.to(torch.float32).reshape(())
    inv = torch.tensor(1.0, dtype=torch.float32) / s
    q = torch.clamp(x.to(torch.float32) * inv, -FP8_E4M3_MAX, FP8_E4M3_MAX).to(FP8)
    if repeat_scale:
        m = x.numel() // x.shape[-1]
        return q, s.reshape(1, 1).repeat(m, 1)
    return q, x_s


# ---------------------------------------------------------------------------
# a4  block-scaled FP8 GEMM
# ---------------------------------------------------------------------------
def fp8_blockwise_scaled_mm(
    a: torch.Tensor,
    b: torch.Tensor,
    scales_a: torch.Tensor,
    scales_b: torch.Tensor,
    out_dtype: torch.dtype,
    acc_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """sgl-kernel/csrc/gemm/fp8_blockwise_gemm_kernel.cu:345-423 (semantics) with
    the per-K-tile accumulation of python/sglang/test/test_block_fp8.py:274-326:

    D[m,n] = sum_kb (sum_{k in kb} A[m,k] B[k,n]) * SFA[m,kb] * SFB[kb, n//128].

    a [M,K] e4m3fn; b [K,N] e4m3fn (any strides); scales_a [M, ceil(K/128)];
    scales_b [ceil(K/128), ceil(N/128)]."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    kb = (k + 127) // 128
    af = a.to(acc_dtype)
    bf = b.to(acc_dtype)
    sa = scales_a.to(acc_dtype)
    sb = scales_b.to(acc_dtype)
    sb_full = sb.repeat_interleave(128, dim=1)[:, :n]  # [kb, N]
    out = torch.zeros((m, n), dtype=acc_dtype)
    for i in range(kb):
        ks = slice(i * 128, min((i + 1) * 128, k))
        p = af[:, ks] @ bf[ks, :]
        out += p * (sa[:, i : i + 1] * sb_full[i : i + 1, :])
    return out.to(out_dtype)


def fp8_blockwise_scaled_grouped_mm(
    a: torch.Tensor,
    b: torch.Tensor,
    scales_a: torch.Tensor,
    scales_b: torch.Tensor,
    problem_sizes: torch.Tensor,
    expert_offsets: torch.Tensor,
    out_dtype: torch.dtype,
    acc_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:587-754 (semantics; callers
    python/sglang/srt/layers/moe/cutlass_moe.py:170-213): expert e computes the block-scaled
    product of rows expert_offsets[e] .. + problem_sizes[e][0] of a [total_m, K] with b[e]
    ([K, N]), activation scales scales_a [total_m, K/128] (K-major), weight scales
    scales_b[e] [K/128, N/128], into the same rows of the output.  Rows that belong to no
    expert are returned as zeros (the operator leaves them untouched)."""
    total_m, n = a.shape[0], b.shape[2]
    out = torch.zeros((total_m, n), dtype=out_dtype)
    for e in range(b.shape[0]):
        rows, first = int(problem_sizes[e][0]), int(expert_offsets[e])
        if rows == 0:
            continue
        sl = slice(first, first + rows)
        out[sl] = fp8_blockwise_scaled_mm(a[sl], b[e], scales_a[sl], scales_b[e], out_dtype, acc_dtype=acc_dtype)
    return out


# ---------------------------------------------------------------------------
# The data movement around the grouped GEMM in an MoE layer
# ---------------------------------------------------------------------------
def prepare_moe_input(topk_ids: torch.Tensor, num_experts: int, n: int, k: int):
    """sgl-kernel/csrc/moe/prepare_moe_input.cu:13-139.  Returns expert_offsets [E + 1],
    blockscale_offsets [E + 1] (:56-76), problem_sizes1 = (count, 2 n, k), problem_sizes2 =
    (count, k, n) (:31-38), input_permutation and output_permutation (:78-96).  The reference
    orders the slots of one expert by thread arrival; any order is a valid result, this one keeps
    slot order.  Slots whose id is outside [0, E) get output_permutation -1 here (the operator
    leaves those entries untouched)."""
    ids = topk_ids.reshape(-1).to(torch.int64)
    topk = topk_ids.shape[1]
    counts = torch.zeros(num_experts, dtype=torch.int64)
    valid = (ids >= 0) & (ids < num_experts)
    counts.scatter_add_(0, ids[valid], torch.ones_like(ids[valid]))
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    rounded = torch.zeros(num_experts + 1, dtype=torch.int64)
    rounded[1:] = torch.cumsum((counts + 127) // 128 * 128, 0)
    ps1 = torch.stack([counts, torch.full_like(counts, 2 * n), torch.full_like(counts, k)], dim=1)
    ps2 = torch.stack([counts, torch.full_like(counts, k), torch.full_like(counts, n)], dim=1)
    a_map = torch.full((ids.numel(),), -1, dtype=torch.int64)
    c_map = torch.full((ids.numel(),), -1, dtype=torch.int64)
    nxt = offsets[:-1].clone()
    for i in range(ids.numel()):
        e = int(ids[i])
        if 0 <= e < num_experts:
            pos = int(nxt[e])
            nxt[e] += 1
            a_map[pos] = i // topk
            c_map[i] = pos
    to32 = lambda t: t.to(torch.int32)
    return to32(offsets), to32(rounded), to32(ps1), to32(ps2), to32(a_map), to32(c_map)


def shuffle_rows(x: torch.Tensor, dst2src_map: torch.Tensor) -> torch.Tensor:
    """prepare_moe_input.cu:168-190: output[d] = input[dst2src_map[d]]."""
    return x[dst2src_map.to(torch.int64)]


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """sgl-kernel/csrc/elementwise/activation.cu:57-60 with the act_and_mul kernel it instantiates
    (:85-103): silu(v) = v / (1 + exp(-v)) in fp32, rounded to the tensor's type; then the product
    with the second half, rounded again."""
    d = x.shape[-1] // 2
    v = x[..., :d].to(torch.float32)
    act = (v / (1.0 + torch.exp(-v))).to(x.dtype)
    return (act.to(torch.float32) * x[..., d:].to(torch.float32)).to(x.dtype)


def apply_shuffle_mul_sum(c2: torch.Tensor, c_map: torch.Tensor, factors: Optional[torch.Tensor], m: int) -> torch.Tensor:
    """prepare_moe_input.cu:258-318: output[i] = sum_j factors[i, j] * c2[c_map[i topk + j]],
    fp32 accumulation in j order, one fused multiply-add per term (the product of two 16-bit
    floats is exact in fp32, so multiply-then-add rounds the same way), rounded to the type."""
    topk = c_map.numel() // m
    acc = torch.zeros((m, c2.shape[1]), dtype=torch.float32)
    cm = c_map.to(torch.int64).reshape(m, topk)
    for j in range(topk):
        f = torch.ones(m, dtype=torch.float32) if factors is None else factors.reshape(m, topk)[:, j].to(torch.float32)
        routed = (cm[:, j] >= 0) & (cm[:, j] < c2.shape[0])  # other entries name no row and add nothing
        term = f.unsqueeze(1) * c2[cm[:, j].clamp(0, max(c2.shape[0] - 1, 0))].to(torch.float32)
        acc = torch.where(routed.unsqueeze(1), acc + term, acc)
    return acc.to(c2.dtype)


def cutlass_fused_experts_fp8(a, w1_q, w2_q, w1_scale, w2_scale, topk_weights, topk_ids) -> torch.Tensor:
    """python/sglang/srt/layers/moe/cutlass_moe.py:140-222 as a sequence of the restatements above:
    a [m, k]; w1_q [E, k, 2 n], w2_q [E, n, k] e4m3fn; w1_scale [E, k/128, 2 n/128], w2_scale
    [E, n/128, k/128]; topk_weights / topk_ids [m, topk]."""
    num_experts, k, n = w1_q.shape[0], w1_q.shape[1], w2_q.shape[1]
    m, topk = topk_ids.shape
    offsets, _, ps1, ps2, a_map, c_map = prepare_moe_input(topk_ids, num_experts, n, k)
    a_q, a1_scale = per_token_group_quant_fp8(a, 128)
    rep_a_q, rep_a1_scales = shuffle_rows(a_q, a_map), shuffle_rows(a1_scale, a_map)
    c1 = fp8_blockwise_scaled_grouped_mm(rep_a_q, w1_q, rep_a1_scales, w1_scale, ps1, offsets[:-1], a.dtype)
    inter = silu_and_mul(c1)
    inter_q, a2_scale = per_token_group_quant_fp8(inter, 128)
    c2 = fp8_blockwise_scaled_grouped_mm(inter_q, w2_q, a2_scale, w2_scale, ps2, offsets[:-1], a.dtype)
    return apply_shuffle_mul_sum(c2, c_map, topk_weights.to(a.dtype), m)


# ---------------------------------------------------------------------------
# a5  INT8 scaled GEMM
# ---------------------------------------------------------------------------
def w8a8_block_int8_matmul(
    a: torch.Tensor,
    b_nk: torch.Tensor,
    scales_a: torch.Tensor,
    scales_b: torch.Tensor,
    out_dtype: torch.dtype,
    acc_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """python/sglang/srt/layers/quantization/int8_kernel.py:273-296 (the Triton kernel's loop):

    C[m,n] = sum_kb float(sum_{k in kb} A[m,k] B[n,k]) * As[m,kb] * Bs[n//128, kb],

    a int8 [M,K]; b_nk int8 [N,K]; scales_a [M, ceil(K/128)]; scales_b [ceil(N/128), ceil(K/128)].
    The int32 block sums are exact (at most 128 * 128^2 < 2^24)."""
    m, k = a.shape
    n, k2 = b_nk.shape
    assert k == k2
    kb = (k + 127) // 128
    af = a.to(torch.float64)
    bf = b_nk.to(torch.float64)
    sa = scales_a.to(acc_dtype)
    sb_full = scales_b.to(acc_dtype).repeat_interleave(128, dim=0)[:n, :]  # [N, kb]
    out = torch.zeros((m, n), dtype=acc_dtype)
    for i in range(kb):
        ks = slice(i * 128, min((i + 1) * 128, k))
        p = (af[:, ks] @ bf[:, ks].t()).to(acc_dtype)  # exact
        out += p * sa[:, i : i + 1] * sb_full[:, i].reshape(1, n)  # (dot * a_s) * b_s as :293
    return out.to(out_dtype)


def block_quant_weight_int8(w: torch.Tensor, block: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """Harness-side block quantization of a weight to int8 (not on the measured path):
    scale = absmax_block / 127 (0 -> 1), q = round-half-even(w / scale), scales [ceil(N/128), ceil(K/128)]."""
    n, k = w.shape
    nb, kb = (n + block - 1) // block, (k + block - 1) // block
    wp = torch.zeros((nb * block, kb * block), dtype=torch.float32)
    wp[:n, :k] = w.float()
    blocks = wp.reshape(nb, block, kb, block)
    amax = blocks.abs().amax(dim=(1, 3))
    scale = amax / 127.0
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = torch.round(blocks / scale[:, None, :, None]).clamp(-127, 127).reshape(nb * block, kb * block)[:n, :k]
    return q.to(torch.int8).contiguous(), scale.contiguous()


def int8_mm_i32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Exact INT32 accumulators of int8 [M,K] x int8 [K,N]
    (sgl-kernel/csrc/gemm/int8_gemm_kernel.cu:38-153, ElementAccumulator int32).
    float64 is exact here: |acc| <= K * 128^2 < 2^53 for any K < 2^39."""
    acc = a.to(torch.float64) @ b.to(torch.float64)
    return acc.to(torch.int64).to(torch.int32)


def int8_scaled_mm(
    a: torch.Tensor,
    b: torch.Tensor,
    scales_a: torch.Tensor,
    scales_b: torch.Tensor,
    out_dtype: torch.dtype,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Epilogue order of
    sgl-kernel/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:278,301:
    out = float(acc) * (s_b[n] * s_a[m]) + float(bias[n])."""
    acc = int8_mm_i32(a, b).to(torch.float32)
    sa = scales_a.reshape(-1, 1).to(torch.float32)
    sb = scales_b.reshape(1, -1).to(torch.float32)
    out = acc * (sb * sa)
    if bias is not None:
        out = out + bias.to(torch.float32).reshape(1, -1)
    return out.to(out_dtype)


# ---------------------------------------------------------------------------
# a6  FP8 scaled GEMM (per-row activation scale, per-column weight scale)
# ---------------------------------------------------------------------------
def fp8_scaled_mm(
    a: torch.Tensor,
    b: torch.Tensor,
    scales_a: torch.Tensor,
    scales_b: torch.Tensor,
    out_dtype: torch.dtype,
    bias: Optional[torch.Tensor] = None,
    acc_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:522-546 (EVT order):
    out = s_a[m] * (s_b[n] * sum_k A B) + bias[n]."""
    acc = a.to(acc_dtype) @ b.to(acc_dtype)
    sa = scales_a.reshape(-1, 1).to(acc_dtype)
    sb = scales_b.reshape(1, -1).to(acc_dtype)
    out = sa * (sb * acc)
    if bias is not None:
        out = out + bias.to(acc_dtype).reshape(1, -1)
    return out.to(out_dtype)


# ---------------------------------------------------------------------------
# Weight preparation for the harness (inputs of the measured ops, not outputs)
# ---------------------------------------------------------------------------
def block_quant_weight(w: torch.Tensor, block: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-128x128-block e4m3fn quantization of W [N,K]: scale = absmax/448
    (0 -> 1), q = (w / scale) -> e4m3fn.  Returns q [N,K] and scales
    [ceil(N/128), ceil(K/128)]  (layout contract of
    python/sglang/srt/layers/quantization/fp8.py:276-306)."""
    n, k = w.shape
    nb, kb = (n + block - 1) // block, (k + block - 1) // block
    wp = torch.zeros((nb * block, kb * block), dtype=torch.float32)
    wp[:n, :k] = w.to(torch.float32)
    t = wp.reshape(nb, block, kb, block).permute(0, 2, 1, 3)
    amax = t.abs().amax(dim=(2, 3))
    scale = amax / FP8_E4M3_MAX
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = torch.clamp(t / scale[:, :, None, None], -FP8_E4M3_MAX, FP8_E4M3_MAX)
    q = q.permute(0, 2, 1, 3).reshape(nb * block, kb * block)[:n, :k].contiguous().to(FP8)
    return q, scale.contiguous()


def per_tensor_quant_weight(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Single fp32 scale for W [N,K] widened to [N,1]
    (python/sglang/srt/layers/quantization/utils.py:72-92)."""
    wf = w.to(torch.float32)
    amax = torch.clamp(wf.abs().amax(), min=1e-12)
    scale = amax / FP8_E4M3_MAX
    q = torch.clamp(wf / scale, -FP8_E4M3_MAX, FP8_E4M3_MAX).to(FP8)
    return q, scale.reshape(1, 1).expand(w.shape[0], 1).contiguous()


# ---------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations (seeded on the CPU)
# ---------------------------------------------------------------------------
def gen_activation(m: int, k: int, seed: int, outliers: bool = False) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    a = torch.randn((m, k), generator=g, dtype=torch.float32)
    if outliers:
        mask = torch.rand((m, k), generator=g) < 0.01
        a = torch.where(mask, a * 20.0, a)
    return a.to(torch.bfloat16)


def gen_weight(n: int, k: int, seed: int, std: float = 0.02) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed + 7919)
    return torch.randn((n, k), generator=g, dtype=torch.float32) * std


def gen_int8_weight(k: int, n: int, seed: int):
    """B int8 [K,N] column-major (stored [N,K]), s_b U[1e-3,1e-2], bias N(0,0.1) bf16."""
    g = torch.Generator().manual_seed(seed + 7919)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    s_b = torch.rand((n,), generator=g, dtype=torch.float32) * 9e-3 + 1e-3
    bias = (torch.randn((n,), generator=g, dtype=torch.float32) * 0.1).to(torch.bfloat16)
    return w.t(), s_b, bias
