"""Pins the CPU oracle (oracle/w8a8_oracle.py) without the reference: closed forms,
an independent bit-level e4m3fn encoder, the scalar C restatement, torch's own
CPU casts, float64/int64 brute force.  The reference holds no golden vectors for
this path (its tests draw fresh random tensors), so none are compared."""
import ctypes
import math

import numpy as np
import pytest
import torch

from helpers import (assert_bits_equal, c_group_quant_fp8, c_tensor_quant_fp8, c_token_quant_fp8, c_token_quant_int8,
                     calc_diff, fp8_bits, moe_case)
from oracle import w8a8_oracle as O

FP8 = torch.float8_e4m3fn


def all_e4m3_values():
    codes = torch.arange(256, dtype=torch.uint8)
    vals = O.e4m3fn_decode(codes)
    return codes, vals


# ------------------------------------------------------------------ e4m3fn
def test_e4m3_decode_matches_torch_and_c(c_oracle):
    codes, vals = all_e4m3_values()
    tv = codes.view(FP8).to(torch.float32)
    finite = ~torch.isnan(vals)
    assert torch.equal(torch.isnan(tv), torch.isnan(vals))
    assert torch.equal(tv[finite], vals[finite])
    assert vals[finite].abs().max().item() == 448.0
    assert int(finite.sum()) == 254
    for c in range(256):
        cv = c_oracle.oracle_e4m3fn_decode(c)
        assert (math.isnan(cv) and math.isnan(vals[c].item())) or cv == vals[c].item()


def test_e4m3_encode_three_ways_agree(c_oracle):
    """Every representable value, every midpoint between neighbours (the ties) and
    the floats just below/above each midpoint: bit-twiddling C encoder, the
    float64 formula encoder and torch's CPU cast give the same byte."""
    _, vals = all_e4m3_values()
    pos = torch.sort(vals[(~torch.isnan(vals)) & (vals >= 0)]).values.unique()
    mids = (pos[:-1].double() + pos[1:].double()) / 2
    mids32 = mids.float()
    assert torch.equal(mids32.double(), mids)  # midpoints are exact in fp32
    cand = torch.cat([pos, mids32, torch.nextafter(mids32, torch.tensor(0.0)), torch.nextafter(mids32, torch.tensor(1e9))])
    g = torch.Generator().manual_seed(1)
    cand = torch.cat([cand, torch.rand(200000, generator=g) * 448, torch.rand(50000, generator=g) * 0.05])
    cand = torch.cat([cand, -cand]).clamp(-448, 448)
    want = fp8_bits(cand.to(FP8))
    got_formula = O.e4m3fn_encode_rne(cand)
    got_c = torch.tensor([c_oracle.oracle_e4m3fn_encode(ctypes.c_float(v)) for v in cand[: 4 * len(pos) * 2 + 4000].tolist()],
                         dtype=torch.uint8)
    # -0.0 keeps its sign bit in all three
    assert_bits_equal(got_formula, want, "formula encoder vs torch cast")
    assert_bits_equal(got_c, want[: got_c.numel()], "C encoder vs torch cast")


def test_e4m3_ties_go_to_even():
    # 17 lies midway between 16 (mantissa 000) and 18 (001): even is 16; 19 -> 20
    x = torch.tensor([17.0, 19.0, -17.0, 0.0009765625, 464.0 - 16.0])
    got = x.to(FP8).float()
    assert got.tolist() == [16.0, 20.0, -16.0, 0.0, 448.0]
    assert O.e4m3fn_decode(O.e4m3fn_encode_rne(x)).tolist() == got.tolist()


# ------------------------------------------------------------------ a1 group quant
def make_closed_form_groups(m, groups, group=128, seed=0, dtype=torch.float32):
    """x = value(code) * scale with +-448 present in every group and power-of-two
    scales, so scale and codes are known without any division rounding
    (the construction of test/srt/quant/test_fp8_kernel.py:24-44)."""
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 256, (m, groups, group), generator=g, dtype=torch.int32)
    codes = torch.where((codes & 0x7F) == 0x7F, codes & 0x80, codes)  # no NaN codes
    codes[:, :, 0] = torch.where(torch.rand((m, groups), generator=g) < 0.5, 0x7E, 0xFE)  # +-448
    vals = O.e4m3fn_decode(codes.to(torch.uint8))
    exp = torch.randint(-8, 5, (m, groups, 1), generator=g)
    scale = torch.pow(2.0, exp.float())
    x = (vals * scale).reshape(m, groups * group)
    return x.to(dtype), codes.to(torch.uint8).reshape(m, groups * group), scale.reshape(m, groups)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_group_quant_closed_form(dtype):
    x, codes, scale = make_closed_form_groups(7, 5, dtype=dtype)
    assert torch.equal(x.float(), (O.e4m3fn_decode(codes).reshape(7, 5, 128) * scale[:, :, None]).reshape(7, 640))
    q, s = O.per_token_group_quant_fp8(x, 128)
    assert_bits_equal(s, scale, "scale")
    # +0 and -0 both decode to 0: compare values, and codes where the value is non-zero
    assert torch.equal(q.float(), O.e4m3fn_decode(codes))
    nz = O.e4m3fn_decode(codes) != 0
    assert torch.equal(fp8_bits(q)[nz], codes[nz])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("group", [128, 64, 32, 16])
def test_group_quant_vs_c_restatement(c_oracle, dtype, group):
    g = torch.Generator().manual_seed(group)
    x = torch.randn((37, 512), generator=g)
    x[3, 128:256] = 0  # all-zero group -> eps floor
    x[5] *= 1e-6
    x[6] *= 3e4 if dtype != torch.float16 else 100.0
    x = x.to(dtype)
    q, s = O.per_token_group_quant_fp8(x, group)
    qc, sc = c_group_quant_fp8(c_oracle, x, group)
    assert_bits_equal(s, sc, "scales")
    assert_bits_equal(fp8_bits(q), qc, "codes")


def test_group_quant_invariants():
    x = O.gen_activation(64, 1024, seed=5, outliers=True)
    q, s = O.per_token_group_quant_fp8(x, 128)
    xf = x.float().reshape(64, 8, 128)
    amax = xf.abs().amax(dim=2)
    assert_bits_equal(s, amax / 448.0, "scale == absmax/448 (one IEEE divide)")
    qf = q.float().reshape(64, 8, 128)
    # the group's max element maps to +-448
    assert torch.equal(qf.abs().amax(dim=2), torch.full((64, 8), 448.0))
    # dequantization error is at most half an e4m3 ulp at the quotient's binade
    quo = (xf / s[:, :, None]).abs()
    ulp = torch.pow(2.0, torch.floor(torch.log2(torch.clamp(quo, min=2.0**-6))) - 3)
    assert bool(((qf.abs() - quo).abs() <= ulp / 2 * (1 + 1e-6)).all())
    # all-zero group: scale = eps/448, codes 0
    z = torch.zeros(2, 256, dtype=torch.bfloat16)
    qz, sz = O.per_token_group_quant_fp8(z, 128)
    assert_bits_equal(sz, torch.full((2, 2), 1e-10, dtype=torch.float32) / 448.0, "zero-group scale")
    assert int(fp8_bits(qz).max()) == 0


def test_group_scale_buffer_layouts():
    for cm, tma in ((False, False), (True, False), (True, True)):
        b = O.make_group_scale_buffer(6, 512, 128, cm, tma)
        assert tuple(b.shape) == (6, 4)
        if cm:
            assert b.stride(0) == 1 and b.stride(1) == (8 if tma else 6)
        else:
            assert b.is_contiguous()


# ------------------------------------------------------------------ a2 int8 per token
def test_int8_quant_closed_form_and_ties():
    # x = k * (absmax / 127) with absmax = 127 * 2^j  ->  x = k * 2^j exactly, code k
    k = torch.arange(-127, 128, dtype=torch.float32)
    for j in (-3, 0, 4):
        x = (k * 2.0**j).reshape(1, -1)
        q, s = O.per_token_quant_int8(x)
        assert q.flatten().tolist() == k.int().tolist()
        assert s.item() == 2.0**j
    # ties: (k + 0.5) * 2^j rounds away from zero, unlike torch.round (half to even)
    halves = torch.tensor([[0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 127.0]])
    q, s = O.per_token_quant_int8(halves)
    assert s.item() == 1.0
    assert q.flatten().tolist() == [1, 2, 3, -1, -2, -3, 127, -127, 127]
    assert torch.round(halves).flatten().tolist()[:6] == [0.0, 2.0, 2.0, -0.0, -2.0, -2.0]
    # 0.49999997 must not round up through x + 0.5
    assert O.round_half_away(torch.tensor([0.49999997, -0.49999997, 8388609.0])).tolist() == [0.0, -0.0, 8388609.0]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_int8_quant_vs_c_restatement(c_oracle, dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn((19, 1000), generator=g)
    x[2] = 0
    x[4] *= 1e-7
    x = x.to(dtype)
    q, s = O.per_token_quant_int8(x)
    qc, sc = c_token_quant_int8(c_oracle, x)
    assert_bits_equal(s, sc, "scales")
    assert_bits_equal(q, qc, "codes")
    assert s[2].item() == np.float32(1e-10) / np.float32(127)
    # library cross-check: half-even rounding differs only at exact .5 products
    prod = x.float() * (torch.tensor(127.0) / torch.clamp(x.float().abs().amax(-1, keepdim=True), min=1e-10))
    he = torch.round(prod).to(torch.int8)
    diff = he != q
    assert bool(((prod[diff] - torch.trunc(prod[diff])).abs() == 0.5).all())


# ------------------------------------------------------------------ a3 fp8 per token
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_token_fp8_quant_vs_c_and_formula(c_oracle, dtype):
    g = torch.Generator().manual_seed(4)
    x = torch.randn((23, 1368), generator=g)
    x[1] = 0  # zero row: scale 0, inverse guarded to 0, codes 0
    x = x.to(dtype)
    q, s = O.per_token_quant_fp8(x)
    qc, sc = c_token_quant_fp8(c_oracle, x)
    assert_bits_equal(s, sc, "scales")
    assert_bits_equal(fp8_bits(q), qc, "codes")
    assert s[1].item() == 0.0 and int(fp8_bits(q)[1].max()) == 0
    # the reference test's formula (sgl-kernel/tests/test_per_token_quant_fp8.py:14-23) on non-zero rows
    rows = [i for i in range(23) if i != 1]
    want = (x.float()[rows] * (1.0 / s[rows])).clamp(-448, 448).to(FP8)
    assert_bits_equal(q[rows], want, "codes vs reference-test formula")


def test_token_fp8_closed_form():
    x, codes, scale = make_closed_form_groups(9, 1, group=256, seed=11)
    q, s = O.per_token_quant_fp8(x)
    assert_bits_equal(s, scale.reshape(9, 1), "scale")
    assert torch.equal(q.float(), O.e4m3fn_decode(codes))


# ------------------------------------------------------------------ f2 fp8 per tensor
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_tensor_fp8_quant_vs_c_and_formula(c_oracle, dtype):
    g = torch.Generator().manual_seed(5)
    x = (torch.randn((37, 203), generator=g) * 3).to(dtype)
    for scale in (None, torch.tensor([0.0123])):
        q, s = O.per_tensor_quant_fp8(x, scale)
        qc, sc = c_tensor_quant_fp8(c_oracle, x, scale)
        assert_bits_equal(s, sc, "scale")
        assert_bits_equal(fp8_bits(q), qc, "codes")
        # the reference test's formula (sgl-kernel/tests/test_per_tensor_quant_fp8.py:28-35)
        want = (x.float() * s.reciprocal()).clamp(-448, 448).to(FP8)
        assert_bits_equal(q, want, "codes vs reference-test formula")
    q, s = O.per_tensor_quant_fp8(x)
    assert s.item() == (x.float().abs().max() / 448).item()
    assert float(q.float().abs().max()) == 448.0


def test_tensor_fp8_closed_form_and_zero_tensor(c_oracle):
    # x = value(code) * 2^e with a +-448 present: scale is 2^e exactly, its inverse too, so the codes come back
    x, codes, scale = make_closed_form_groups(1, 1, group=512, seed=12)
    q, s = O.per_tensor_quant_fp8(x)
    assert_bits_equal(s, scale.reshape(1), "scale")
    assert torch.equal(q.float(), O.e4m3fn_decode(codes))
    # static scale of 2^-3: codes of x / 2^-3
    q, s = O.per_tensor_quant_fp8(torch.tensor([[0.5, -1.0, 100.0, 0.0]]), torch.tensor([0.125]))
    assert q.float().tolist() == [[4.0, -8.0, 448.0, 0.0]]
    # all-zero tensor, dynamic: scale 0, 0 * inf = NaN, fminf / fmaxf turn it into +448 (per_tensor_quant_fp8.cu:70)
    z = torch.zeros(3, 8)
    q, s = O.per_tensor_quant_fp8(z)
    qc, sc = c_tensor_quant_fp8(c_oracle, z)
    assert s.item() == 0.0 and sc.item() == 0.0
    assert fp8_bits(q).unique().tolist() == [0x7E] and qc.unique().tolist() == [0x7E]


# ------------------------------------------------------------------ f2 UE8M0 group scales
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_group_quant_ue8m0_pins(dtype):
    """Power-of-two scales: the reference test's formula 2^ceil(log2(amax / 448))
    (python/sglang/test/test_block_fp8_deep_gemm_blackwell.py:48-59) evaluated in float64, where
    log2 of these fp32 quotients cannot round across an integer; exponent bytes, packing and
    codes from first principles."""
    g = torch.Generator().manual_seed(31)
    x = (torch.randn((37, 640), generator=g) * torch.logspace(-6, 4, 37).unsqueeze(1)).to(dtype)
    x[5, 128:256] = 0  # an all-zero group: eps / 448 < 1e-10, so the scale is the power of two >= 1e-10
    q, exps, packed = O.per_token_group_quant_fp8_ue8m0(x)
    amax = x.float().view(37, 5, 128).abs().amax(dim=2).clamp(min=1e-10)
    y = (amax / 448.0).clamp(min=1e-10)  # fp32, as the kernel
    want_scale = torch.pow(2.0, torch.ceil(torch.log2(y.double())))
    got_scale = torch.pow(2.0, exps.double() - 127)
    assert torch.equal(got_scale, want_scale)
    # the regular scale amax / 448 is at most the power-of-two scale and more than half of it
    assert bool((got_scale >= y.double()).all()) and bool((got_scale < 2 * y.double()).all())
    assert exps[5, 1].item() == 127 + math.ceil(math.log2(1e-10))  # 2^-33
    # codes: exact division by a power of two, then the e4m3fn cast that the other quant ops use
    want_q = (x.float().view(37, 5, 128) / got_scale.float().unsqueeze(2)).clamp(-448, 448).to(FP8).view(37, 640)
    assert_bits_equal(q, want_q, "codes")
    assert float(q.float().abs().max()) <= 448.0 and float(q.float().abs().max()) > 224.0
    # packing: byte g % 4 of word g / 4; words of groups that do not exist stay zero; column-major, stride ceil4(M)
    assert tuple(packed.shape) == (37, 2) and packed.stride() == (1, 40) and packed.dtype == torch.int32
    by = packed.contiguous().view(torch.uint8).view(37, 2, 4)
    assert torch.equal(by[:, 0, :], exps[:, 0:4]) and torch.equal(by[:, 1, 0], exps[:, 4])
    assert int(by[:, 1, 1:].max()) == 0


def test_group_quant_ue8m0_exact_powers_of_two():
    # amax = 448 * 2^e: the quotient is a power of two and stays; one ulp above it doubles the scale
    for e in (-20, -3, 0, 5):
        x = torch.zeros((1, 128))
        x[0, 7] = 448.0 * 2.0 ** e
        x[0, 9] = -3.0 * 2.0 ** e
        q, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
        assert exps.item() == 127 + e and q[0, 7].float().item() == 448.0 and q[0, 9].float().item() == -3.0
        x[0, 7] = float(np.nextafter(np.float32(448.0 * 2.0 ** e), np.float32(np.inf)))
        q, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
        assert exps.item() == 127 + e + 1 and q[0, 7].float().item() == 224.0 and q[0, 9].float().item() == -1.5


# ------------------------------------------------------------------ f2 static per-tensor quant
@pytest.mark.parametrize("dtype", [torch.half, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("num_tokens,d", [(7, 512), (83, 4096), (33, 5120)])
def test_static_quant_fp8_vs_reference_test_formula(c_oracle, dtype, num_tokens, d):
    """The reference's own check (python/sglang/test/test_block_fp8.py:98-159): uniform inputs,
    scale = max / 448 in the input's dtype, native torch formula, allclose at rtol 0.5.  In fp32
    the native formula is the kernel's arithmetic, so the codes must be identical; the C
    restatement's static per-tensor path must agree bit for bit for every dtype."""
    g = torch.Generator().manual_seed(0)
    x = torch.rand((num_tokens, d), generator=g).to(dtype)
    x_s = x.max() / 448.0
    native = (x * (1.0 / x_s)).clamp(min=-448.0, max=448.0).to(FP8)
    q, s = O.static_quant_fp8(x, x_s, repeat_scale=True)
    assert torch.allclose(q.float(), native.float(), rtol=0.50)
    if dtype == torch.float32:
        assert_bits_equal(q, native, "codes vs the reference test's native formula")
    assert tuple(s.shape) == (num_tokens, 1) and s.dtype == torch.float32
    assert torch.all(s == x_s.float())
    qc, _ = c_tensor_quant_fp8(c_oracle, x, x_s.float().reshape(1))
    assert_bits_equal(fp8_bits(q), qc, "codes vs C restatement")
    q2, s2 = O.static_quant_fp8(x, x_s)
    assert s2 is x_s and torch.equal(fp8_bits(q2), fp8_bits(q))


def test_static_quant_fp8_closed_form():
    # power-of-two scale: x / s is exact, representable values come back, the rest saturates or rounds to even
    x = torch.tensor([[0.5, -1.0, 100.0, 0.0, 0.0634765625, -1e9, 3.25 * 0.125, 17.0 * 0.125]])
    q, s = O.static_quant_fp8(x, torch.tensor(0.125))
    assert q.float().tolist() == [[4.0, -8.0, 448.0, 0.0, 0.5, -448.0, 3.25, 16.0]]
    q, s = O.static_quant_fp8(x.reshape(2, 2, 2), torch.tensor([0.125], dtype=torch.bfloat16), repeat_scale=True)
    assert tuple(q.shape) == (2, 2, 2) and s.tolist() == [[0.125]] * 4


# ------------------------------------------------------------------ GEMMs
def rand_fp8(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).clamp(-448, 448).to(FP8)


def test_blockwise_mm_reduces_to_plain_matmul_with_unit_scales():
    a, w = rand_fp8((5, 256), 1), rand_fp8((128, 256), 2)
    sa, sb = torch.ones(5, 2), torch.ones(2, 1)
    out = O.fp8_blockwise_scaled_mm(a, w.t(), sa, sb, torch.float32)
    ref = a.double() @ w.double().t()
    torch.testing.assert_close(out.double(), ref, rtol=1e-6, atol=1e-5)


def test_blockwise_mm_one_hot_rows_select_scaled_weight_rows():
    w = rand_fp8((256, 384), 3)
    sb = torch.rand(3, 2) + 0.5  # [K/128, N/128]
    sa = torch.rand(4, 3) + 0.5
    a = torch.zeros(4, 384)
    ks = [0, 130, 255, 383]
    for i, k in enumerate(ks):
        a[i, k] = 2.0
    out = O.fp8_blockwise_scaled_mm(a.to(FP8), w.t(), sa, sb, torch.float32)
    for i, k in enumerate(ks):
        kb = k // 128
        want = 2.0 * w.float()[:, k] * sa[i, kb] * sb[kb].repeat_interleave(128)
        torch.testing.assert_close(out[i], want, rtol=1e-6, atol=0)


def test_blockwise_mm_vs_c_double_brute_force(c_oracle):
    m, n, k = 3, 136, 384  # N not a multiple of 128: scale index n // 128 with ceil-div shape
    a, w = rand_fp8((m, k), 5, 50.0), rand_fp8((n, k), 6, 0.5)
    g = torch.Generator().manual_seed(7)
    sa = torch.rand((m, 3), generator=g) * 1e-2
    sbw = torch.rand((2, 3), generator=g) * 1e-3  # weight_scale_inv layout [N/128, K/128]
    out = O.fp8_blockwise_scaled_mm(a, w.t(), sa, sbw.t(), torch.float32, acc_dtype=torch.float64)
    ref = torch.empty((m, n), dtype=torch.float64)
    c_oracle.oracle_fp8_blockwise_mm(
        ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(w.contiguous().data_ptr()), ctypes.c_void_p(sa.contiguous().data_ptr()),
        ctypes.c_void_p(sbw.contiguous().data_ptr()), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
        ctypes.c_void_p(ref.data_ptr()))
    torch.testing.assert_close(out.double(), ref, rtol=1e-6, atol=1e-9)
    # the reference tests' dequantize-then-matmul baseline (sgl-kernel/tests/test_fp8_blockwise_gemm.py:19-58)
    deq_a = a.double() * sa.double().repeat_interleave(128, dim=1)
    deq_w = w.double() * sbw.double().repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)
    torch.testing.assert_close(out.double(), deq_a @ deq_w.t(), rtol=1e-6, atol=1e-9)


@pytest.mark.parametrize("out_dtype", [torch.half, torch.bfloat16])
def test_grouped_mm_oracle_vs_reference_test_baseline(out_dtype):
    """The reference accepts its grouped GEMM when, per expert, 1 - cosine-like similarity with
    torch.mm of the unquantized operands is below 0.001 (test_fp8_blockwise_moe.py:247-251)."""
    rows = [16, 64, 0, 48, 112, 16, 32, 80]
    c = moe_case(len(rows), rows, n=256, k=512, seed=21, dtype=out_dtype)
    out = O.fp8_blockwise_scaled_grouped_mm(c["a"], c["b"], c["scales_a"], c["scales_b"], c["problem_sizes"],
                                            c["expert_offsets"], out_dtype)
    first = 0
    for e, m_g in enumerate(rows):
        if m_g:
            baseline = torch.mm(c["a_orig"][e].float(), c["b_orig"][e].float().t())
            assert calc_diff(out[first:first + m_g], baseline) < 0.001
        first += m_g


def test_grouped_mm_oracle_reduces_to_dense_and_leaves_gaps():
    # one expert: the dense operator; experts in any order, with rows between them that belong to nobody
    c = moe_case(1, [40], n=128, k=256, seed=3)
    dense = O.fp8_blockwise_scaled_mm(c["a"], c["b"][0], c["scales_a"], c["scales_b"][0], torch.bfloat16)
    out = O.fp8_blockwise_scaled_grouped_mm(c["a"], c["b"], c["scales_a"], c["scales_b"], c["problem_sizes"],
                                            c["expert_offsets"], torch.bfloat16)
    assert torch.equal(out, dense)
    c = moe_case(3, [16, 16, 16], n=128, k=128, seed=4)
    sizes = torch.tensor([[8, 128, 128], [16, 128, 128], [5, 128, 128]], dtype=torch.int32)
    offsets = torch.tensor([32, 0, 20], dtype=torch.int32)  # expert 0 -> rows 32..39, 1 -> 0..15, 2 -> 20..24
    out = O.fp8_blockwise_scaled_grouped_mm(c["a"], c["b"], c["scales_a"], c["scales_b"], sizes, offsets, torch.bfloat16)
    for e, (first, m_g) in enumerate([(32, 8), (0, 16), (20, 5)]):
        sl = slice(first, first + m_g)
        want = O.fp8_blockwise_scaled_mm(c["a"][sl], c["b"][e], c["scales_a"][sl], c["scales_b"][e], torch.bfloat16)
        assert torch.equal(out[sl], want)
    assert float(out[16:20].abs().max()) == 0.0 and float(out[25:32].abs().max()) == 0.0 and float(out[40:].abs().max()) == 0.0


def test_moe_routing_tables_from_their_definition():
    """prepare_moe_input (prepare_moe_input.cu:13-139): counts are a histogram, offsets their
    running sums (and those of the counts rounded up to 128), every routed slot owns exactly one
    expert-major position inside its expert's range, and the two permutations invert each other."""
    g = torch.Generator().manual_seed(8)
    m, topk, e, n, k = 37, 4, 9, 256, 512
    ids = torch.randint(0, e, (m, topk), generator=g, dtype=torch.int32)
    ids[3, 1] = -1  # routed nowhere
    ids[5, 0] = e   # out of range as well
    offsets, rounded, ps1, ps2, a_map, c_map = O.prepare_moe_input(ids, e, n, k)
    flat = ids.reshape(-1).long()
    hist = torch.bincount(flat[(flat >= 0) & (flat < e)], minlength=e)
    assert torch.equal(ps1[:, 0].long(), hist) and torch.equal(ps2[:, 0].long(), hist)
    assert ps1[:, 1].unique().tolist() == [2 * n] and ps1[:, 2].unique().tolist() == [k]
    assert ps2[:, 1].unique().tolist() == [k] and ps2[:, 2].unique().tolist() == [n]
    assert offsets.tolist() == [0] + torch.cumsum(hist, 0).tolist()
    assert rounded.tolist() == [0] + torch.cumsum((hist + 127) // 128 * 128, 0).tolist()
    routed = (flat >= 0) & (flat < e)
    pos = c_map[routed].long()
    assert sorted(pos.tolist()) == list(range(int(hist.sum())))  # a bijection onto the used positions
    for i in routed.nonzero().flatten().tolist():
        ex, p = int(flat[i]), int(c_map[i])
        assert offsets[ex] <= p < offsets[ex + 1] and int(a_map[p]) == i // topk
    assert c_map[~routed].tolist() == [-1, -1]
    # slot order is kept inside an expert
    for ex in range(e):
        mine = c_map[(flat == ex)].tolist()
        assert mine == sorted(mine)


def test_moe_combine_and_activation_from_their_definitions():
    g = torch.Generator().manual_seed(9)
    m, topk, row = 11, 3, 64
    c2 = torch.randn((m * topk, row), generator=g).to(torch.bfloat16)
    c_map = torch.randperm(m * topk, generator=g).to(torch.int32)
    w = torch.softmax(torch.rand((m, topk), generator=g), dim=-1).to(torch.bfloat16)
    out = O.apply_shuffle_mul_sum(c2, c_map, w, m)
    # the reference's own description of the operator (prepare_moe_input.cu:368-373), in float64
    want = (c2[c_map.long()].view(m, topk, row).double() * w.view(m, topk, 1).double()).sum(dim=1)
    torch.testing.assert_close(out.double(), want, rtol=2 ** -8, atol=1e-6)
    assert torch.equal(O.apply_shuffle_mul_sum(c2, c_map, None, m), O.apply_shuffle_mul_sum(c2, c_map, torch.ones_like(w), m))
    # silu_and_mul: x * sigmoid(x) times the gate, two roundings to the 16-bit type
    x = (torch.randn((5, 96), generator=g) * 3).to(torch.bfloat16)
    got = O.silu_and_mul(x)
    silu = torch.nn.functional.silu(x[:, :48].double())
    want = silu.to(torch.bfloat16).double() * x[:, 48:].double()
    torch.testing.assert_close(got.double(), want, rtol=2 ** -8, atol=1e-30)
    assert O.silu_and_mul(torch.zeros((1, 16), dtype=torch.float16)).abs().max().item() == 0.0
    assert torch.equal(O.shuffle_rows(c2, torch.tensor([2, 2, 0], dtype=torch.int32)), c2[[2, 2, 0]])


def test_moe_layer_oracle_vs_dequantized_float_reference():
    """The whole expert layer against the same layer computed in float64 on dequantized weights
    and unquantized activations.  The reference's check has the form max |err| / max(|ref|, c) < 0.5
    (python/sglang/test/test_cutlass_moe.py:241-254, c = 1e-2 on outputs of the order of 1e-7);
    here c is the outputs' root mean square, plus bounds on the mean and the largest error that
    FP8 quantization of activations and weights explains (a few per cent)."""
    g = torch.Generator().manual_seed(10)
    m, topk, e, n, k = 24, 2, 4, 128, 256
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    w1 = torch.randn((e, 2 * n, k), generator=g) * 0.1
    w2 = torch.randn((e, k, n), generator=g) * 0.1
    q = lambda w: [O.block_quant_weight(w[i]) for i in range(w.shape[0])]
    w1q, w2q = q(w1), q(w2)
    w1_q = torch.stack([t[0] for t in w1q]).transpose(1, 2)       # [E, k, 2n]
    w1_s = torch.stack([t[1] for t in w1q]).transpose(1, 2)       # [E, k/128, 2n/128]
    w2_q = torch.stack([t[0] for t in w2q]).transpose(1, 2)       # [E, n, k]
    w2_s = torch.stack([t[1] for t in w2q]).transpose(1, 2)       # [E, n/128, k/128]
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    tw = torch.softmax(torch.rand((m, topk), generator=g), dim=-1).to(torch.bfloat16)
    out = O.cutlass_fused_experts_fp8(x, w1_q, w2_q, w1_s, w2_s, tw, ids)
    deq = lambda wq, ws: wq.float().double() * ws.double().repeat_interleave(128, 0).repeat_interleave(128, 1)[: wq.shape[0], : wq.shape[1]]
    ref = torch.zeros((m, k), dtype=torch.float64)
    for t in range(m):
        for j in range(topk):
            ex = int(ids[t, j])
            h = deq(*w1q[ex]) @ x[t].double()
            act = torch.nn.functional.silu(h[:n]) * h[n:]
            ref[t] += tw[t, j].double() * (deq(*w2q[ex]) @ act)
    err = (out.double() - ref).abs()
    rms = float(ref.pow(2).mean().sqrt())
    print("moe layer oracle: rms", rms, "mean err", float(err.mean()), "max err", float(err.max()))
    assert float((err / ref.abs().clamp(min=rms)).max()) < 0.5  # the reference's form, clamped at the outputs' scale
    assert float(err.mean()) < 0.04 * rms and float(err.max()) < 0.25 * rms


def test_block_int8_mm_pins(c_oracle):
    """w8a8_block_int8_matmul: unit scales reduce to the exact integer product, one-hot rows select
    scaled weight rows, a double-precision C brute force on N % 128 != 0 and K % 128 != 0, and the
    reference test's block-wise dequantization (test/srt/quant/test_block_int8.py:40-92)."""
    g = torch.Generator().manual_seed(21)
    m, n, k = 4, 136, 320
    a = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int8)
    a[0, :128] = -128
    w[5, :128] = -128  # the extreme block sum 128 * 128^2 = 2^21 is exact
    ones_a, ones_w = torch.ones(m, 3), torch.ones(2, 3)
    out = O.w8a8_block_int8_matmul(a, w, ones_a, ones_w, torch.float32, acc_dtype=torch.float64)
    assert torch.equal(out.double(), a.double() @ w.double().t())
    sa = torch.rand((m, 3), generator=g) * 1e-2
    sw = torch.rand((2, 3), generator=g) * 1e-3
    onehot = torch.zeros((3, k), dtype=torch.int8)
    onehot[0, 7], onehot[1, 200], onehot[2, 319] = 1, -2, 3
    out = O.w8a8_block_int8_matmul(onehot, w, sa[:3], sw, torch.float32)
    for r, (col, v) in enumerate(((7, 1), (200, -2), (319, 3))):
        want = (w[:, col].float() * v) * sa[r, col // 128] * sw.repeat_interleave(128, dim=0)[:n, col // 128]
        torch.testing.assert_close(out[r], want, rtol=1e-6, atol=0)
    out = O.w8a8_block_int8_matmul(a, w, sa, sw, torch.float32, acc_dtype=torch.float64)
    ref = torch.empty((m, n), dtype=torch.float64)
    c_oracle.oracle_int8_blockwise_mm(
        ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(sa.contiguous().data_ptr()),
        ctypes.c_void_p(sw.contiguous().data_ptr()), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
        ctypes.c_void_p(ref.data_ptr()))
    torch.testing.assert_close(out.double(), ref, rtol=1e-6, atol=1e-9)  # the oracle rounds its result to fp32
    deq_a = a.double() * sa.double().repeat_interleave(128, dim=1)[:, :k]
    deq_w = w.double() * sw.double().repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)[:, :k]
    torch.testing.assert_close(out.double(), deq_a @ deq_w.t(), rtol=1e-6, atol=1e-9)
    # harness-side weight quantization round trip
    wf = torch.randn((136, 300), generator=g)
    q, s = O.block_quant_weight_int8(wf)
    deq = q.float() * s.repeat_interleave(128, dim=0)[:136].repeat_interleave(128, dim=1)[:, :300]
    assert float((deq - wf).abs().max()) <= float(s.max()) * 0.5 + 1e-7


def test_int8_accumulators_exact(c_oracle):
    g = torch.Generator().manual_seed(8)
    a = torch.randint(-128, 128, (5, 4096), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (24, 4096), generator=g, dtype=torch.int8)
    acc = O.int8_mm_i32(a, w.t())
    ref = torch.empty((5, 24), dtype=torch.int32)
    c_oracle.oracle_int8_mm_i32(ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(w.data_ptr()), ctypes.c_int64(5),
                                ctypes.c_int64(24), ctypes.c_int64(4096), ctypes.c_void_p(ref.data_ptr()))
    assert torch.equal(acc, ref)
    assert torch.equal(acc.long(), a.long() @ w.long().t())
    # extreme case: all -128 against all -128
    a2 = torch.full((1, 4096), -128, dtype=torch.int8)
    assert O.int8_mm_i32(a2, a2.t()).item() == 4096 * 128 * 128


def test_scaled_mm_epilogues_match_reference_test_formulas():
    g = torch.Generator().manual_seed(9)
    a8 = torch.randint(-127, 128, (6, 64), generator=g, dtype=torch.int8)
    w8 = torch.randint(-127, 128, (16, 64), generator=g, dtype=torch.int8)
    sa, sb = torch.rand((6, 1), generator=g), torch.rand((16, 1), generator=g)
    bias = torch.randn(16, generator=g).to(torch.bfloat16)
    out = O.int8_scaled_mm(a8, w8.t(), sa, sb, torch.bfloat16, bias)
    # sgl-kernel/tests/test_int8_gemm.py:10-16
    ref = (torch.matmul(a8.float(), w8.t().float()) * sa.view(-1, 1) * sb.view(1, -1) + bias).to(torch.bfloat16)
    torch.testing.assert_close(out.float(), ref.float(), rtol=1e-2, atol=1e-2)
    af, wf = rand_fp8((6, 64), 10), rand_fp8((16, 64), 11)
    out = O.fp8_scaled_mm(af, wf.t(), sa, sb, torch.bfloat16, bias)
    # sgl-kernel/tests/test_fp8_gemm.py:6-14
    ref = ((af.float() @ wf.t().float()) * sa.view(-1, 1) * sb.view(1, -1)).to(torch.bfloat16) + bias
    torch.testing.assert_close(out.float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_block_quant_weight_roundtrip():
    w = O.gen_weight(200, 300, seed=1)
    q, s = O.block_quant_weight(w)
    assert tuple(q.shape) == (200, 300) and tuple(s.shape) == (2, 3)
    deq = q.float() * s.repeat_interleave(128, 0)[:200].repeat_interleave(128, 1)[:, :300]
    assert float((deq - w).abs().max()) <= float(s.max()) * 16 + 1e-12  # within half an ulp at the top binade (32/2)
    qt, st = O.per_tensor_quant_weight(w)
    assert tuple(st.shape) == (200, 1) and float(qt.float().abs().max()) == 448.0
