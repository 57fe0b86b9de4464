"""Load-time helpers of the FP8 / INT8 linear methods (plain torch, CPU): closed forms and brute
force, no device involved."""
import pytest
import torch

from sglang_amd.quantization import fp8_utils as F
from sglang_amd.quantization import int8_utils as I

FP8 = torch.float8_e4m3fn


def e4m3_codes(shape, seed):
    """Random finite e4m3fn values (as fp32) with the largest magnitude, 448, present."""
    g = torch.Generator().manual_seed(seed)
    bits = torch.randint(0, 256, shape, generator=g, dtype=torch.int32).to(torch.uint8)
    bits = torch.where((bits & 0x7F) == 0x7F, torch.zeros_like(bits), bits)  # no NaN patterns
    v = bits.view(FP8).float()
    v.view(-1)[0] = 448.0
    return v


def test_input_to_float8_recovers_codes_and_scale():
    # x = code * 2^-5 with a 448 present: 448 / amax = 2^5 exactly, every product is the code itself
    codes = e4m3_codes((37, 50), seed=1)
    q, inv = F.input_to_float8(codes * 2.0**-5)
    assert q.dtype == FP8 and q.is_contiguous()
    assert inv.item() == 2.0**-5
    assert torch.equal(q.float(), codes)
    # all zeros: the clamp at 1e-12 keeps the scale finite, codes are zero
    q0, inv0 = F.input_to_float8(torch.zeros(4, 8))
    assert torch.equal(q0.float(), torch.zeros(4, 8)) and torch.isfinite(inv0)
    # values beyond the maximum cannot occur; the sign of the extreme value does not matter
    qn, invn = F.input_to_float8(-codes * 2.0**-5)
    assert invn.item() == 2.0**-5 and torch.equal(qn.float(), -codes)


def test_block_dequant_against_loops():
    n, k, bn, bk = 150, 200, 64, 128  # neither a multiple of the block
    q = e4m3_codes((n, k), seed=2).to(FP8)
    s = torch.rand((3, 2), generator=torch.Generator().manual_seed(3)) + 0.5
    want = torch.empty(n, k)
    for i in range(n):
        for j in range(k):
            want[i, j] = q[i, j].float() * s[i // bn, j // bk]
    got = F.block_quant_dequant(q, s, [bn, bk], torch.float32)
    assert torch.equal(got, want)
    assert torch.equal(I.block_dequant(q, s, [bn, bk]), want)
    # a leading batch dimension, another output dtype
    got3 = F.block_quant_dequant(q[None].expand(2, n, k), s[None].expand(2, 3, 2), [bn, bk], torch.bfloat16)
    assert got3.shape == (2, n, k) and torch.equal(got3[1], want.to(torch.bfloat16))


def test_tensor_requant_with_equal_scales_keeps_the_codes():
    # every block scaled by 2^-4 and a 448 present: one scale 2^-4 for the tensor, same codes
    codes = e4m3_codes((256, 384), seed=4)
    s = torch.full((2, 3), 2.0**-4)
    q, inv = F.block_quant_to_tensor_quant(codes.to(FP8), s, [128, 128])
    assert inv.item() == 2.0**-4 and torch.equal(q.float(), codes)
    q2, inv2 = F.channel_quant_to_tensor_quant(codes.to(FP8), torch.full((256, 1), 2.0**-4))
    assert inv2.item() == 2.0**-4 and torch.equal(q2.float(), codes)


def test_tensor_requant_with_unequal_scales_is_one_rounding_away():
    codes = e4m3_codes((256, 256), seed=5)
    s = torch.tensor([[1.0, 0.25], [0.5, 0.125]])
    q, inv = F.block_quant_to_tensor_quant(codes.to(FP8), s, [128, 128])
    deq = F.block_quant_dequant(codes.to(FP8), s, [128, 128], torch.float32)
    assert inv.item() == deq.abs().max().item() / 448.0
    # e4m3 keeps 3 mantissa bits: relative error at most 2^-4 for normal values, absolute 2^-10 * scale below
    err = (q.float() * inv - deq).abs()
    assert bool((err <= torch.maximum(deq.abs() * 2.0**-4, inv * 2.0**-10)).all())


def test_per_block_cast_uses_power_of_two_scales():
    assert torch.equal(F.ceil_to_ue8m0(torch.tensor([1.0, 1.5, 0.3, -4.0, 5.0])), torch.tensor([1.0, 2.0, 0.5, 4.0, 8.0]))
    codes = e4m3_codes((128, 256), seed=6)
    codes[0, 128] = 448.0  # each of the two blocks holds a 448
    x = torch.cat([codes[:, :128] * 2.0**3, codes[:, 128:] * 2.0**-7], dim=1)
    q, sf = F.per_block_cast_to_fp8(x)
    assert torch.equal(sf, torch.tensor([[2.0**3, 2.0**-7]]))
    assert torch.equal(q.float(), codes)
    # ragged shape: padded with zeros, cut back; an all-zero block gets the clamp's scale
    xr = torch.zeros(130, 140)
    xr[:128, :128] = codes[:, :128]
    qr, sfr = F.per_block_cast_to_fp8(xr)
    assert qr.shape == (130, 140) and sfr.shape == (2, 2)
    assert sfr[0, 0].item() == 1.0 and sfr[1, 1].item() == 2.0**-22  # ceil_to_ue8m0(1e-4 / 448)
    assert torch.equal(qr.float(), xr)


def test_input_to_int8_truncates_toward_zero():
    # amax = 127 * 0.5: the multiplier is exactly 2, the conversion drops the fraction
    x = torch.tensor([[63.5, -63.5, 0.2, -0.2, 0.74, -0.74, 0.99, 31.0]])
    q, inv = I.input_to_int8(x)
    assert q.dtype == torch.int8 and inv.item() == 0.5
    assert q.tolist() == [[127, -127, 0, 0, 1, -1, 1, 62]]


def test_dispatch_names():
    assert F.dispatch_w8a8_block_fp8_linear() is F.cutlass_w8a8_block_fp8_linear_with_fallback
    assert F.cutlass_w8a8_block_fp8_linear_with_fallback is F.w8a8_block_fp8_linear
    assert callable(F.deepgemm_w8a8_block_fp8_linear_with_fallback)
    # no GPU here (or no library): the predicates say so instead of raising
    assert F.cutlass_fp8_supported() in (True, False)
    assert F.cutlass_block_fp8_supported() == F.cutlass_fp8_supported()


def test_convert_to_channelwise_and_dequantize():
    from sglang_amd.quantization import utils as U

    s = torch.tensor([0.5, 0.25, 2.0])
    got = U.convert_to_channelwise(s, [2, 1, 3])
    assert got.shape == (6, 1) and got.dtype == torch.float32
    assert got.view(-1).tolist() == [0.5, 0.5, 0.25, 2.0, 2.0, 2.0]
    scalar = U.convert_to_channelwise(torch.tensor(0.125), [2, 2])
    assert scalar.shape == (4, 1) and scalar.view(-1).tolist() == [0.125] * 4
    assert U.all_close_1d(torch.tensor([1.0, 1.0, 1.0])) and not U.all_close_1d(torch.tensor([1.0, 1.5]))
    codes = e4m3_codes((4, 8), seed=7)
    assert torch.equal(U.per_tensor_dequantize(codes.to(FP8), 0.5), (codes * 0.5).half())


def test_fp8_process_weights_after_loading():
    from sglang_amd.quantization import fp8 as P

    # 16-bit checkpoint: channel c holds codes * 2^-c with a 448 in it: scale 2^-c, the codes back
    codes = e4m3_codes((3, 64), seed=8)
    codes[:, 0] = 448.0
    w = (codes * torch.tensor([[1.0], [0.5], [0.25]])).to(torch.bfloat16)
    wt, scale, in_scale = P.process_weights_after_loading(w, is_checkpoint_fp8_serialized=False)
    assert wt.shape == (64, 3) and wt.stride(0) == 1 and in_scale is None
    assert scale.shape == (3, 1) and scale.view(-1).tolist() == [1.0, 0.5, 0.25]
    assert torch.equal(wt.t().float(), codes)
    # an all-zero channel: eps keeps the division defined
    q0, s0 = P.quantize_weight_per_channel(torch.zeros(1, 16))
    assert s0.item() == (torch.tensor(1e-10) / 448).item() and torch.equal(q0.float(), torch.zeros(1, 16))
    # FP8 checkpoint, two fused shards, static activations
    q = codes.to(FP8)
    wt2, scale2, in2 = P.process_weights_after_loading(q, torch.tensor([0.5, 2.0]), [1, 2], input_scale=torch.tensor([0.1, 0.3]),
                                                       static_activations=True)
    assert wt2.shape == (64, 3) and scale2.view(-1).tolist() == [0.5, 2.0, 2.0] and abs(in2.item() - 0.3) < 1e-7
    # block quantization: nothing to do
    ws = torch.ones(1, 1)
    assert P.process_weights_after_loading(q, ws, block_quant=True) == (q, ws, None)


def test_pow2_scale_check_rejects_other_scales():
    """w8a8_block_fp8_matmul_deepgemm reads only the exponents of the weight's block scales where the matrix
    instruction applies them: scales with mantissa bits (a weight that skipped requant_weight_ue8m0_inplace) must
    raise instead of being rounded down on some batch sizes and used in full on others."""
    from sglang_amd.quantization.fp8_kernel import check_pow2_scales

    check_pow2_scales(torch.tensor([[1.0, 0.5], [2.0**-20, 8.0]]))
    for bad in ([[1.0, 0.75]], [[3e-4, 1.0]], [[0.0, 1.0]], [[-2.0, 1.0]]):
        with pytest.raises(ValueError, match="powers of two"):
            check_pow2_scales(torch.tensor(bad))
    # ceil_to_ue8m0 is what makes a scale pass
    check_pow2_scales(F.ceil_to_ue8m0(torch.tensor([[3e-4, 0.75]])))
