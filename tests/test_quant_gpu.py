"""GPU parity of the quantization kernels against the CPU oracle: FP8 codes, INT8
codes and fp32 scales must be bit-identical.  Everything goes through the
operator wrappers, i.e. through the C ABI of libsglq.so."""
import pytest
import torch

from helpers import assert_bits_equal, fp8_bits
from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def say(*a):
    print(*a, flush=True)


def group_quant_gpu(x, group, column_major=False, tma=False, eps=1e-10):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    return sglang_per_token_group_quant_fp8(x, group, eps=eps, column_major_scales=column_major, scale_tma_aligned=tma)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 128), (3, 256), (127, 512), (256, 7168), (1000, 1536), (33, 16384)])
def test_group_quant_fp8_bit_exact(gpu, dtype, shape):
    say("group_quant", dtype, shape)
    m, k = shape
    x = O.gen_activation(m, k, seed=m * 7 + k, outliers=True).float()
    if m > 2:
        x[1, :128] = 0
        x[2] *= 1e-5
        x[0, 1:9] = torch.tensor([-0.0, 0.0, -0.0, -1e-30, 1e-30, -0.0, 0.0, -0.0])  # signed zeros survive
    x = x.to(dtype)
    q_ref, s_ref = O.per_token_group_quant_fp8(x, 128)
    for cm, tma in ((False, False), (True, False), (True, True)):
        q, s = group_quant_gpu(x.to(gpu), 128, cm, tma)
        torch.cuda.synchronize()
        if cm:
            assert s.stride(0) == 1
        assert_bits_equal(s, s_ref, f"scales cm={cm} tma={tma}")
        assert_bits_equal(q, q_ref, f"codes cm={cm} tma={tma}")


@pytest.mark.parametrize("group", [8, 16, 32, 64, 128])
def test_group_quant_fp8_group_sizes(gpu, group):
    say("group_quant group", group)
    x = O.gen_activation(129, 1024, seed=group, outliers=True)
    q_ref, s_ref = O.per_token_group_quant_fp8(x, group)
    q, s = group_quant_gpu(x.to(gpu), group)
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")
    q, s = group_quant_gpu(x.to(gpu), group, column_major=True)
    assert_bits_equal(s, s_ref, "scales (column-major)")


def test_group_quant_fp8_every_code_and_tie(gpu):
    """fp32 groups whose scale is exactly 1 (absmax 448): every e4m3fn value, every
    midpoint between neighbours and the floats next to each midpoint."""
    say("group_quant conversions")
    codes = torch.arange(256, dtype=torch.uint8)
    vals = O.e4m3fn_decode(codes)
    pos = torch.sort(vals[(~torch.isnan(vals)) & (vals >= 0)]).values.unique()
    mids = ((pos[:-1].double() + pos[1:].double()) / 2).float()
    cand = torch.cat([pos, mids, torch.nextafter(mids, torch.tensor(0.0)), torch.nextafter(mids, torch.tensor(1e9))])
    cand = torch.cat([cand, -cand])
    n = (cand.numel() + 126) // 127
    x = torch.zeros(n, 128)
    x[:, 0] = 448.0
    flat = torch.zeros(n * 127)
    flat[: cand.numel()] = cand
    x[:, 1:] = flat.reshape(n, 127)
    q_ref, s_ref = O.per_token_group_quant_fp8(x, 128)
    assert float(s_ref.min()) == 1.0 and float(s_ref.max()) == 1.0
    q, s = group_quant_gpu(x.to(gpu), 128)
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")


def test_group_quant_fp8_custom_bounds(gpu):
    """Bounds other than +-448 take the clamping variant of the kernel."""
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8

    say("group_quant custom bounds")
    x = O.gen_activation(65, 512, seed=12, outliers=True)
    x[0, 3] = -0.0
    for lo, hi in ((-224.0, 224.0), (-448.0, 240.0)):
        q_ref, s_ref = O.per_token_group_quant_8bit(x, 128, 1e-10, lo, hi, FP8)
        xg = x.to(gpu)
        q = torch.empty_like(xg, dtype=FP8)
        s = torch.empty((65, 4), dtype=torch.float32, device=gpu)
        sgl_per_token_group_quant_fp8(xg, q, s, 128, 1e-10, lo, hi, False)
        assert_bits_equal(s, s_ref, f"scales {lo},{hi}")
        assert_bits_equal(q, q_ref, f"codes {lo},{hi}")


def test_group_quant_int8_bit_exact(gpu):
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_int8

    say("group_quant int8")
    x = O.gen_activation(77, 1024, seed=3, outliers=True)
    q_ref, s_ref = O.per_token_group_quant_8bit(x, 128, 1e-10, -128.0, 127.0, torch.int8)
    xg = x.to(gpu)
    q = torch.empty_like(xg, dtype=torch.int8)
    s = torch.empty((77, 8), dtype=torch.float32, device=gpu)
    sgl_per_token_group_quant_int8(xg, q, s, 128, 1e-10, -128.0, 127.0)
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")


@pytest.mark.parametrize("to_int8", [False, True], ids=["fp8", "int8"])
@pytest.mark.parametrize("group", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("shape", [(127, 256), (512, 1024), (128, 4096)])
def test_group_quant_grid_of_the_reference_test(gpu, shape, group, to_int8):
    """The grid of sgl-kernel/tests/test_per_token_group_quant_8bit.py:266-279 (token counts and
    hidden sizes thinned): every group size, both code types, row-major scales and the two
    column-major buffers of create_per_token_group_quant_fp8_output_scale written by the op itself."""
    from sglang_amd.quantization.fp8_kernel import create_per_token_group_quant_fp8_output_scale
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8, sgl_per_token_group_quant_int8

    say("group_quant grid", shape, group, to_int8)
    m, k = shape
    x = O.gen_activation(m, k, seed=m + k + group, outliers=True)
    lo, hi = (-128.0, 127.0) if to_int8 else (-448.0, 448.0)
    q_dtype = torch.int8 if to_int8 else torch.float8_e4m3fn
    q_ref, s_ref = O.per_token_group_quant_8bit(x, group, 1e-10, lo, hi, q_dtype)
    xg = x.to(gpu)
    for cm, tma in ((False, False), (True, False), (True, True)):
        q = torch.empty_like(xg, dtype=q_dtype)
        s = create_per_token_group_quant_fp8_output_scale(xg.shape, gpu, group, column_major_scales=cm, scale_tma_aligned=tma,
                                                          scale_ue8m0=False)
        if to_int8:
            sgl_per_token_group_quant_int8(xg, q, s, group, 1e-10, lo, hi)
        else:
            sgl_per_token_group_quant_fp8(xg, q, s, group, 1e-10, lo, hi, False)
        assert_bits_equal(s, s_ref, f"scales cm={cm} tma={tma}")
        assert_bits_equal(q, q_ref, f"codes cm={cm} tma={tma}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 4096), (16, 4096), (128, 4096), (1024, 4096), (5, 1000), (7, 1003), (3, 14336),
                                   (2, 20000), (9, 512), (300, 256), (4, 8)])
def test_token_quant_int8_bit_exact(gpu, dtype, shape):
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8

    say("token_quant_int8", dtype, shape)
    m, k = shape
    x = O.gen_activation(m, k, seed=m + k).float()
    if m > 2:
        x[1] = 0
        x[2, 0] = 0.5 * x[2].abs().max()  # an exact .5 product when absmax/127 is a power of two is rare; force ties below
    x = x.to(dtype)
    q_ref, s_ref = O.per_token_quant_int8(x)
    q, s = per_token_quant_int8(x.to(gpu))
    assert tuple(s.shape) == (m, 1)
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")


def test_token_quant_int8_ties_round_away(gpu):
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8

    say("token_quant_int8 ties")
    k = torch.arange(-127, 128, dtype=torch.float32)
    row = torch.cat([k, k[:-1] + 0.5, torch.zeros(6)]).reshape(1, -1)  # 255 + 254 + 6 = 515 -> pad to 520
    row = torch.cat([row, torch.zeros(1, 5)], dim=1)
    q_ref, s_ref = O.per_token_quant_int8(row)
    assert s_ref.item() == 1.0
    q, s = per_token_quant_int8(row.to(gpu))
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")
    assert q[0, 255:259].tolist() == [-127, -126, -125, -124]  # -126.5 -> -127 ...


def test_token_quant_int8_row_sum(gpu):
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8

    x = O.gen_activation(33, 4096, seed=9)
    q, s, rs = per_token_quant_int8(x.to(gpu), cal_sum=True)
    # summation order is not defined by the reference (a Triton reduction): tolerance only
    torch.testing.assert_close(rs.float().cpu(), x.float().sum(-1), rtol=2e-2, atol=0.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 4096), (32, 4096), (256, 14336), (2048, 4096), (5, 1368), (130, 512), (3, 24576), (2, 8)])
def test_token_quant_fp8_bit_exact(gpu, dtype, shape):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_quant_fp8

    say("token_quant_fp8", dtype, shape)
    m, k = shape
    x = O.gen_activation(m, k, seed=3 * m + k).float()
    if m > 1:
        x[1] = 0  # zero row: scale 0, codes 0
    x = x.to(dtype)
    q_ref, s_ref = O.per_token_quant_fp8(x)
    q, s = sglang_per_token_quant_fp8(x.to(gpu))
    assert tuple(s.shape) == (m, 1)
    assert_bits_equal(s, s_ref, "scales")
    assert_bits_equal(q, q_ref, "codes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 8), (3, 7), (128, 512), (512, 4096), (33, 1003), (2048, 14336)])
def test_tensor_quant_fp8_bit_exact(gpu, dtype, shape):
    """sgl_per_tensor_quant_fp8, dynamic and static, against the oracle bit for bit (shapes of
    sgl-kernel/tests/test_per_tensor_quant_fp8.py:40-43 plus lengths that are not a multiple of 8)."""
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant

    say("tensor_quant", dtype, shape)
    m, k = shape
    x = (O.gen_activation(m, k, seed=m + 3 * k, outliers=True).float() * 1.7).to(dtype)
    q_ref, s_ref = O.per_tensor_quant_fp8(x)
    q, s = scaled_fp8_quant(x.to(gpu))
    assert_bits_equal(s, s_ref, "dynamic scale")
    assert_bits_equal(q, q_ref, "dynamic codes")
    static = torch.tensor([0.0371], dtype=torch.float32)
    q_ref, _ = O.per_tensor_quant_fp8(x, static)
    q, s = scaled_fp8_quant(x.to(gpu), static.to(gpu))
    assert_bits_equal(q, q_ref, "static codes")
    assert s.item() == static.item()


def test_tensor_quant_fp8_unaligned_zero_and_padding(gpu):
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant
    from sglang_amd.sgl_kernel import sgl_per_tensor_quant_fp8

    # a view that starts 2 bytes into an allocation: the element-wise kernels
    base = O.gen_activation(5, 1001, seed=9).to(torch.bfloat16).flatten()
    xg = base.to(gpu)[1:]
    q = torch.empty(xg.numel() + 1, dtype=FP8, device=gpu)[1:]
    s = torch.zeros(1, dtype=torch.float32, device=gpu)
    sgl_per_tensor_quant_fp8(xg, q, s, False)
    q_ref, s_ref = O.per_tensor_quant_fp8(base[1:])
    assert_bits_equal(s, s_ref, "scale, unaligned")
    assert_bits_equal(q, q_ref, "codes, unaligned")
    # all-zero tensor, dynamic: scale 0 and the +448 codes of the reference's fminf / fmaxf clamp
    z = torch.zeros((4, 64), dtype=torch.float16, device=gpu)
    q, s = scaled_fp8_quant(z)
    assert s.item() == 0.0 and fp8_bits(q).unique().tolist() == [0x7E]
    # the scale is merged with an atomic max: a larger value already in the buffer survives
    x = torch.ones((2, 16), dtype=torch.bfloat16, device=gpu)
    q = torch.empty((2, 16), dtype=FP8, device=gpu)
    s = torch.full((1,), 2.0, dtype=torch.float32, device=gpu)
    sgl_per_tensor_quant_fp8(x, q, s, False)
    assert s.item() == 2.0 and q.float().unique().tolist() == [0.5]
    # num_token_padding only enlarges the output
    x = O.gen_activation(3, 64, seed=1).to(torch.bfloat16)
    q, s = scaled_fp8_quant(x.to(gpu), num_token_padding=17)
    assert q.shape == (17, 64)
    q_ref, s_ref = O.per_tensor_quant_fp8(x)
    assert_bits_equal(q[:3], q_ref, "codes, padded output")
    # per-token dynamic branch of the same helper
    q, s = scaled_fp8_quant(x.to(gpu), use_per_token_if_dynamic=True)
    q_ref, s_ref = O.per_token_quant_fp8(x)
    assert_bits_equal(q, q_ref, "per-token codes")
    assert_bits_equal(s, s_ref, "per-token scales")


@pytest.mark.parametrize("dtype", [torch.half, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("num_tokens", [7, 83, 2048])
@pytest.mark.parametrize("d", [512, 4096, 5120, 13824])
def test_static_quant_fp8_bit_exact(gpu, dtype, num_tokens, d):
    """static_quant_fp8 on the grid of the reference's test (python/sglang/test/test_block_fp8.py:119-159:
    uniform inputs, scale = max / 448 in the input's dtype), bit for bit against the oracle, with
    and without the repeated scale."""
    from sglang_amd.quantization.fp8_kernel import static_quant_fp8

    say("static_quant", dtype, num_tokens, d)
    g = torch.Generator().manual_seed(0)
    x = torch.rand((num_tokens, d), generator=g).to(dtype)
    x_s = x.max() / 448.0
    q_ref, s_ref = O.static_quant_fp8(x, x_s, repeat_scale=True)
    xg, sg = x.to(gpu), x_s.to(gpu)
    q, s = static_quant_fp8(xg, sg, repeat_scale=True)
    assert q.dtype == FP8 and q.shape == x.shape and tuple(s.shape) == (num_tokens, 1) and s.dtype == torch.float32
    assert_bits_equal(q, q_ref, "codes")
    assert_bits_equal(s, s_ref, "repeated scale")
    q, s = static_quant_fp8(xg, sg)
    assert s is sg
    assert_bits_equal(q, q_ref, "codes, scale not repeated")


def test_static_quant_fp8_shapes_and_errors(gpu):
    from sglang_amd.quantization.fp8_kernel import static_quant_fp8

    # ndim 3, a length that is not a multiple of 8, values beyond the range
    x = (O.gen_activation(6, 203, seed=4, outliers=True).float() * 40).reshape(2, 3, 203).contiguous()
    scale = torch.tensor([0.25])
    q_ref, s_ref = O.static_quant_fp8(x, scale, repeat_scale=True)
    q, s = static_quant_fp8(x.to(gpu), scale.to(gpu), repeat_scale=True)
    assert q.shape == x.shape and tuple(s.shape) == (6, 1)
    assert_bits_equal(q, q_ref, "codes, 3-D input")
    assert_bits_equal(s, s_ref, "repeated scale, 3-D input")
    assert float(q.float().abs().max()) == 448.0
    with pytest.raises(AssertionError, match="not contiguous"):
        static_quant_fp8(x.to(gpu).transpose(0, 1), scale.to(gpu))
    with pytest.raises(AssertionError, match="per-tensor"):
        static_quant_fp8(x.to(gpu), torch.ones(2, device=gpu))
    q, s = static_quant_fp8(torch.empty((0, 64), device=gpu, dtype=torch.bfloat16), scale.to(gpu), repeat_scale=True)
    assert q.shape == (0, 64) and s.shape == (0, 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 128), (7, 512), (83, 1536), (130, 7168), (2048, 640)])
def test_group_quant_ue8m0_bit_exact(gpu, dtype, shape):
    """scale_ue8m0: codes and the packed exponent words (the reference's int32 tensor, padding
    words included) bit for bit against the oracle."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    say("group_quant ue8m0", dtype, shape)
    m, k = shape
    x = (O.gen_activation(m, k, seed=m + k, outliers=True).float() * torch.logspace(-4, 3, m).unsqueeze(1)).to(dtype)
    if m > 2:
        x[2, :128] = 0
    q_ref, exps_ref, packed_ref = O.per_token_group_quant_fp8_ue8m0(x)
    q, s = sglang_per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    assert s.dtype == torch.int32 and tuple(s.shape) == tuple(packed_ref.shape) and s.stride() == packed_ref.stride()
    assert_bits_equal(q, q_ref, "codes")
    assert torch.equal(s.cpu(), packed_ref), "packed exponents"
    # dequantized with the power-of-two scales: within half an e4m3 step of the input
    scale = torch.pow(2.0, exps_ref.float() - 127).repeat_interleave(128, dim=1)
    err = (q.cpu().float() * scale - x.float()).abs()
    assert bool((err <= 0.0625 * x.float().abs() + scale * 2.0 ** -10).all())


def test_group_quant_ue8m0_argument_checks(gpu):
    from sglang_amd.sgl_kernel import sgl_per_token_group_quant_fp8

    x = torch.randn((8, 256), device=gpu, dtype=torch.bfloat16)
    q = torch.empty((8, 256), device=gpu, dtype=FP8)
    row_major = torch.zeros((8, 1), device=gpu, dtype=torch.int32)
    s = torch.zeros((1, 8), device=gpu, dtype=torch.int32).t()
    with pytest.raises(RuntimeError, match="Int32"):
        sgl_per_token_group_quant_fp8(x, q, torch.zeros((2, 8), device=gpu).t(), 128, 1e-10, -448.0, 448.0, True)
    with pytest.raises(NotImplementedError, match="group_size 128"):
        sgl_per_token_group_quant_fp8(x, q, s, 64, 1e-10, -448.0, 448.0, True)
    sgl_per_token_group_quant_fp8(x, q, s, 128, 1e-10, -448.0, 448.0, True)
    _, _, packed = O.per_token_group_quant_fp8_ue8m0(x.cpu())
    assert torch.equal(s.cpu(), packed)
    del row_major


def test_tensor_quant_full_size_properties(gpu):
    """8192 x 16384 (the largest activation of the configurations): quantizing the dequantized
    tensor with the same static scale reproduces the codes; the maximum code is 448."""
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant

    g = torch.Generator(device=gpu).manual_seed(7)
    x = torch.randn((8192, 16384), generator=g, device=gpu, dtype=torch.bfloat16)
    q, s = scaled_fp8_quant(x)
    assert s.item() == (x.float().abs().max() / 448).item()
    assert float(q[:64].float().abs().max()) <= 448.0 and int((fp8_bits(q) & 0x7F).max()) == 0x7E
    deq = (q.float() * s).to(torch.float32)
    q2, _ = scaled_fp8_quant(deq, s)
    assert torch.equal(fp8_bits(q2), fp8_bits(q))


def test_quant_empty_inputs(gpu):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8, sglang_per_token_quant_fp8
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8

    x = torch.empty((0, 256), dtype=torch.bfloat16, device=gpu)
    q, s = sglang_per_token_group_quant_fp8(x, 128)
    assert tuple(q.shape) == (0, 256) and tuple(s.shape) == (0, 2)
    q, s = per_token_quant_int8(x)
    assert tuple(q.shape) == (0, 256) and tuple(s.shape) == (0, 1)
    q, s = sglang_per_token_quant_fp8(x)
    assert tuple(q.shape) == (0, 256)


def test_group_quant_full_size_properties(gpu):
    """Largest configuration (8192 x 16384): idempotence of the codes under
    re-quantization of the dequantized tensor, max code 448 in every group, and
    bit-exactness on a row sample."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    say("group_quant full size")
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((8192, 16384), generator=g, device=gpu, dtype=torch.float32).to(torch.bfloat16)
    q, s = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
    qa = q.view(8192, 128, 128).float().abs().amax(dim=2)
    assert bool((qa == 448.0).all())
    rows = torch.tensor([0, 1, 17, 4095, 4096, 8191])
    q_ref, s_ref = O.per_token_group_quant_fp8(x[rows.to(gpu)].cpu(), 128)
    assert_bits_equal(q[rows.to(gpu)], q_ref, "codes (row sample)")
    assert_bits_equal(s[rows.to(gpu)].contiguous(), s_ref, "scales (row sample)")
    # dequantize (exactly representable in fp32) and quantize again: same codes, same scales
    deq = (q.view(8192, 128, 128).float() * s.contiguous().view(8192, 128, 1)).view(8192, 16384)
    q2, s2 = sglang_per_token_group_quant_fp8(deq, 128, column_major_scales=True)
    assert bool((s2 == s).all())
    assert bool((q2.view(torch.uint8) == q.view(torch.uint8)).all())


@pytest.mark.parametrize("shape", [(1, 128), (5, 384), (33, 1024), (257, 7168)])
def test_quant_kernels_write_only_their_outputs(gpu, shape):
    """Codes and scales land in windows of sentinel-filled buffers (guard bytes before and after):
    every quantization entry point, through the C ABI, must leave the guards alone."""
    from sglang_amd import _lib

    lib = _lib.load()
    m, k = shape
    say("quant output windows", shape)
    x = O.gen_activation(m, k, seed=m * 7 + k, outliers=True).to(torch.bfloat16).to(gpu)
    st = _lib.stream_ptr(gpu)
    G = 64  # guard elements on each side

    def window(numel, dtype, fill):
        buf = torch.full((numel + 2 * G,), fill, dtype=dtype, device=gpu)
        return buf, buf[G:G + numel]

    def guards_intact(buf, numel, fill):
        host = buf.cpu()
        return bool((host[:G] == fill).all()) and bool((host[G + numel:] == fill).all())

    groups = k // 128
    cases = []
    # per-token-group FP8, row-major and column-major (padded) scales; INT8 twin
    for col_major in (False, True):
        qb, q = window(m * k, torch.uint8, 0xAB)
        ld = (m + 3) // 4 * 4
        sb, s = window(ld * groups if col_major else m * groups, torch.float32, -7.0)
        sr, sc = (1, ld) if col_major else (groups, 1)
        rc = lib.sglq_per_token_group_quant_fp8(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), m, k, 128, sr, sc, 1e-10, -448.0, 448.0, st)
        cases.append(("group fp8", rc, qb, m * k, 0xAB, sb, s.numel(), -7.0))
    qb, q = window(m * k, torch.uint8, 0xAB)
    sb, s = window(m * groups, torch.float32, -7.0)
    rc = lib.sglq_per_token_group_quant_int8(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), m, k, 128, groups, 1, 1e-10, -128.0, 127.0, st)
    cases.append(("group int8", rc, qb, m * k, 0xAB, sb, m * groups, -7.0))
    # UE8M0: packed int32 words, column stride ceil4(M)
    qb, q = window(m * k, torch.uint8, 0xAB)
    ld = (m + 3) // 4 * 4
    words = (groups + 3) // 4
    sb, s = window(ld * words, torch.int32, 0x55555555)
    rc = lib.sglq_per_token_group_quant_fp8_ue8m0(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), m, k, ld, 1e-10, -448.0, 448.0, st)
    cases.append(("ue8m0", rc, qb, m * k, 0xAB, sb, ld * words, 0x55555555))
    # per-token FP8 / INT8
    for name, fn in (("token fp8", lambda q, s: lib.sglq_per_token_quant_fp8(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), m, k, st)),
                     ("token int8", lambda q, s: lib.sglq_per_token_quant_int8(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), None, m, k, st))):
        qb, q = window(m * k, torch.uint8, 0xAB)
        sb, s = window(m, torch.float32, -7.0)
        cases.append((name, fn(q, s), qb, m * k, 0xAB, sb, m, -7.0))
    # per-tensor dynamic / static, static with the repeated scale
    qb, q = window(m * k, torch.uint8, 0xAB)
    sb, s = window(1, torch.float32, -7.0)
    s.zero_()
    rc = lib.sglq_per_tensor_quant_fp8(x.data_ptr(), 0, q.data_ptr(), s.data_ptr(), m * k, 0, st)
    cases.append(("tensor dynamic", rc, qb, m * k, 0xAB, sb, 1, -7.0))
    qb, q = window(m * k, torch.uint8, 0xAB)
    sb, s = window(m, torch.float32, -7.0)
    scale = torch.tensor([0.05], device=gpu)
    rc = lib.sglq_static_quant_fp8(x.data_ptr(), 0, q.data_ptr(), scale.data_ptr(), s.data_ptr(), m, k, st)
    cases.append(("static repeat", rc, qb, m * k, 0xAB, sb, m, -7.0))
    torch.cuda.synchronize()
    for name, rc, qb, qn, qfill, sb, sn, sfill in cases:
        assert rc == 0, (name, lib.sglq_last_error())
        assert guards_intact(qb, qn, qfill), f"{name}: codes written outside the output"
        assert guards_intact(sb, sn, sfill), f"{name}: scales written outside the output"
    assert scale.item() == torch.tensor(0.05).item()
