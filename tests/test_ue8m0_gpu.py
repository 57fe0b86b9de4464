"""The block-scaled FP8 path with power-of-two (UE8M0) scales: the quantization that stores such scales as
fp32, the GEMM whose matrix instructions apply them, and the linear that chains both (the reference's
deepgemm_w8a8_block_fp8_linear_with_fallback, fp8_utils.py:214-258, whose GEMM is a third-party kernel
there).  Codes and scales bit-exact against the oracle, bf16 outputs within rtol 1e-2 / atol 1e-2."""
import pytest
import torch

from helpers import rows_per_tile
from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
RTOL, ATOL = 1e-2, 1e-2


def say(*a):
    print(*a, flush=True)


def pow2_block_case(m, n, k, seed):
    """Codes and power-of-two scales as the path produces them: activations through the oracle's UE8M0
    quantization, the weight block-quantized with ceil-to-power-of-two scales (fp8_utils.py:468-486)."""
    x = O.gen_activation(m, k, seed=seed, outliers=True)
    xq, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
    xs = torch.pow(2.0, exps.float() - 127.0)
    w = O.gen_weight(n, k, seed=seed + 1).float()
    np_, kp = (n + 127) // 128 * 128, k
    wp = torch.zeros((np_, kp))
    wp[:n] = w
    blocks = wp.view(np_ // 128, 128, kp // 128, 128)
    amax = blocks.abs().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    y = amax / 448.0
    bits = y.view(torch.int32)
    sf = (((bits >> 23) + ((bits & 0x7FFFFF) != 0).to(torch.int32)) << 23).view(torch.float32)
    wq = (blocks * (1.0 / sf)).to(FP8).view(np_, kp)[:n].contiguous()
    return x, xq, xs, wq, sf.view(np_ // 128, kp // 128)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 128), (7, 512), (83, 1536), (130, 7168), (2048, 640)])
@pytest.mark.parametrize("column_major", [True, False])
def test_group_quant_pow2_bit_exact(gpu, dtype, shape, column_major):
    """Codes bit for bit the oracle's UE8M0 codes; scales exactly 2^(exponent byte - 127), in the layout asked for."""
    from sglang_amd.quantization.fp8_kernel import per_token_group_quant_fp8_pow2

    say("group_quant pow2", dtype, shape, column_major)
    m, k = shape
    x = (O.gen_activation(m, k, seed=m + k, outliers=True).float() * torch.logspace(-4, 3, m).unsqueeze(1)).to(dtype)
    if m > 2:
        x[2, :128] = 0
    q_ref, exps_ref, _ = O.per_token_group_quant_fp8_ue8m0(x)
    q, s = per_token_group_quant_fp8_pow2(x.to(gpu), 128, column_major_scales=column_major)
    assert s.dtype == torch.float32 and tuple(s.shape) == (m, k // 128)
    if m > 1 and k > 128:
        assert (s.stride(0) == 1) == column_major and (s.stride(1) == 1) == (not column_major)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8)), "codes"
    assert torch.equal(s.cpu(), torch.pow(2.0, exps_ref.float() - 127.0)), "scales"


def test_group_quant_pow2_large_input_matches_the_packed_kernel(gpu):
    """An input of 128 MiB and more takes the non-temporal loads: same codes and exponents as the packed-scale kernel."""
    from sglang_amd.quantization.fp8_kernel import per_token_group_quant_fp8_pow2, sglang_per_token_group_quant_fp8, unpack_ue8m0_scales

    m, k = 4096, 16384
    x = torch.randn((m, k), device=gpu, dtype=torch.bfloat16)
    q0, s0 = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    q1, s1 = per_token_group_quant_fp8_pow2(x, 128)
    assert torch.equal(q0.view(torch.uint8), q1.view(torch.uint8))
    assert torch.equal(unpack_ue8m0_scales(s0, k // 128), s1.contiguous())


# (M, N, K), forced tile code (0 = the rules' choice), whether the scaled-MFMA kernels must have run
UE8M0_CASES = [
    ((1, 512, 512), 0, False), ((64, 4096, 1024), 0, False), ((128, 2048, 1024), 0, False),
    ((300, 2112, 1536), 258, True), ((300, 2112, 1536), 130, True), ((513, 640, 2048), 192, True),
    ((513, 704, 2048), 224, True), ((513, 512, 2048), 257, True), ((1000, 256, 1536), 130, True),
    ((2048, 2112, 1024), 0, True), ((4096, 4096, 512), 0, True), ((1024, 7168, 2048), 0, True),
]


@pytest.mark.parametrize("mnk,tile,hw", UE8M0_CASES)
def test_fp8_blockwise_scaled_mm_ue8m0(gpu, mnk, tile, hw):
    """Against the oracle (float64 accumulation) on rows of every row tile, and against the fp32-scale entry
    point, which computes the same sums in another order."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    say("fp8_blockwise ue8m0", mnk, "tile", tile)
    m, n, k = mnk
    lib = _lib.load()
    _, xq, xs, wq, ws = pow2_block_case(m, n, k, seed=m + n + k)
    rows = rows_per_tile(m, 48)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    lib.sglq_debug_force_tile(tile)
    try:
        out = fp8_blockwise_scaled_mm_ue8m0(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
        assert bool(lib.sglq_debug_last_gemm_hw_scaled()) == hw, lib.sglq_debug_last_gemm_kernel().decode()
        plain = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
        assert not lib.sglq_debug_last_gemm_hw_scaled()
    finally:
        lib.sglq_debug_force_tile(0)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (m, n)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(out.float(), plain.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("splits", [2, 4])
def test_fp8_blockwise_scaled_mm_ue8m0_split_k(gpu, splits):
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    lib = _lib.load()
    for (m, n, k), tile in (((512, 640, 4096), 258), ((300, 384, 2048), 130)):
        say("fp8_blockwise ue8m0 split-K", (m, n, k), tile, splits)
        _, xq, xs, wq, ws = pow2_block_case(m, n, k, seed=m + n + k + splits)
        rows = rows_per_tile(m, 32)
        ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
        lib.sglq_debug_force_tile(tile)
        lib.sglq_debug_force_splits(splits)
        try:
            out = fp8_blockwise_scaled_mm_ue8m0(xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), torch.bfloat16)
            assert lib.sglq_debug_last_gemm_hw_scaled() and "splitk" in lib.sglq_debug_last_gemm_kernel().decode()
        finally:
            lib.sglq_debug_force_tile(0)
            lib.sglq_debug_force_splits(0)
        torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


def test_fp8_blockwise_scaled_mm_ue8m0_fp16_output_runs_the_plain_kernels(gpu):
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    m, n, k = 600, 2112, 1024
    _, xq, xs, wq, ws = pow2_block_case(m, n, k, seed=11)
    rows = rows_per_tile(m, 24)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    out = fp8_blockwise_scaled_mm_ue8m0(xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), torch.float16)
    assert not _lib.load().sglq_debug_last_gemm_hw_scaled()
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


def pack_codes(exps, gpu):
    """UE8M0 codes [M, K/128] as the reference's quantization stores them with scale_ue8m0=True (fp8_kernel.py:308-320):
    int32 words of four codes, column-major with the rows padded to a multiple of four."""
    m, nkb = exps.shape
    words = -(-nkb // 4)
    padded = torch.zeros((m, 4 * words), dtype=torch.int64)
    padded[:, :nkb] = exps.to(torch.int64)
    shifts = torch.tensor([0, 8, 16, 24], dtype=torch.int64)
    packed = (padded.view(m, words, 4) << shifts).sum(dim=-1)
    packed = torch.where(packed >= 2**31, packed - 2**32, packed).to(torch.int32)
    store = torch.full((words, -(-m // 4) * 4), 0x7F7F7F7F, dtype=torch.int32, device=gpu)
    store[:, :m] = packed.t().to(gpu)
    return store.t()[:m, :]


PACKED_CASES = UE8M0_CASES + [
    ((130, 640, 640), 130, True), ((257, 512, 896), 258, True), ((515, 448, 2176), 224, True), ((2050, 2112, 7168), 0, True),
    ((33, 1024, 640), 0, False), ((511, 4096, 7168), 0, None), ((96, 7168, 2048), 0, None), ((4096, 256, 256), 0, False),
]


@pytest.mark.parametrize("mnk,tile,hw", PACKED_CASES)
def test_fp8_blockwise_scaled_mm_ue8m0_packed_scales(gpu, mnk, tile, hw):
    """The entry point that takes the activation scales as packed UE8M0 words gives the bits of the one that takes
    them as fp32 powers of two, on the kernels that read the words themselves and on those that get them
    expanded first (K blocks that do not fill the last word, rows that do not fill the padding)."""
    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul_deepgemm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    say("fp8_blockwise ue8m0 packed", mnk, "tile", tile)
    m, n, k = mnk
    lib = _lib.load()
    x = O.gen_activation(m, k, seed=m + n + k, outliers=True)
    _, xq, xs, wq, ws = pow2_block_case(m, n, k, seed=m + n + k)
    _, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
    packed = pack_codes(exps, gpu)
    assert packed.stride(0) == 1 and packed.stride(1) % 4 == 0
    lib.sglq_debug_force_tile(tile)
    try:
        want = fp8_blockwise_scaled_mm_ue8m0(xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), torch.bfloat16)
        want_kernel, want_hw = lib.sglq_debug_last_gemm_kernel().decode(), bool(lib.sglq_debug_last_gemm_hw_scaled())
        got = w8a8_block_fp8_matmul_deepgemm(xq.to(gpu), wq.to(gpu), packed, ws.to(gpu), [128, 128], torch.bfloat16)
        assert lib.sglq_debug_last_gemm_kernel().decode() == want_kernel and bool(lib.sglq_debug_last_gemm_hw_scaled()) == want_hw
        if hw is not None:
            assert want_hw == hw, want_kernel
    finally:
        lib.sglq_debug_force_tile(0)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), want_kernel


@pytest.mark.parametrize("splits", [2, 4])
def test_fp8_blockwise_scaled_mm_ue8m0_packed_scales_split_k(gpu, splits):
    """Work units that start in the middle of a word of four codes (K ranges of 6 and 3 K blocks)."""
    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul_deepgemm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    lib = _lib.load()
    for (m, n, k), tile in (((512, 640, 1536), 258), ((300, 384, 1536), 130), ((130, 256, 3072), 130)):
        say("fp8_blockwise ue8m0 packed split-K", (m, n, k), tile, splits)
        x = O.gen_activation(m, k, seed=m + n + k + splits, outliers=True)
        _, xq, xs, wq, ws = pow2_block_case(m, n, k, seed=m + n + k + splits)
        _, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
        lib.sglq_debug_force_tile(tile)
        lib.sglq_debug_force_splits(splits)
        try:
            want = fp8_blockwise_scaled_mm_ue8m0(xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), torch.bfloat16)
            assert lib.sglq_debug_last_gemm_hw_scaled() and "splitk" in lib.sglq_debug_last_gemm_kernel().decode()
            got = w8a8_block_fp8_matmul_deepgemm(xq.to(gpu), wq.to(gpu), pack_codes(exps, gpu), ws.to(gpu), [128, 128], torch.bfloat16)
            assert lib.sglq_debug_last_gemm_hw_scaled() and "splitk" in lib.sglq_debug_last_gemm_kernel().decode()
        finally:
            lib.sglq_debug_force_tile(0)
            lib.sglq_debug_force_splits(0)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_fp8_blockwise_scaled_mm_ue8m0_packed_checks_the_workspace(gpu):
    from sglang_amd import _lib
    from sglang_amd._lib import DTYPE_CODE

    lib = _lib.load()
    m, n, k = 64, 256, 512
    a = torch.zeros((m, k), device=gpu, dtype=torch.uint8)
    b = torch.zeros((n, k), device=gpu, dtype=torch.uint8)
    sa = torch.zeros((1, m), device=gpu, dtype=torch.int32)
    sb = torch.ones((2, 4), device=gpu)
    out = torch.empty((m, n), device=gpu, dtype=torch.bfloat16)
    small = torch.empty(512, device=gpu, dtype=torch.uint8)
    rc = lib.sglq_fp8_blockwise_scaled_mm_ue8m0_packed(a.data_ptr(), k, b.data_ptr(), k, sa.data_ptr(), 1, m, sb.data_ptr(), 1, 4,
                                                       out.data_ptr(), n, DTYPE_CODE[torch.bfloat16], m, n, k, small.data_ptr(), 512, 0)
    assert rc != 0 and b"workspace" in lib.sglq_last_error()
    rc = lib.sglq_fp8_blockwise_scaled_mm_ue8m0_packed(a.data_ptr(), k + 64, b.data_ptr(), k + 64, sa.data_ptr(), 1, m, sb.data_ptr(), 1, 4,
                                                       out.data_ptr(), n, DTYPE_CODE[torch.bfloat16], m, n, k - 64, small.data_ptr(), 512, 0)
    assert rc != 0


@pytest.mark.parametrize("m", [3, 200, 1030])
@pytest.mark.parametrize("with_bias", [False, True])
def test_deepgemm_linear(gpu, monkeypatch, m, with_bias):
    """deepgemm_w8a8_block_fp8_linear_with_fallback end to end against the oracle's quantization and GEMM, and
    w8a8_block_fp8_matmul_deepgemm on the packed int32 scales of scale_ue8m0=True."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8, w8a8_block_fp8_matmul_deepgemm
    import sglang_amd.quantization.fp8_utils as F
    from sglang_amd.quantization.fp8_utils import deepgemm_w8a8_block_fp8_linear_with_fallback, requant_weight_ue8m0_inplace

    monkeypatch.setattr(F, "DEEPGEMM_SCALE_UE8M0", True)
    n, k = 2112, 1536
    say("deepgemm linear", m, n, k, with_bias)
    x = O.gen_activation(m, k, seed=m, outliers=True)
    w0q, w0s = O.block_quant_weight(O.gen_weight(n, k, seed=m + 1))  # a checkpoint with ordinary fp32 block scales
    weight = torch.nn.Parameter(w0q.to(gpu), requires_grad=False)
    scale = torch.nn.Parameter(w0s.to(gpu), requires_grad=False)
    requant_weight_ue8m0_inplace(weight, scale, [128, 128])
    ws = scale.data.cpu()
    assert torch.equal(ws, torch.pow(2.0, torch.ceil(torch.log2(ws)))) and tuple(ws.shape) == tuple(w0s.shape)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(5)) * 0.1).to(torch.bfloat16) if with_bias else None
    out = deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu).view(1, m, k), weight.data, [128, 128], scale.data,
                                                       bias=bias.to(gpu) if with_bias else None)
    assert tuple(out.shape) == (1, m, n) and out.dtype == torch.bfloat16
    xq, exps, _ = O.per_token_group_quant_fp8_ue8m0(x)
    xs = torch.pow(2.0, exps.float() - 127.0)
    rows = rows_per_tile(m, 24)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], weight.data.cpu().t(), xs[rows], ws.t(), torch.bfloat16, acc_dtype=torch.float64)
    if with_bias:
        ref = ref + bias
    torch.testing.assert_close(out.cpu()[0][rows].float(), ref.float(), rtol=RTOL, atol=ATOL)
    # the packed scales of the reference's quantization call (fp8_utils.py:240-246) give the same result
    q_in, s_packed = sglang_per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    out2 = w8a8_block_fp8_matmul_deepgemm(q_in, weight.data, s_packed, scale.data, [128, 128], output_dtype=torch.bfloat16)
    if with_bias:
        out2 += bias.to(gpu)
    assert torch.equal(out2.view(torch.int16), out[0].view(torch.int16))


def test_deepgemm_linear_falls_back_like_the_reference(gpu, monkeypatch):
    """fp16 activations, or N not a multiple of 64: the Triton linear's call sequence (fp8_utils.py:227-234)."""
    import sglang_amd.quantization.fp8_utils as F
    from sglang_amd.quantization.fp8_utils import deepgemm_w8a8_block_fp8_linear_with_fallback, triton_w8a8_block_fp8_linear

    monkeypatch.setattr(F, "DEEPGEMM_SCALE_UE8M0", True)
    m, n, k = 40, 328, 512
    x = O.gen_activation(m, k, seed=3).to(gpu)
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=4))
    a = deepgemm_w8a8_block_fp8_linear_with_fallback(x, wq.to(gpu), [128, 128], ws.to(gpu))
    b = triton_w8a8_block_fp8_linear(x, wq.to(gpu), [128, 128], ws.to(gpu))
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    xh = x.to(torch.float16)
    wq2, ws2 = O.block_quant_weight(O.gen_weight(384, k, seed=6))
    a = deepgemm_w8a8_block_fp8_linear_with_fallback(xh, wq2.to(gpu), [128, 128], ws2.to(gpu))
    b = triton_w8a8_block_fp8_linear(xh, wq2.to(gpu), [128, 128], ws2.to(gpu))
    assert a.dtype == torch.float16 and torch.equal(a.view(torch.int16), b.view(torch.int16))
