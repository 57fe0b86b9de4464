"""GPU parity of the three GEMMs against the CPU oracle: INT32 accumulators
bit-exact, bf16/fp16 outputs within rtol 1e-2 / atol 1e-2 (the tolerance the
path's contract states for floating-point outputs)."""
import pytest
import torch

from helpers import rows_per_tile
from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
RTOL, ATOL = 1e-2, 1e-2


def say(*a):
    print(*a, flush=True)


def rand_i8(shape, seed, lo=-128, hi=128):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g, dtype=torch.int8)


def sample_rows(m, cap=48):
    """Rows of every row tile (see helpers.rows_per_tile)."""
    return rows_per_tile(m, cap)


@pytest.fixture(params=[1, 0], ids=["direct_lds", "via_regs"])
def load_path(request):
    from sglang_amd import _lib

    _lib.load().sglq_debug_set_direct_lds(request.param)
    yield request.param
    _lib.load().sglq_debug_set_direct_lds(1)


# tile_auto sends M <= 64 to the decode kernel; 192 / 224 / 257 are the 4 x 2-wave kernel's tile widths (257 = 256 wide), 258 the pipelined 256 x 256 kernel, 130 the same kernel with 128-row tiles,
# 16 / 32 the M <= 32 full-K decode kernel with that many weight rows per block, 66 the split-K decode kernel with 64 weight rows per block (M <= 512)
# 68 / 69 the full-K decode kernel on 64 x 64 / 32 x 64 tiles (32 < M <= 1024)
@pytest.fixture(params=[0, 128, 256, 192, 224, 257, 258, 130, 16, 32, 66, 68, 69],
                ids=["tile_auto", "tile128", "tile256", "wide192", "wide224", "wide256", "pipe256", "pipe128", "stream16", "stream32", "skinny64",
                     "stream64x64", "stream32x64"])
def tile(request):
    from sglang_amd import _lib

    _lib.load().sglq_debug_force_tile(request.param)
    yield request.param
    _lib.load().sglq_debug_force_tile(0)


@pytest.mark.parametrize("mnk", [(1, 128, 64), (5, 136, 128), (16, 8, 16), (33, 264, 208), (127, 256, 4096), (128, 1024, 512),
                                 (130, 640, 1040), (512, 14336, 4096)])
def test_int8_accumulators_bit_exact(gpu, load_path, tile, mnk):
    from sglang_amd.sgl_kernel import int8_mm_i32

    if (tile >= 192 or tile in (16, 32)) and not load_path:
        pytest.skip("the 256x256 kernel only has the direct-to-LDS path")
    say("int8 acc", mnk, "direct" if load_path else "regs", "tile", tile)
    m, n, k = mnk
    a, w = rand_i8((m, k), 1), rand_i8((n, k), 2)
    if m > 2:
        a[1] = -128
        w[0] = -128  # extreme products
    rows = sample_rows(m)
    ref = O.int8_mm_i32(a[rows], w.t())
    got = int8_mm_i32(a.to(gpu), w.to(gpu).t()).cpu()
    assert tuple(got.shape) == (m, n)
    bad = got[rows] != ref
    assert not bool(bad.any()), f"{int(bad.sum())} accumulators differ, first {bad.nonzero()[:4].tolist()}"


@pytest.mark.parametrize("m", [1, 16, 128, 1024])
def test_int8_scaled_mm_config(gpu, m):
    """A[M,4096] per-token INT8 x B[4096,14336] with per-column scales and bf16 bias."""
    from sglang_amd import _lib
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import int8_mm_i32, int8_scaled_mm

    lib = _lib.load()
    say("int8_scaled_mm config M", m)
    x = O.gen_activation(m, 4096, seed=1000 + m)
    wt, s_b, bias = O.gen_int8_weight(4096, 14336, seed=1000)
    xq_ref, xs_ref = O.per_token_quant_int8(x)
    xq, xs = per_token_quant_int8(x.to(gpu))
    assert torch.equal(xq.cpu(), xq_ref) and torch.equal(xs.cpu(), xs_ref)
    wg = wt.t().contiguous().to(gpu).t()  # [K, N] view with stride(0) == 1
    # every INT32 accumulator of the whole output against the oracle (the float64 product is exact here)
    acc = int8_mm_i32(xq, wg).cpu()
    acc_ref = O.int8_mm_i32(xq_ref, wt)
    bad = acc != acc_ref
    assert not bool(bad.any()), f"{int(bad.sum())} of {acc.numel()} accumulators differ, first {bad.nonzero()[:4].tolist()}"
    for b in (None, bias):
        run = lambda: int8_scaled_mm(xq, wg, xs, s_b.to(gpu), torch.bfloat16, None if b is None else b.to(gpu))
        out = run()
        selected = lib.sglq_debug_last_gemm_kernel().decode()
        # ... and every scaled output: against the oracle's epilogue on those accumulators
        ref = O.int8_scaled_mm(xq_ref, wt, xs_ref, s_b, torch.bfloat16, b)
        torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL, msg=lambda s: f"{selected}: {s}")
        if m >= 512:  # and against the same GEMM on the generic 128 x 128 kernel, as the other configurations' whole-output check
            lib.sglq_debug_force_tile(128)
            try:
                generic = run()
                assert lib.sglq_debug_last_gemm_kernel().decode().startswith("gemm_kernel")
            finally:
                lib.sglq_debug_force_tile(0)
            torch.testing.assert_close(out.float(), generic.float(), rtol=RTOL, atol=ATOL, msg=lambda s: f"{selected} vs generic kernel: {s}")


def make_block_case(m, n, k, seed, outliers=False):
    x = O.gen_activation(m, k, seed=seed, outliers=outliers)
    w = O.gen_weight(n, k, seed=seed)
    wq, ws = O.block_quant_weight(w)
    xq, xs = O.per_token_group_quant_fp8(x, 128) if k % 128 == 0 else (None, None)
    return x, xq, xs, wq, ws


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(1, 128, 128), (3, 256, 512), (5, 2112, 1536), (127, 512, 7168), (128, 4096, 512),
                                 (256, 2048, 7168), (512, 1536, 1024), (1024, 640, 2048)])
def test_fp8_blockwise_scaled_mm(gpu, load_path, tile, mnk, out_dtype):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    if (tile >= 192 or tile in (16, 32)) and not load_path:
        pytest.skip("the 256x256 kernel only has the direct-to-LDS path")
    say("fp8_blockwise", mnk, out_dtype, "direct" if load_path else "regs", "tile", tile)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = sample_rows(m)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()  # [M, K/128], stride(0) == 1
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (m, n)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(192, 192, 384), (193, 200, 512), (500, 2112, 1536), (1000, 640, 7168), (2048, 392, 1024), (4096, 2112, 896)])
def test_fp8_blockwise_scaled_mm_192_row_tiles(gpu, mnk, out_dtype):
    """The 4 x 2-wave kernel on 192 x 192 tiles (three fragment rows per wave, an epilogue of three passes): tiles cut by M
    and by N, the shortest K it takes and a long one; rows of every row tile against the oracle, the whole output against
    the generic 128 x 128 kernel."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    lib = _lib.load()
    say("fp8_blockwise 192-row tiles", mnk, out_dtype)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = rows_per_tile(m, 64, tile=192)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    args = (xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), out_dtype)
    lib.sglq_debug_force_tile(193)
    try:
        out = fp8_blockwise_scaled_mm(*args)
        assert lib.sglq_debug_last_gemm_kernel().decode() == "gemm_wide_kernel<6, 192 rows>"
        lib.sglq_debug_force_tile(128)
        generic = fp8_blockwise_scaled_mm(*args)
    finally:
        lib.sglq_debug_force_tile(0)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(out.float(), generic.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(256, 256, 384), (300, 520, 512), (1000, 1288, 1536), (2048, 4096, 512), (4096, 16640, 512), (515, 768, 7168)])
def test_fp8_blockwise_scaled_mm_direct_stores(gpu, mnk, out_dtype):
    """The pipelined 256 x 256 kernel that stores from the accumulators and copies on across tile boundaries: tiles cut
    by M, tiles cut by N (guarded stores), the shortest K, one tile per block and several (the first step behind a tile's
    stores); rows of every row tile against the oracle, the whole output against the generic 128 x 128 kernel."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    lib = _lib.load()
    say("fp8_blockwise direct stores", mnk, out_dtype)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = rows_per_tile(m, 48)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    args = (xq.to(gpu), wq.to(gpu).t(), xs.t().contiguous().to(gpu).t(), ws.to(gpu).t(), out_dtype)
    lib.sglq_debug_force_tile(259)
    lib.sglq_debug_force_splits(1)
    try:
        out = fp8_blockwise_scaled_mm(*args)
        assert lib.sglq_debug_last_gemm_kernel().decode() == "gemm_pipe_kernel<direct stores>"
        lib.sglq_debug_force_tile(128)
        lib.sglq_debug_force_splits(0)
        generic = fp8_blockwise_scaled_mm(*args)
    finally:
        lib.sglq_debug_force_tile(0)
        lib.sglq_debug_force_splits(0)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(out.float(), generic.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(3, 14080, 512), (127, 512, 14080), (5, 8192, 16384), (1024, 14080, 4096), (4096, 14080, 14080)])
def test_fp8_blockwise_scaled_mm_sizes_of_the_reference_test(gpu, mnk, out_dtype):
    """Corner points of the grid of sgl-kernel/tests/test_fp8_blockwise_gemm.py:84-87 (M from 1 to 4096,
    N and K up to 14080 = 110 x 128 and 16384), against the oracle on a sample of rows."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    say("fp8_blockwise, reference grid", mnk, out_dtype)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = sample_rows(m, 24)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (m, n)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(1, 128, 128), (5, 2112, 1536), (17, 7168, 2048), (127, 512, 7168), (128, 4096, 256),
                                 (300, 2048, 1024), (512, 1544, 1024), (1024, 640, 2048)])
def test_fp8_blockwise_scaled_mm_fused_bias(gpu, tile, mnk, out_dtype):
    """The fused variant performs the caller's two steps (fp8_utils.py:207-211: the GEMM rounded
    to the output type, then `output += bias`) in one kernel: bit-identical to doing them apart,
    on every kernel selection, with and without split-K."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_bias

    say("fp8_blockwise fused bias", mnk, out_dtype, "tile", tile)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(out_dtype).to(gpu)
    a, b = xq.to(gpu), wq.to(gpu).t()
    sa, sb = xs.t().contiguous().to(gpu).t(), ws.to(gpu).t()
    lib = _lib.load()
    for splits in (0, 2):
        lib.sglq_debug_force_splits(splits)
        try:
            plain = fp8_blockwise_scaled_mm(a, b, sa, sb, out_dtype)
            kernel_plain = lib.sglq_debug_last_gemm_kernel().decode()
            fused = fp8_blockwise_scaled_mm_bias(a, b, sa, sb, out_dtype, bias)
            assert lib.sglq_debug_last_gemm_kernel().decode() == kernel_plain
        finally:
            lib.sglq_debug_force_splits(0)
        plain += bias
        assert torch.equal(fused.view(torch.int16), plain.view(torch.int16)), (kernel_plain, splits)
    rows = sample_rows(m)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64) + bias.cpu().float()
    torch.testing.assert_close(fused.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


def make_block_int8_case(m, n, k, seed):
    x = O.gen_activation(m, k, seed=seed, outliers=True)
    wq, ws = O.block_quant_weight_int8(O.gen_weight(n, k, seed=seed))
    xq, xs = O.per_token_group_quant_8bit(x, 128, 1e-10, -128.0, 127.0, torch.int8)
    return xq, xs, wq, ws


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(1, 128, 128), (3, 256, 512), (5, 2112, 1536), (17, 7168, 2048), (127, 512, 7168), (128, 4096, 512),
                                 (256, 2048, 7168), (512, 1536, 1024), (1024, 640, 2048)])
def test_w8a8_block_int8_matmul(gpu, tile, mnk, out_dtype):
    """Block-scaled INT8 (w8a8_block_int8_matmul, int8_kernel.py:339-425) on every GEMM kernel:
    row-major activation scales, the weight and its scales as stored."""
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    say("block int8", mnk, out_dtype, "tile", tile)
    m, n, k = mnk
    xq, xs, wq, ws = make_block_int8_case(m, n, k, seed=m + n + k)
    rows = sample_rows(m)
    ref = O.w8a8_block_int8_matmul(xq[rows], wq, xs[rows], ws, torch.float32, acc_dtype=torch.float64)
    out = w8a8_block_int8_matmul(xq.to(gpu), wq.to(gpu), xs.to(gpu), ws.to(gpu), [128, 128], out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (m, n)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("mnk", [(5, 2112, 1536), (100, 640, 1024), (300, 2048, 1024), (1024, 640, 2048)])
def test_w8a8_block_int8_matmul_fused_bias(gpu, tile, mnk):
    """Block-scaled INT8 with the caller's `output + bias` (int8_utils.py:31-32) fused: bit-identical
    to the two steps done apart, on every kernel selection."""
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    say("block int8 fused bias", mnk, "tile", tile)
    m, n, k = mnk
    xq, xs, wq, ws = make_block_int8_case(m, n, k, seed=m + n + k)
    args = (xq.to(gpu), wq.to(gpu), xs.to(gpu), ws.to(gpu), [128, 128])
    for dt in (torch.bfloat16, torch.float16):
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(dt).to(gpu)
        plain = w8a8_block_int8_matmul(*args, dt)
        fused = w8a8_block_int8_matmul(*args, dt, bias=bias)
        assert torch.equal(fused.view(torch.int16), (plain + bias).view(torch.int16)), dt


def test_w8a8_block_int8_unit_scales_exact_and_linear(gpu):
    """Unit scales and small integers: exact whatever the summation order; then the glue
    (per-token-group INT8 quant, GEMM, bias) against the oracle's same sequence."""
    from sglang_amd.quantization.int8_kernel import per_token_group_quant_int8, w8a8_block_int8_matmul
    from sglang_amd.quantization.int8_utils import apply_w8a8_block_int8_linear

    say("block int8 exact integers + linear")
    g = torch.Generator().manual_seed(6)
    m, n, k = 300, 384, 1024
    a = torch.randint(-8, 9, (m, k), generator=g, dtype=torch.int8)
    w = torch.randint(-8, 9, (n, k), generator=g, dtype=torch.int8)
    ref = a.double() @ w.double().t()
    out = w8a8_block_int8_matmul(a.to(gpu), w.to(gpu), torch.ones((m, 8), device=gpu), torch.ones((3, 8), device=gpu),
                                 [128, 128], torch.bfloat16).cpu()
    assert torch.equal(out.double(), ref.to(torch.bfloat16).double())
    x = O.gen_activation(40, 2048, seed=77, outliers=True)
    wq, ws = O.block_quant_weight_int8(O.gen_weight(1536, 2048, seed=78))
    bias = (torch.randn(1536, generator=g) * 0.1).to(torch.bfloat16)
    xq_ref, xs_ref = O.per_token_group_quant_8bit(x, 128, 1e-10, -128.0, 127.0, torch.int8)
    xq, xs = per_token_group_quant_int8(x.to(gpu), 128)
    assert torch.equal(xq.cpu(), xq_ref) and torch.equal(xs.cpu(), xs_ref)
    mm = O.w8a8_block_int8_matmul(xq_ref, wq, xs_ref, ws, torch.float32)
    ref = mm + bias.float()
    out = apply_w8a8_block_int8_linear(x.to(gpu).view(2, 20, 2048), wq.to(gpu), [128, 128], ws.to(gpu), bias=bias.to(gpu))
    assert tuple(out.shape) == (2, 20, 1536) and out.dtype == torch.bfloat16
    tol = 1e-2 + 1e-2 * ref.abs() + mm.abs() * 2.0**-8  # the GEMM output is rounded to bf16 before the bias is added
    err = (out.cpu().view(40, 1536).float() - ref).abs()
    assert bool((err <= tol).all()), f"max excess {(err - tol).max().item()}"


def test_fp8_blockwise_unit_scales_is_plain_matmul(gpu):
    """All scales 1 and small integer-valued operands: every partial sum is an
    integer below 2^24, so the result is exact whatever the summation order."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    say("fp8_blockwise exact integers")
    g = torch.Generator().manual_seed(5)
    m, n, k = 77, 384, 1024
    a = torch.randint(-4, 5, (m, k), generator=g).float().to(FP8)
    w = torch.randint(-4, 5, (n, k), generator=g).float().to(FP8)
    ref = (a.double() @ w.double().t())
    assert float(ref.abs().max()) < 2**24  # exact in the fp32 accumulator
    sa = torch.ones((k // 128, m)).t().to(gpu)
    sb = torch.ones((n // 128, k // 128)).to(gpu).t()
    out = fp8_blockwise_scaled_mm(a.to(gpu), w.to(gpu).t(), sa, sb, torch.bfloat16).cpu()
    assert torch.equal(out.double(), ref.to(torch.bfloat16).double())


def test_fp8_blockwise_row_major_scales_vector(gpu):
    """K = 128: scales_a is a contiguous [M, 1] vector, which the reference accepts
    as well as an M-major matrix."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    m, n, k = 9, 256, 128
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=77)
    ref = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32, acc_dtype=torch.float64)
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs.to(gpu), ws.to(gpu).t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("mnk", [(1, 4096, 4096), (32, 6144, 4096), (256, 4096, 14336), (2048, 1024, 4096), (7, 16, 32), (100, 264, 1040)])
def test_fp8_scaled_mm(gpu, tile, mnk, with_bias):
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    say("fp8_scaled_mm", mnk, with_bias, "tile", tile)
    m, n, k = mnk
    x = O.gen_activation(m, k, seed=3000 + m)
    w = O.gen_weight(n, k, seed=3000 + n)
    xq, xs = O.per_token_quant_fp8(x)
    wq, ws = O.per_tensor_quant_weight(w)
    g = torch.Generator().manual_seed(m)
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16) if with_bias else None
    rows = sample_rows(m)
    ref = O.fp8_scaled_mm(xq[rows], wq.t(), xs[rows], ws, torch.float32, bias, acc_dtype=torch.float64)
    out = fp8_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs.to(gpu), ws.to(gpu), torch.bfloat16,
                        None if bias is None else bias.to(gpu))
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("mnk", [(1, 16, 512), (8192, 16, 16384), (64, 16384, 512), (4096, 128, 8192), (32, 8192, 16384), (512, 1024, 1024)])
def test_scaled_mm_sizes_of_the_reference_tests(gpu, mnk, with_bias, out_dtype):
    """Corner points of the grids of sgl-kernel/tests/test_int8_gemm.py:33-37 and test_fp8_gemm.py:39-43
    (M 1 ... 8192, N 16 ... 16384, K 512 ... 16384, bias or not, both output types): INT32
    accumulators exactly, both epilogues against the oracle on a sample of rows."""
    from sglang_amd.sgl_kernel import fp8_scaled_mm, int8_mm_i32, int8_scaled_mm

    say("scaled_mm, reference grids", mnk, with_bias, out_dtype)
    m, n, k = mnk
    g = torch.Generator().manual_seed(m + n + k)
    bias = (torch.randn(n, generator=g) * 0.1).to(out_dtype) if with_bias else None
    bias_g = None if bias is None else bias.to(gpu)
    rows = sample_rows(m, 24)
    x = O.gen_activation(m, k, seed=m + k)
    # INT8
    wt, s_b, _ = O.gen_int8_weight(k, n, seed=n + k)
    xq, xs = O.per_token_quant_int8(x)
    wg = wt.t().contiguous().to(gpu).t()
    assert torch.equal(int8_mm_i32(xq.to(gpu), wg).cpu()[rows], O.int8_mm_i32(xq[rows], wt))
    out = int8_scaled_mm(xq.to(gpu), wg, xs.to(gpu), s_b.to(gpu), out_dtype, bias_g)
    ref = O.int8_scaled_mm(xq[rows], wt, xs[rows], s_b, torch.float32, bias)
    assert out.dtype == out_dtype
    torch.testing.assert_close(out.cpu()[rows].float(), ref.float(), rtol=RTOL, atol=ATOL)
    # FP8 per token / per channel
    fq, fs = O.per_token_quant_fp8(x)
    wq, ws = O.per_tensor_quant_weight(O.gen_weight(n, k, seed=n))
    out = fp8_scaled_mm(fq.to(gpu), wq.to(gpu).t(), fs.to(gpu), ws.to(gpu), out_dtype, bias_g)
    ref = O.fp8_scaled_mm(fq[rows], wq.t(), fs[rows], ws, torch.float32, bias, acc_dtype=torch.float64)
    assert out.dtype == out_dtype
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


def test_gemm_linearity_at_full_size(gpu):
    """Full-size DeepSeek-V3 shape (M=4096, N=7168, K=16384): doubling the
    activation scales doubles the output exactly (power-of-two scaling commutes
    with every rounding), and a row sample matches the oracle."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    say("fp8_blockwise full size")
    m, n, k = 4096, 7168, 16384
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((m, k), generator=g, device=gpu).to(torch.bfloat16)
    w = O.gen_weight(n, k, seed=2)
    wq, ws = O.block_quant_weight(w)
    xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
    wqg, wsg = wq.to(gpu), ws.to(gpu)
    out = fp8_blockwise_scaled_mm(xq, wqg.t(), xs, wsg.t(), torch.bfloat16)
    out2 = fp8_blockwise_scaled_mm(xq, wqg.t(), (xs * 2.0).t().contiguous().t(), wsg.t(), torch.bfloat16)
    assert torch.equal(out2.float(), out.float() * 2.0)
    rows = sample_rows(m, 12)
    ref = O.fp8_blockwise_scaled_mm(xq[rows.to(gpu)].cpu(), wq.t(), xs[rows.to(gpu)].cpu(), ws.t(), torch.float32)
    torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)


@pytest.fixture(params=[0, 1, 2, 5], ids=["splits_auto", "splits1", "splits2", "splits5"])
def splits(request):
    from sglang_amd import _lib

    _lib.load().sglq_debug_force_splits(request.param)
    yield request.param
    _lib.load().sglq_debug_force_splits(0)


def check_every_kind(gpu, m, n, k):
    """Block-scaled FP8 (both output types), per-row / per-column FP8 and INT8 with bias, raw
    INT32 accumulators: against the oracle on all rows."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32, int8_scaled_mm

    # block-scaled FP8
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m * n + k, outliers=True)
    ref = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs.to(gpu) if k == 128 else xs_cm, ws.to(gpu).t(), torch.float16)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    # per-row / per-column FP8 with bias
    g = torch.Generator().manual_seed(m + n)
    sa = torch.rand((m, 1), generator=g) * 0.05 + 0.01
    sb = torch.rand((n, 1), generator=g) * 0.001 + 0.0005
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    ref = O.fp8_scaled_mm(xq, wq.t(), sa, sb, torch.float32, bias, acc_dtype=torch.float64)
    out = fp8_scaled_mm(xq.to(gpu), wq.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    # INT8: accumulators exact, epilogue within tolerance
    a8, w8 = rand_i8((m, k), 3), rand_i8((n, k), 4)
    acc_ref = O.int8_mm_i32(a8, w8.t())
    acc = int8_mm_i32(a8.to(gpu), w8.to(gpu).t()).cpu()
    assert torch.equal(acc, acc_ref)
    sa8 = sa * 0.01
    ref = O.int8_scaled_mm(a8, w8.t(), sa8, sb, torch.bfloat16, bias)
    out = int8_scaled_mm(a8.to(gpu), w8.to(gpu).t(), sa8.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL)


def test_output_beyond_the_last_level_cache(gpu):
    """An output of more than 384 MiB is stored with the non-temporal hint.  The same rows
    computed as two launches of half the rows each (plain stores, the same 256-row tiles) must
    give the same bits, and a row sample matches the oracle."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    say("fp8_blockwise, output above 384 MiB")
    m, n, k = 8192, 24832, 512
    assert 2 * m * n > 384 << 20 >= m * n
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((m, k), generator=g, device=gpu).to(torch.bfloat16)
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=5))
    wqg, wsg = wq.to(gpu), ws.to(gpu)
    xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
    out = fp8_blockwise_scaled_mm(xq, wqg.t(), xs, wsg.t(), torch.bfloat16)
    h = m // 2
    for lo in (0, h):
        part = fp8_blockwise_scaled_mm(xq[lo:lo + h], wqg.t(), xs[lo:lo + h].t().contiguous().t(), wsg.t(), torch.bfloat16)
        assert torch.equal(out[lo:lo + h], part)
        del part
    rows = sample_rows(m, 12)
    ref = O.fp8_blockwise_scaled_mm(xq[rows.to(gpu)].cpu(), wq.t(), xs[rows.to(gpu)].cpu(), ws.t(), torch.float32)
    torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("mnk", [(1, 128, 128), (7, 2112, 7168), (16, 7168, 2048), (17, 264, 1024), (33, 4096, 512),
                                 (64, 1536, 4096), (48, 136, 16384)])
def test_decode_kernel_split_k(gpu, splits, mnk):
    """M <= 64 runs on the weight-streaming kernel; its split-K partial sums and the
    reduction must reproduce the oracle for every kind and any split factor."""
    say("decode kernel", mnk, "splits", splits)
    check_every_kind(gpu, *mnk)


@pytest.mark.parametrize("mnk", [(65, 264, 1024), (100, 2112, 1536), (128, 4096, 512), (129, 640, 2048), (300, 384, 1024),
                                 (512, 256, 4096), (256, 4096, 4096), (200, 1096, 896)])
@pytest.mark.parametrize("weight_rows", [128, 64])
def test_decode_kernel_row_tiles(gpu, splits, mnk, weight_rows):
    """The weight-streaming kernel with a second grid dimension of 64-row tiles (up to M = 512), with
    128 or 64 weight rows per block: every kind, any split factor, ragged last tiles in both directions."""
    from sglang_amd import _lib

    say("decode kernel, row tiles", mnk, "splits", splits, "weight rows per block", weight_rows)
    lib = _lib.load()
    lib.sglq_debug_force_tile(64 if weight_rows == 128 else 66)
    try:
        check_every_kind(gpu, *mnk)
        name = lib.sglq_debug_last_gemm_kernel().decode()
        assert name.startswith("gemm_skinny_kernel<64 columns>" if weight_rows == 64 else "gemm_skinny_kernel") and \
            ("<64 columns>" in name) == (weight_rows == 64), name
    finally:
        lib.sglq_debug_force_tile(0)


@pytest.mark.parametrize("mnk", [(65, 264, 1024), (100, 2112, 1536), (128, 4096, 512), (129, 640, 2048), (300, 384, 1024),
                                 (512, 256, 4096), (256, 4096, 4096), (200, 1096, 896), (1000, 200, 640)])
@pytest.mark.parametrize("rows", [64, 32])
def test_full_k_decode_kernel_on_row_tiles(gpu, mnk, rows):
    """The full-K decode kernel on 64 x 64 and 32 x 64 tiles (several row tiles per weight tile, the four waves of
    a block take every fourth K block): every kind, ragged last tiles in both directions, fewer K blocks than waves + 1."""
    from sglang_amd import _lib

    say("full-K decode kernel,", rows, "x 64 tiles", mnk)
    lib = _lib.load()
    lib.sglq_debug_force_tile(68 if rows == 64 else 69)
    try:
        check_every_kind(gpu, *mnk)
        assert lib.sglq_debug_last_gemm_kernel().decode() == f"gemm_stream_kernel<{rows} x 64 tiles>"
    finally:
        lib.sglq_debug_force_tile(0)


@pytest.fixture(params=[16, 32], ids=["rows16", "rows32"])
def stream_rows(request):
    from sglang_amd import _lib

    _lib.load().sglq_debug_force_tile(request.param)
    yield request.param
    _lib.load().sglq_debug_force_tile(0)


@pytest.mark.parametrize("mnk", [(1, 128, 512), (1, 7168, 2048), (7, 2112, 7168), (16, 264, 640), (17, 136, 1024), (32, 4096, 512),
                                 (8, 48, 16384), (3, 24, 896)])
def test_decode_kernel_full_k(gpu, stream_rows, mnk):
    """M <= 32 with enough weight rows runs on the kernel whose blocks own all of K and add
    their four waves' partial sums in LDS (forced here for small N as well): every kind,
    N not a multiple of the block's rows, K blocks not a multiple of four."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32, int8_scaled_mm

    say("full-K decode kernel", mnk, "rows per block", stream_rows)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m * n + k, outliers=True)
    ref = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.float16)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    g = torch.Generator().manual_seed(m + n)
    sa = torch.rand((m, 1), generator=g) * 0.05 + 0.01
    sb = torch.rand((n, 1), generator=g) * 0.001 + 0.0005
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    ref = O.fp8_scaled_mm(xq, wq.t(), sa, sb, torch.float32, bias, acc_dtype=torch.float64)
    out = fp8_scaled_mm(xq.to(gpu), wq.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    a8, w8 = rand_i8((m, k), 3), rand_i8((n, k), 4)
    if m > 1:
        a8[1] = -128
        w8[n - 1] = -128
    acc = int8_mm_i32(a8.to(gpu), w8.to(gpu).t()).cpu()
    assert torch.equal(acc, O.int8_mm_i32(a8, w8.t()))
    sa8 = sa * 0.01
    ref = O.int8_scaled_mm(a8, w8.t(), sa8, sb, torch.bfloat16, bias)
    out = int8_scaled_mm(a8.to(gpu), w8.to(gpu).t(), sa8.to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("mnk", [(100, 384, 1024), (256, 2048, 7168), (130, 136, 2048), (1000, 256, 1536)])
def test_mid_m_split_k(gpu, splits, mnk):
    """The 128 x 128 kernel splits K across blocks when its tiles do not fill the chip."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32

    say("mid-M split-K", mnk, "splits", splits)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = sample_rows(m)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    g = torch.Generator().manual_seed(m)
    sa = torch.rand((m, 1), generator=g) * 0.05 + 0.01
    sb = torch.rand((n, 1), generator=g) * 0.001 + 0.0005
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.float16)
    ref = O.fp8_scaled_mm(xq[rows], wq.t(), sa[rows], sb, torch.float32, bias, acc_dtype=torch.float64)
    out = fp8_scaled_mm(xq.to(gpu), wq.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.float16, bias.to(gpu))
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    a8, w8 = rand_i8((m, k), 5), rand_i8((n, k), 6)
    assert torch.equal(int8_mm_i32(a8.to(gpu), w8.to(gpu).t()).cpu()[rows], O.int8_mm_i32(a8[rows], w8.t()))


@pytest.mark.parametrize("rows", [256, 128], ids=["pipe256", "pipe128"])
@pytest.mark.parametrize("mnk", [(100, 384, 1536), (512, 640, 7168), (300, 2112, 3072), (1000, 256, 1536)])
def test_pipelined_kernel_split_k(gpu, splits, mnk, rows):
    """The pipelined 256 x 256 kernel takes (tile, K range) work units when the tiles do not fill
    the chip (forced here): every kind, block-scaled INT8 included, and any split factor that
    leaves three K blocks per unit."""
    from sglang_amd import _lib
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32

    say("pipelined kernel split-K", mnk, "splits", splits, "rows per tile", rows)
    lib = _lib.load()
    lib.sglq_debug_force_tile(258 if rows == 256 else 130)
    try:
        m, n, k = mnk
        _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
        rows = sample_rows(m)
        ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
        xs_cm = xs.t().contiguous().to(gpu).t()
        out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
        kernel = lib.sglq_debug_last_gemm_kernel().decode()
        assert kernel.startswith("gemm_pipe_kernel")
        if splits in (2, 3, 4) and (k // 128) % splits == 0 and (k // 128) // splits >= 3:
            assert kernel.endswith("splitk_reduce_kernel")
        torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
        g = torch.Generator().manual_seed(m)
        sa = torch.rand((m, 1), generator=g) * 0.05 + 0.01
        sb = torch.rand((n, 1), generator=g) * 0.001 + 0.0005
        bias = (torch.randn(n, generator=g) * 0.1).to(torch.float16)
        ref = O.fp8_scaled_mm(xq[rows], wq.t(), sa[rows], sb, torch.float32, bias, acc_dtype=torch.float64)
        out = fp8_scaled_mm(xq.to(gpu), wq.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.float16, bias.to(gpu))
        torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
        a8, w8 = rand_i8((m, k), 5), rand_i8((n, k), 6)
        assert torch.equal(int8_mm_i32(a8.to(gpu), w8.to(gpu).t()).cpu()[rows], O.int8_mm_i32(a8[rows], w8.t()))
        x8, s8, wq8, ws8 = make_block_int8_case(m, n, k, seed=n + k)
        ref = O.w8a8_block_int8_matmul(x8[rows], wq8, s8[rows], ws8, torch.float32, acc_dtype=torch.float64)
        out = w8a8_block_int8_matmul(x8.to(gpu), wq8.to(gpu), s8.to(gpu), ws8.to(gpu), [128, 128], torch.bfloat16)
        torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)
    finally:
        lib.sglq_debug_force_tile(0)


def test_gemm_empty_m(gpu):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, int8_scaled_mm

    a = torch.empty((0, 128), dtype=torch.int8, device=gpu)
    w = torch.zeros((16, 128), dtype=torch.int8, device=gpu)
    out = int8_scaled_mm(a, w.t(), torch.empty((0, 1), device=gpu), torch.ones((16, 1), device=gpu), torch.bfloat16)
    assert tuple(out.shape) == (0, 16)


def test_tuned_table_selects_the_kernel(gpu):
    """An entry of the tuned table (the counterpart of the reference's per-(N, K) JSON configs) picks
    the kernel and split-K factor for its N, K and range of M only; the test hooks still override it;
    the results stay within tolerance of the oracle whatever kernel runs."""
    from sglang_amd import _lib
    from sglang_amd.quantization.tuned_configs import load_tuned_configs
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    lib = _lib.load()
    m, n, k = 300, 512, 1024
    x, xq, xs, wq, ws = make_block_case(m, n, k, seed=31)
    args = (xq.to(gpu), wq.to(gpu).t(), xs.to(gpu).t().contiguous().t(), ws.to(gpu).t(), torch.bfloat16)
    ref = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32, acc_dtype=torch.float64)
    try:
        lib.sglq_tuned_clear()
        fp8_blockwise_scaled_mm(*args)
        default_kernel = lib.sglq_debug_last_gemm_kernel().decode()
        other_n = (args[0], args[1][:, :256], args[2], args[3][:, :2], torch.bfloat16)
        fp8_blockwise_scaled_mm(*other_n)
        default_other_n = lib.sglq_debug_last_gemm_kernel().decode()
        assert lib.sglq_tuned_add(0, n, k, 200, 400, 258, 1) == 0   # this shape: the pipelined 256 x 256 kernel
        assert lib.sglq_tuned_add(0, n, k, 0, 199, 64, 2) == 0      # smaller M of the same (N, K)
        assert lib.sglq_tuned_add(4, n, k, 0, 1 << 30, 128, 0) == 0  # another kind: no effect here
        out = fp8_blockwise_scaled_mm(*args)
        assert lib.sglq_debug_last_gemm_kernel().decode() == "gemm_pipe_kernel" != default_kernel
        torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
        small = fp8_blockwise_scaled_mm(args[0][:50], args[1], args[2][:50], args[3], torch.bfloat16)
        assert lib.sglq_debug_last_gemm_kernel().decode() == "gemm_skinny_kernel+splitk_reduce_kernel"
        torch.testing.assert_close(small.cpu().float(), ref[:50], rtol=RTOL, atol=ATOL)
        fp8_blockwise_scaled_mm(*other_n)  # another N: no entry
        assert lib.sglq_debug_last_gemm_kernel().decode() == default_other_n != "gemm_pipe_kernel"
        lib.sglq_debug_force_tile(128)
        fp8_blockwise_scaled_mm(*args)
        assert lib.sglq_debug_last_gemm_kernel().decode().startswith("gemm_kernel")
    finally:
        lib.sglq_debug_force_tile(0)
        load_tuned_configs()


def test_shipped_tuned_tables_give_oracle_results(gpu):
    """Every selection in the tables shipped under sglang_amd/quantization/configs/ (block FP8 and
    block INT8) is run once at its own (M, N, K) with the tables loaded as a user has them, and
    checked against the oracle on the first and last 256 output columns."""
    import json

    from sglang_amd import _lib
    from sglang_amd.quantization import tuned_configs as T
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    _lib.load()
    assert T.load_tuned_configs() >= 0
    cases = []
    for path in sorted(T.CONFIG_DIR.iterdir()):
        parsed = T.parse_file_name(path.name)
        if parsed is None or parsed[3] not in T.KIND_OF_DTYPE:
            continue
        table = {int(key): val for key, val in json.loads(path.read_text()).items()}
        cases += [(parsed[3], m, parsed[0], parsed[1], v["tile"], v["splits"]) for m, v in table.items() if v["tile"] or v["splits"]]
    say("tuned selections shipped:", len(cases))
    assert {c[0] for c in cases} == {"fp8_w8a8", "int8_w8a8"}
    gg = torch.Generator(device=gpu).manual_seed(3)

    def codes(shape, int8):
        if int8:
            return torch.randint(-127, 128, shape, generator=gg, device=gpu, dtype=torch.int32).to(torch.int8)
        return (torch.randn(shape, generator=gg, device=gpu) * 2).to(FP8)

    weights = {}
    for dtype, m, n, k, tile, splits in cases:
        say("tuned entry", dtype, m, n, k, tile, splits)
        int8 = dtype == "int8_w8a8"
        if (dtype, n, k) not in weights:
            weights.clear()  # one weight at a time on the device
            ws = torch.rand(((n + 127) // 128, k // 128), generator=gg, device=gpu) * 1e-2 + 1e-3
            weights[(dtype, n, k)] = (codes((n, k), int8), ws)
        w, ws = weights[(dtype, n, k)]
        rows = min(m, 48)
        a = codes((m, k), int8)
        sa = (torch.rand((k // 128, m), generator=gg, device=gpu) * 1e-2 + 1e-3).t()
        if int8:
            sa = sa.contiguous()
            out = w8a8_block_int8_matmul(a, w, sa, ws, [128, 128], torch.bfloat16)
        else:
            out = fp8_blockwise_scaled_mm(a, w.t(), sa, ws.t(), torch.bfloat16)
        for cols in (slice(0, 256), slice(n - 256, n)):
            if cols.start % 128:
                continue
            nb = slice(cols.start // 128, (cols.stop + 127) // 128)
            if int8:
                ref = O.w8a8_block_int8_matmul(a[:rows].cpu(), w[cols].cpu(), sa[:rows].cpu(), ws[nb].cpu(), torch.float32,
                                               acc_dtype=torch.float64)
            else:
                ref = O.fp8_blockwise_scaled_mm(a[:rows].cpu(), w[cols].cpu().t(), sa[:rows].cpu().contiguous(),
                                                ws[nb].cpu().t()[:, : 2], torch.float32, acc_dtype=torch.float64)
            torch.testing.assert_close(out[:rows, cols].cpu().float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("mnk,kernel", [((8, 576, 7168), "gemm_stream_kernel<16 rows>"), ((32, 256, 7168), "gemm_stream_kernel<16 rows>"),
                                        ((64, 512, 7168), "gemm_stream_kernel<16 rows>"),
                                        ((96, 36864, 2048), "gemm_pipe_kernel<128 rows>")])
def test_narrow_weights_and_few_rows(gpu, mnk, kernel):
    """Shapes of the reference's tuned tables at the edges of the selection rules (N = 256 ... 576 of the
    DeepSeek-V3 projections; up to 128 rows on a wide weight): the kernel the rules choose, against the oracle."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    say("narrow / few rows", mnk, kernel)
    m, n, k = mnk
    _, xq, xs, wq, ws = make_block_case(m, n, k, seed=m + n + k, outliers=True)
    rows = sample_rows(m, 16)
    ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32, acc_dtype=torch.float64)
    xs_cm = xs.t().contiguous().to(gpu).t()
    out = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), torch.bfloat16)
    assert _lib.load().sglq_debug_last_gemm_kernel().decode() == kernel
    torch.testing.assert_close(out.cpu()[rows].float(), ref, rtol=RTOL, atol=ATOL)


BASELINE_KERNELS = [
    # (M, N, K) of the headline step and the kernel the profile summaries under profiles/ name for it
    ((4096, 24576, 1536), "gemm_pipe_kernel<direct stores>"),
    ((4096, 32768, 512), "gemm_pipe_kernel<direct stores>"),
    ((4096, 7168, 16384), "gemm_wide_kernel<7>"),
    ((4096, 4096, 7168), "gemm_pipe_kernel"),
    ((4096, 2112, 7168), "gemm_wide_kernel<6, 192 rows>"),
    # decode launches of the same shapes
    ((1, 7168, 16384), "gemm_stream_kernel<16 rows>"),
    ((8, 7168, 16384), "gemm_stream_kernel<16 rows>"),
    ((64, 7168, 16384), "gemm_skinny_kernel+splitk_reduce_kernel"),
    ((1, 4096, 7168), "gemm_stream_kernel<16 rows>"),
    ((64, 4096, 7168), "gemm_stream_kernel<16 rows>"),
    ((1, 24576, 1536), "gemm_skinny_kernel"),
    ((64, 24576, 1536), "gemm_skinny_kernel"),
]


@pytest.mark.parametrize("mnk,kernel", BASELINE_KERNELS)
def test_baseline_shapes_select_the_profiled_kernels(gpu, mnk, kernel):
    """The kernel selection is a set of measured rules and tuned tables; the profile summaries and the
    design notes name the kernel that serves each headline shape.  An edit of the rules that moves one of
    them must show up here (and in those summaries)."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    m, n, k = mnk
    lib = _lib.load()
    g = torch.Generator(device=gpu).manual_seed(5)
    a = torch.randn((m, k), generator=g, device=gpu).to(FP8)
    b = torch.randn((n, k), generator=g, device=gpu).to(FP8)
    sa = torch.rand((k // 128, m), generator=g, device=gpu).t() * 0.01 + 0.001
    sb = torch.rand(((n + 127) // 128, k // 128), generator=g, device=gpu) * 0.01 + 0.001
    fp8_blockwise_scaled_mm(a, b.t(), sa, sb.t(), torch.bfloat16)
    assert lib.sglq_debug_last_gemm_kernel().decode() == kernel
