"""Per-token quantize-and-multiply as one operator (sglq_w8a8_int8_linear, sglq_w8a8_fp8_linear): the output
must equal per_token_quant_int8 + int8_scaled_mm (w8a8_int8.py:387-391) and sgl_per_token_quant_fp8 +
fp8_scaled_mm (fp8_utils.py:693,725-732) bit for bit, whether the call runs as the single fused decode kernel
(M <= 8) or as the two kernels in turn, and must match the oracle's quantize -> GEMM: exactly for INT8 (the
accumulators are exact and the epilogue is one expression), to the path's tolerance for FP8."""
import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-2

CFG1_NK = [(14336, 4096)]
CFG3_NK = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
_weights = {}


def int8_weight(n, k, seed, gpu):
    key = ("i8", n, k, seed)
    if key not in _weights:
        _weights.clear()
        w, s_b, bias = O.gen_int8_weight(k, n, seed)  # w [K, N] column-major
        _weights[key] = (w, s_b, bias, w.t().contiguous().to(gpu).t(), s_b.to(gpu), bias.to(gpu))
    return _weights[key]


def fp8_weight(n, k, seed, gpu):
    key = ("f8", n, k, seed)
    if key not in _weights:
        _weights.clear()
        wq, ws = O.per_tensor_quant_weight(O.gen_weight(n, k, seed=seed))
        bias = (torch.randn(n, generator=torch.Generator().manual_seed(seed)) * 0.1).to(torch.bfloat16)
        _weights[key] = (wq.t(), ws, bias, wq.to(gpu).t(), ws.to(gpu), bias.to(gpu))
    return _weights[key]


def two_ops(kind, x, w_g, s_g, bias):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_quant_fp8
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import fp8_scaled_mm, int8_scaled_mm

    if kind == "int8":
        xq, xs = per_token_quant_int8(x)
        return int8_scaled_mm(xq, w_g, xs, s_g, x.dtype, bias)
    xq, xs = sglang_per_token_quant_fp8(x)
    return fp8_scaled_mm(xq, w_g, xs, s_g, x.dtype, bias)


def check_case(gpu, kind, m, n, k, seed, dtype=torch.bfloat16, with_bias=False, outliers=False, expect_fused=None, x=None):
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel.gemm import fp8_linear, int8_linear

    lib = _lib.load()
    print("fused per-token linear case", kind, m, n, k, dtype, "bias" if with_bias else "", flush=True)
    w, s_b, bias, w_g, s_g, bias_g = (int8_weight if kind == "int8" else fp8_weight)(n, k, seed, gpu)
    if x is None:
        x = O.gen_activation(m, k, seed=seed + 1, outliers=outliers)
    x = x.to(dtype)
    b, bg = (bias.to(dtype), bias_g.to(dtype)) if with_bias else (None, None)
    xg = x.to(gpu)
    want = two_ops(kind, xg, w_g, s_g, bg)
    two_op_kernel = lib.sglq_debug_last_gemm_kernel().decode()
    got = (int8_linear if kind == "int8" else fp8_linear)(xg, w_g, s_g, bg)
    kernel = lib.sglq_debug_last_gemm_kernel().decode()
    if expect_fused is not None:
        assert kernel.startswith("gemm_stream_tokenquant_kernel") == expect_fused, (kernel, two_op_kernel)
    if kernel.startswith("gemm_stream_tokenquant_kernel"):
        # the fused kernel is the two-op path's decode kernel with the quantization folded in
        assert two_op_kernel == kernel.replace("gemm_stream_tokenquant_kernel", "gemm_stream_kernel"), (kernel, two_op_kernel)
    else:
        assert kernel == two_op_kernel
    torch.cuda.synchronize()
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{kernel}: differs from quantize + GEMM ({two_op_kernel})"
    if kind == "int8":
        xq, xs = O.per_token_quant_int8(x)
        ref = O.int8_scaled_mm(xq, w, xs, s_b, dtype, b)
        # exact accumulators and one fused multiply-add per output: at most the last place of the 16-bit result moves
        # (the host evaluates acc * (s_b * s_a) + bias with two roundings, the kernel with one)
        torch.testing.assert_close(got.cpu().float(), ref.float(), rtol=2 ** -7, atol=1e-3)
    else:
        xq, xs = O.per_token_quant_fp8(x)
        ref = O.fp8_scaled_mm(xq, w, xs, s_b, torch.float32, None if b is None else b.float())
        torch.testing.assert_close(got.cpu().float(), ref, rtol=RTOL, atol=ATOL if b is None else 2e-2)


@pytest.mark.parametrize("nk", CFG1_NK)
def test_fused_int8_linear_config1_decode_rows(gpu, nk):
    n, k = nk
    for m in (1, 2, 8, 16):
        check_case(gpu, "int8", m, n, k, seed=1000, with_bias=True)


@pytest.mark.parametrize("nk", CFG3_NK)
def test_fused_fp8_linear_config3_decode_rows(gpu, nk):
    n, k = nk
    for m in (1, 2, 8, 32):
        check_case(gpu, "fp8", m, n, k, seed=3000 + CFG3_NK.index(nk), with_bias=(m == 2))


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("m", [1, 2, 3, 5, 7, 8])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_token_kernel_every_row_count(gpu, kind, m, dtype):
    """Every M of the single-launch kernel, both activation types, 16- and 32-row blocks, with outliers (x20 on
    1 % of the entries); rows longer than one sweep of the block (K > 8192) included."""
    from sglang_amd import _lib

    lib = _lib.load()
    for tile, (n, k) in ((16, (2112, 1536)), (32, (4096, 1024)), (16, (1024, 9216)), (0, (8192, 2048))):
        lib.sglq_debug_force_tile(tile)
        try:
            check_case(gpu, kind, m, n, k, seed=100 * m + tile, dtype=dtype, with_bias=(m % 2 == 1), outliers=True,
                       expect_fused=(tile != 0 or m <= 2))
        finally:
            lib.sglq_debug_force_tile(0)


@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_fused_token_kernel_zero_rows_and_ties(gpu, kind):
    """An all-zero row (FP8: scale 0, guarded inverse, zero codes; INT8: the 1e-10 floor), a row of -0.0, and
    INT8 ties: values k + 0.5 times a row scale of 2^j round half away from zero."""
    n, k = 2048, 1024
    x = O.gen_activation(6, k, seed=8).float()
    x[1] = 0
    x[4] = -0.0
    ks = torch.arange(k, dtype=torch.float32) % 126
    x[2] = (ks + 0.5) * 0.25          # row maximum 125.5 * 0.25 ...
    x[2, 0] = 127 * 0.25              # ... raised to 127 * 2^-2: the multiplier is exactly 4, every other entry a tie
    x[3] = -x[2]
    from sglang_amd import _lib

    lib = _lib.load()
    for tile in (16, 32):
        lib.sglq_debug_force_tile(tile)
        try:
            check_case(gpu, kind, 6, n, k, seed=9, x=x.to(torch.bfloat16), expect_fused=True)
        finally:
            lib.sglq_debug_force_tile(0)


def test_fused_token_linear_other_shapes_take_two_launches(gpu):
    """M > 8, K not a multiple of 128 and shapes that the split-K decode kernel keeps: the operators still
    return the two-op result, through the workspace."""
    check_case(gpu, "int8", 9, 4096, 4096, seed=31, expect_fused=False)
    check_case(gpu, "fp8", 300, 2048, 1024, seed=32, with_bias=True, expect_fused=False)
    check_case(gpu, "fp8", 1, 32768, 512, seed=33, expect_fused=False)   # short K on a wide weight: split-K kernel's shape
    check_case(gpu, "int8", 2, 2048, 1040, seed=34, expect_fused=False)  # K % 128 != 0
    check_case(gpu, "int8", 4, 8192, 2048, seed=36, expect_fused=False)  # more rows than the rule fuses


def test_linear_methods_use_it(gpu):
    """W8A8Int8LinearMethod.apply and apply_fp8_linear (dynamic per-token) give decode rows the same bits as
    the same rows computed by the two operators."""
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear
    from sglang_amd.quantization.w8a8_int8 import apply_w8a8_int8_linear

    print("fused per-token linear through the glue", flush=True)
    n, k = 4096, 4096
    w, s_b, bias, w_g, s_g, bias_g = int8_weight(n, k, 51, gpu)
    x = O.gen_activation(2, k, seed=52).to(gpu)
    got = apply_w8a8_int8_linear(x.view(1, 2, k), w_g, s_g.view(n, 1), bias_g)
    assert tuple(got.shape) == (1, 2, n)
    assert torch.equal(got.view(2, n).view(torch.int16), two_ops("int8", x, w_g, s_g, bias_g).view(torch.int16))
    w, s_b, bias, w_g, s_g, bias_g = fp8_weight(n, k, 53, gpu)
    got = apply_fp8_linear(x.view(1, 2, k), w_g, s_g, bias=bias_g, use_per_token_if_dynamic=True)
    assert tuple(got.shape) == (1, 2, n)
    assert torch.equal(got.view(2, n).view(torch.int16), two_ops("fp8", x, w_g, s_g, bias_g).view(torch.int16))
