"""Quantize-and-multiply as one operator (sglq_w8a8_block_fp8_linear): the output must equal
per-token-group quantization followed by the block-scaled GEMM (and the caller's bias add) bit
for bit, whether the call runs as the single fused decode kernel (M <= 8) or as the two kernels
in turn, and must match the oracle's quantize -> GEMM to the path's tolerance."""
import pytest
import torch

from helpers import rows_per_tile
from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-2

DSV3_NK = [(24576, 1536), (32768, 512), (7168, 16384), (4096, 7168), (2112, 7168)]
LLAMA70B_NK = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]
_weights = {}


def block_weight(n, k, seed, gpu):
    key = (n, k, seed)
    if key not in _weights:
        _weights.clear()
        wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=seed))
        _weights[key] = (wq, ws, wq.to(gpu), ws.to(gpu))
    return _weights[key]


def two_ops(x, wq_g, ws_g, bias):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_bias

    xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
    if bias is None:
        return fp8_blockwise_scaled_mm(xq, wq_g.t(), xs, ws_g.t(), x.dtype)
    return fp8_blockwise_scaled_mm_bias(xq, wq_g.t(), xs, ws_g.t(), x.dtype, bias)


def check_case(gpu, m, n, k, seed, dtype=torch.bfloat16, with_bias=False, outliers=False, expect_fused=None):
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel.gemm import block_fp8_linear

    lib = _lib.load()
    print("fused linear case", m, n, k, dtype, "bias" if with_bias else "", flush=True)
    wq, ws, wq_g, ws_g = block_weight(n, k, seed, gpu)
    x = O.gen_activation(m, k, seed=seed + 1, outliers=outliers).to(dtype)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(seed)) * 0.1).to(dtype) if with_bias else None
    xg, bg = x.to(gpu), None if bias is None else bias.to(gpu)
    want = two_ops(xg, wq_g, ws_g, bg)
    two_op_kernel = lib.sglq_debug_last_gemm_kernel().decode()
    got = block_fp8_linear(xg, wq_g.t(), ws_g.t(), bg)
    kernel = lib.sglq_debug_last_gemm_kernel().decode()
    if expect_fused is not None:
        assert kernel.startswith("gemm_stream_quant_kernel") == expect_fused, (kernel, two_op_kernel)
    if kernel.startswith("gemm_stream_quant_kernel"):
        # the fused kernel is the two-op path's decode kernel with the quantization folded in
        assert two_op_kernel == kernel.replace("gemm_stream_quant_kernel", "gemm_stream_kernel"), (kernel, two_op_kernel)
    else:
        assert kernel == two_op_kernel
    torch.cuda.synchronize()
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{kernel}: differs from quantize + GEMM ({two_op_kernel})"
    rows = rows_per_tile(m, cap=16)
    xq_ref, xs_ref = O.per_token_group_quant_fp8(x[rows], 128)
    ref = O.fp8_blockwise_scaled_mm(xq_ref, wq.t(), xs_ref, ws.t(), torch.float32)
    if bias is not None:
        ref = ref.to(dtype).float() + bias.float()
    torch.testing.assert_close(got[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL if bias is None else 2e-2)


@pytest.mark.parametrize("nk", DSV3_NK)
def test_fused_linear_config2_decode_rows(gpu, nk):
    n, k = nk
    for m in (1, 8, 64):
        check_case(gpu, m, n, k, seed=2000 + DSV3_NK.index(nk))


@pytest.mark.parametrize("nk", LLAMA70B_NK)
def test_fused_linear_config4_decode_rows(gpu, nk):
    n, k = nk
    for m in (1, 8, 64):
        check_case(gpu, m, n, k, seed=4000 + LLAMA70B_NK.index(nk))


@pytest.mark.parametrize("m", [1, 2, 3, 5, 7, 8])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_kernel_every_row_count(gpu, m, dtype):
    """Every M of the single-launch kernel, both activation types, 16- and 32-row blocks, with
    outliers (x20 on 1 % of the entries), an all-zero row and an all-zero group."""
    from sglang_amd import _lib

    lib = _lib.load()
    for tile, (n, k) in ((16, (2112, 1536)), (32, (4096, 1024)), (0, (8192, 2048))):
        lib.sglq_debug_force_tile(tile)
        try:
            # without a forced block height the single kernel is chosen for up to 4 rows on this shape (256 blocks of 32 rows)
            check_case(gpu, m, n, k, seed=100 * m + tile, dtype=dtype, with_bias=(m % 2 == 1), outliers=True,
                       expect_fused=(tile != 0 or m <= 4))
        finally:
            lib.sglq_debug_force_tile(0)


def test_fused_kernel_zero_rows_and_groups(gpu):
    from sglang_amd.sgl_kernel.gemm import block_fp8_linear

    print("fused linear: zero rows and groups", flush=True)
    n, k = 2048, 1024
    wq, ws, wq_g, ws_g = block_weight(n, k, 7, gpu)
    x = O.gen_activation(6, k, seed=8)
    x[1] = 0
    x[3, 256:384] = 0
    x[4, :128] = -0.0
    xg = x.to(gpu)
    got = block_fp8_linear(xg, wq_g.t(), ws_g.t())
    want = two_ops(xg, wq_g, ws_g, None)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert float(got[1].abs().max()) == 0.0


def test_fused_linear_other_shapes_take_two_launches(gpu):
    """M > 8, float32 activations... and shapes that the split-K decode kernel keeps: the operator
    still returns the two-op result, through the workspace."""
    check_case(gpu, 9, 4096, 7168, seed=31, expect_fused=False)
    check_case(gpu, 300, 2048, 1024, seed=32, with_bias=True, expect_fused=False)
    check_case(gpu, 4, 32768, 512, seed=33, expect_fused=False)   # short K on a wide weight: split-K kernel's shape
    check_case(gpu, 4, 512, 1024, seed=34, expect_fused=False)    # N < 1024
    check_case(gpu, 2, 2112, 7168, seed=35, expect_fused=False)   # 132 blocks: too few to hide the quantization
    check_case(gpu, 6, 8192, 2048, seed=36, expect_fused=False)   # more than 4 rows


def test_w8a8_block_fp8_linear_uses_it(gpu):
    """The glue function (fp8_utils.py:182-212) gives the same result for decode rows as for the
    same rows inside a larger batch (which takes the two-launch path)."""
    from sglang_amd.quantization.fp8_utils import w8a8_block_fp8_linear

    print("fused linear through the glue", flush=True)
    n, k = 4096, 7168
    wq, ws, wq_g, ws_g = block_weight(n, k, 2003, gpu)
    x = O.gen_activation(64, k, seed=41).to(gpu)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(5)) * 0.1).to(torch.bfloat16).to(gpu)
    for b in (None, bias):
        small = w8a8_block_fp8_linear(x[:4].view(2, 2, k), wq_g, [128, 128], ws_g, bias=b)
        assert tuple(small.shape) == (2, 2, n)
        big = w8a8_block_fp8_linear(x, wq_g, [128, 128], ws_g, bias=b)
        torch.testing.assert_close(small.view(4, n).float(), big[:4].float(), rtol=RTOL, atol=ATOL)
