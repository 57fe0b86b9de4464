"""The five benchmark configurations end to end on the GPU (quantize -> GEMM),
checked against the oracle: codes and scales bit-exact, INT32 accumulators exact,
bf16 outputs within rtol/atol 1e-2.  Activations are generated on the CPU with
the configuration's seed and the same bytes go to both sides; for large M the
oracle is evaluated on rows of every row tile (first, last and a random row of each tile plus
every position inside an MFMA fragment: about 110 rows at M = 8192), and the whole output is
compared with the generic 128 x 128 kernel's, which the same oracle rows validate."""
import pytest
import torch

from helpers import assert_bits_equal, rows_per_tile
from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-2

DSV3_NK = [(24576, 1536), (32768, 512), (7168, 16384), (4096, 7168), (2112, 7168)]
LLAMA8B_NK = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
LLAMA70B_NK = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]

_weights = {}


def block_weight(n, k, seed):
    key = ("block", n, k, seed)
    if key not in _weights:
        _weights.clear()  # keep one weight at a time: the largest is 470 MB
        _weights[key] = O.block_quant_weight(O.gen_weight(n, k, seed=seed))
    return _weights[key]


def rows_of(m):
    return rows_per_tile(m, cap=16)


def whole_output_check(fn, out, m, what):
    """Every element of a large output against the same GEMM on the generic 128 x 128 kernel
    (forced through the test hook), whose result the oracle rows validate as well: a wrong tile,
    scale or K block anywhere in the output of the selected kernel shows up here."""
    from sglang_amd import _lib

    if m < 512:
        return
    lib = _lib.load()
    selected = lib.sglq_debug_last_gemm_kernel().decode()
    lib.sglq_debug_force_tile(128)
    try:
        generic = fn()
        assert lib.sglq_debug_last_gemm_kernel().decode().startswith("gemm_kernel")
    finally:
        lib.sglq_debug_force_tile(0)
    torch.testing.assert_close(out.float(), generic.float(), rtol=RTOL, atol=ATOL, msg=lambda s: f"{what} ({selected}) vs generic kernel: {s}")
    return generic


def run_block_case(gpu, m, n, k, seed, outliers=False):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    print("block case", m, n, k, flush=True)
    x = O.gen_activation(m, k, seed=seed, outliers=outliers)
    wq, ws = block_weight(n, k, seed)
    rows = rows_of(m)
    xq_ref, xs_ref = O.per_token_group_quant_fp8(x[rows], 128)
    xq, xs = sglang_per_token_group_quant_fp8(x.to(gpu), 128, column_major_scales=True)
    assert_bits_equal(xq[rows.to(gpu)], xq_ref, "FP8 codes")
    assert_bits_equal(xs[rows.to(gpu)].contiguous(), xs_ref, "group scales")
    wq_g = wq.to(gpu)
    ws_g = ws.to(gpu)
    out = fp8_blockwise_scaled_mm(xq, wq_g.t(), xs, ws_g.t(), torch.bfloat16)
    ref = O.fp8_blockwise_scaled_mm(xq_ref, wq.t(), xs_ref, ws.t(), torch.float32)
    torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)
    generic = whole_output_check(lambda: fp8_blockwise_scaled_mm(xq, wq_g.t(), xs, ws_g.t(), torch.bfloat16), out, m, f"block {m}x{n}x{k}")
    if generic is not None:
        torch.testing.assert_close(generic[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)


def test_config0(gpu):
    run_block_case(gpu, 256, 2048, 7168, seed=0, outliers=True)


@pytest.mark.parametrize("nk", DSV3_NK)
def test_config2(gpu, nk):
    n, k = nk
    for m in (1, 8, 64, 512, 4096, 8192):
        run_block_case(gpu, m, n, k, seed=2000 + DSV3_NK.index(nk))


@pytest.mark.parametrize("nk", LLAMA8B_NK)
def test_config3(gpu, nk):
    n, k = nk
    wq, ws = O.per_tensor_quant_weight(O.gen_weight(n, k, seed=3000 + LLAMA8B_NK.index(nk)))
    for m in (1, 32, 256, 2048):
        _config3_case(gpu, m, n, k, wq, ws)


def _config3_case(gpu, m, n, k, wq, ws):
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_quant_fp8
    from sglang_amd.sgl_kernel import fp8_scaled_mm

    print("config3", m, n, k, flush=True)
    x = O.gen_activation(m, k, seed=3000 + m)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.1).to(torch.bfloat16)
    rows = rows_of(m)
    xq_ref, xs_ref = O.per_token_quant_fp8(x[rows])
    xq, xs = sglang_per_token_quant_fp8(x.to(gpu))
    assert_bits_equal(xq[rows.to(gpu)], xq_ref, "FP8 codes")
    assert_bits_equal(xs[rows.to(gpu)], xs_ref, "token scales")
    wq_g, ws_g = wq.to(gpu), ws.to(gpu)
    for b in (None, bias):
        bg = None if b is None else b.to(gpu)
        out = fp8_scaled_mm(xq, wq_g.t(), xs, ws_g, torch.bfloat16, bg)
        ref = O.fp8_scaled_mm(xq_ref, wq.t(), xs_ref, ws, torch.float32, b)
        torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)
        whole_output_check(lambda: fp8_scaled_mm(xq, wq_g.t(), xs, ws_g, torch.bfloat16, bg), out, m, f"per-channel {m}x{n}x{k}")


@pytest.mark.parametrize("nk", LLAMA70B_NK)
def test_config4(gpu, nk):
    n, k = nk
    for m in (64, 4096):
        run_block_case(gpu, m, n, k, seed=4000 + LLAMA70B_NK.index(nk))
