"""The five benchmark configurations end to end on the GPU (quantize -> GEMM),
checked against the oracle: codes and scales bit-exact, INT32 accumulators exact,
bf16 outputs within rtol/atol 1e-2.  Activations are generated on the CPU with
the configuration's seed and the same bytes go to both sides; for large M the
oracle is evaluated on a row sample (every row is independent of the others)."""
import pytest
import torch

from helpers import assert_bits_equal
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


def rows_of(m, cap=16):
    if m <= cap:
        return torch.arange(m)
    g = torch.Generator().manual_seed(m)
    return torch.cat([torch.randperm(m, generator=g)[: cap - 2], torch.tensor([0, m - 1])]).unique()


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
    out = fp8_blockwise_scaled_mm(xq, wq_g.t(), xs, ws.to(gpu).t(), torch.bfloat16)
    ref = O.fp8_blockwise_scaled_mm(xq_ref, wq.t(), xs_ref, ws.t(), torch.float32)
    torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)


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
    for b in (None, bias):
        out = fp8_scaled_mm(xq, wq.to(gpu).t(), xs, ws.to(gpu), torch.bfloat16, None if b is None else b.to(gpu))
        ref = O.fp8_scaled_mm(xq_ref, wq.t(), xs_ref, ws, torch.float32, b)
        torch.testing.assert_close(out[rows.to(gpu)].cpu().float(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("nk", LLAMA70B_NK)
def test_config4(gpu, nk):
    n, k = nk
    for m in (64, 4096):
        run_block_case(gpu, m, n, k, seed=4000 + LLAMA70B_NK.index(nk))
