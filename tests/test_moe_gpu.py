"""GPU parity of the grouped (MoE) block-scaled FP8 GEMM: against the CPU oracle within
rtol 1e-2 / atol 1e-2, bit for bit against the dense operator run expert by expert with the
same tile shape, and the reference test's own acceptance criterion."""
import pytest
import torch

from oracle import w8a8_oracle as O
from helpers import calc_diff, moe_case

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
RTOL, ATOL = 1e-2, 1e-2
SENTINEL = 768.0  # exact in bf16 and fp16


def say(*a):
    print(*a, flush=True)


# the row tile: chosen from the average group, the 128-row kernel's tiles, the pipelined kernel with 128 and 256 rows
@pytest.fixture(params=[0, 32, 64, 128, 130, 256], ids=["rows_auto", "rows32", "rows64", "rows128", "rows128_pipelined", "rows256"])
def gtile(request):
    from sglang_amd import _lib

    _lib.load().sglq_debug_grouped_tile(request.param)
    yield request.param
    _lib.load().sglq_debug_grouped_tile(0)


def run_grouped(gpu, c, out_dtype, problem_sizes=None, expert_offsets=None, scales_b=None):
    """Calls the operator with the reference's argument list (scratch tensors included); the
    output starts filled with a sentinel so that untouched rows can be told apart."""
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    e = c["b"].shape[0]
    a, b = c["a"].to(gpu), c["b"].transpose(1, 2).contiguous().to(gpu).transpose(1, 2)  # [E, K, N], column-major slices
    sa = c["scales_a"].to(gpu)
    sb = (c["scales_b"] if scales_b is None else scales_b).to(gpu)
    ps = (c["problem_sizes"] if problem_sizes is None else problem_sizes).to(gpu)
    eo = (c["expert_offsets"] if expert_offsets is None else expert_offsets).to(gpu)
    out = torch.full((a.shape[0], b.shape[2]), SENTINEL, dtype=out_dtype, device=gpu)
    i64 = lambda: torch.empty((e,), dtype=torch.int64, device=gpu)
    strides = torch.full((e,), a.stride(0), dtype=torch.int64, device=gpu)
    c_strides = torch.full((e,), out.stride(0), dtype=torch.int64, device=gpu)
    layout = lambda: torch.zeros((e, 5), dtype=torch.int32, device=gpu)
    workspace = torch.empty((1 << 20,), dtype=torch.uint8, device=gpu)
    fp8_blockwise_scaled_grouped_mm(out, i64(), i64(), i64(), i64(), i64(), a, b, sa, sb, strides, strides, c_strides,
                                    layout(), layout(), ps, eo, workspace)
    return out


def check_against_oracle(c, out, rows_per_expert, out_dtype, cap=24):
    first = 0
    for e, m_g in enumerate(rows_per_expert):
        if m_g:
            pick = torch.arange(m_g) if m_g <= cap else torch.cat(
                [torch.arange(4), torch.randperm(m_g, generator=torch.Generator().manual_seed(e))[: cap - 8], torch.arange(m_g - 4, m_g)]).unique()
            rows = first + pick
            ref = O.fp8_blockwise_scaled_mm(c["a"][rows], c["b"][e], c["scales_a"][rows], c["scales_b"][e], torch.float32,
                                            acc_dtype=torch.float64)
            torch.testing.assert_close(out[rows].float(), ref, rtol=RTOL, atol=ATOL)
        first += m_g


@pytest.mark.parametrize("out_dtype", [torch.half, torch.bfloat16])
@pytest.mark.parametrize("num_experts", [8, 16])
def test_grouped_mm_reference_test_grid(gpu, gtile, num_experts, out_dtype):
    """The reference's test (sgl-kernel/tests/test_fp8_blockwise_moe.py:109-251): 8 or 16 experts
    with 16 .. 1024 rows each in steps of 16, N and K multiples of 2048; its acceptance
    criterion per expert, and the oracle on sampled rows."""
    import random

    rnd = random.Random(num_experts)
    rows = [16 * rnd.randint(1, 64) for _ in range(num_experts)]
    n, k = 2048 * rnd.randint(1, 2), 2048 * rnd.randint(1, 2)
    say("grouped mm, reference grid", num_experts, out_dtype, rows, n, k, "row tile", gtile)
    c = moe_case(num_experts, rows, n, k, seed=num_experts, dtype=out_dtype)
    out = run_grouped(gpu, c, out_dtype).cpu()
    assert out.dtype == out_dtype
    check_against_oracle(c, out, rows, out_dtype)
    first = 0
    for e, m_g in enumerate(rows):
        baseline = torch.mm(c["a_orig"][e].float(), c["b_orig"][e].float().t())
        assert calc_diff(out[first:first + m_g], baseline) < 0.001
        first += m_g


@pytest.mark.parametrize("rows", [[1, 0, 7, 129, 128, 0, 3, 255, 64, 33],   # average 62: 64-row tiles
                                  [1, 2, 0, 17, 31, 5, 32, 33],              # average 15: 32-row tiles
                                  [300, 0, 1, 257, 128, 127]],               # average 135: 128-row tiles
                         ids=["tiles64", "tiles32", "tiles128"])
def test_grouped_mm_ragged_groups(gpu, gtile, rows):
    """Groups of any size, empty ones included: a tile that straddles two experts must not
    write the other expert's rows; N not a multiple of 128."""
    say("grouped mm, ragged", rows, "row tile", gtile)
    c = moe_case(len(rows), rows, n=384, k=640, seed=len(rows))
    out = run_grouped(gpu, c, torch.bfloat16).cpu()
    check_against_oracle(c, out, rows, torch.bfloat16, cap=1 << 30)
    assert not bool((out == SENTINEL).any())


def test_grouped_mm_gaps_order_and_scale_strides(gpu, gtile):
    """Experts in any order with unowned rows between them (left untouched); weight scales
    passed as a transposed view (the reference's [E, N/128, K/128] storage)."""
    c = moe_case(3, [64, 64, 64], n=256, k=384, seed=5)
    sizes = torch.tensor([[40, 256, 384], [64, 256, 384], [9, 256, 384]], dtype=torch.int32)
    offsets = torch.tensor([128, 0, 80], dtype=torch.int32)
    sb_t = c["scales_b"].transpose(1, 2).contiguous().transpose(1, 2)  # same values, strides of [E, N/128, K/128]
    assert sb_t.stride() != c["scales_b"].stride()
    out = run_grouped(gpu, c, torch.bfloat16, sizes, offsets, sb_t).cpu()
    owned = torch.zeros(192, dtype=torch.bool)
    for e, (first, m_g) in enumerate([(128, 40), (0, 64), (80, 9)]):
        sl = slice(first, first + m_g)
        owned[sl] = True
        ref = O.fp8_blockwise_scaled_mm(c["a"][sl], c["b"][e], c["scales_a"][sl], c["scales_b"][e], torch.float32, acc_dtype=torch.float64)
        torch.testing.assert_close(out[sl].float(), ref, rtol=RTOL, atol=ATOL)
    assert bool((out[~owned] == SENTINEL).all())


@pytest.mark.parametrize("rows_per_tile", [128, 130, 256])
def test_grouped_mm_matches_dense_operator_bit_for_bit(gpu, rows_per_tile):
    """DeepSeek-V3-shaped expert GEMM (N = 4096, K = 7168, 32 experts, 8192 routed rows): every
    expert's rows equal the dense operator's result on that expert with the same kernel (the
    128 x 128 one, the pipelined one with 128 x 256 and 256 x 256 tiles) and no split-K, bit for bit (same
    summation order)."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    g = torch.Generator().manual_seed(11)
    gg = torch.Generator(device=gpu).manual_seed(11)
    e, n, k, total = 32, 4096, 7168, 8192
    cuts = torch.cat([torch.zeros(1, dtype=torch.long), torch.sort(torch.randint(0, total + 1, (e - 1,), generator=g)).values,
                      torch.tensor([total])])
    rows = (cuts[1:] - cuts[:-1]).tolist()
    say("grouped vs dense", rows)
    a = (torch.randn((total, k), generator=gg, device=gpu) * 2).to(FP8)
    b = torch.randn((e, n, k), generator=gg, device=gpu).to(FP8)
    sa = torch.rand((total, k // 128), generator=gg, device=gpu) * 0.01 + 0.001
    sb = torch.rand((e, k // 128, n // 128), generator=gg, device=gpu) * 0.01 + 0.001
    c = dict(a=a, b=b.transpose(1, 2), scales_a=sa, scales_b=sb,
             problem_sizes=torch.tensor([[r, n, k] for r in rows], dtype=torch.int32),
             expert_offsets=cuts[:-1].to(torch.int32))
    lib = _lib.load()
    lib.sglq_debug_grouped_tile(rows_per_tile)
    try:
        out = run_grouped(gpu, c, torch.bfloat16)
    finally:
        lib.sglq_debug_grouped_tile(0)
    want_kernel = {128: "grouped_plan_kernel+gemm_kernel<grouped>", 130: "grouped_plan_kernel+gemm_pipe_kernel<grouped, 128 rows>",
                   256: "grouped_plan_kernel+gemm_pipe_kernel<grouped>"}[rows_per_tile]
    assert lib.sglq_debug_last_gemm_kernel().decode() == want_kernel
    lib.sglq_debug_force_tile({128: 128, 130: 130, 256: 258}[rows_per_tile])
    lib.sglq_debug_force_splits(1)
    try:
        for x in (0, 5, 17, 31):
            if rows[x] <= 64:
                continue  # the dense operator would take a narrower tile
            sl = slice(int(cuts[x]), int(cuts[x + 1]))
            sa_cm = sa[sl].t().contiguous().t()  # the dense operator takes M-major activation scales
            dense = fp8_blockwise_scaled_mm(a[sl], b[x].t(), sa_cm, sb[x].t().contiguous().t(), torch.bfloat16)  # K-major weight scales
            assert lib.sglq_debug_last_gemm_kernel().decode() == {128: "gemm_kernel", 130: "gemm_pipe_kernel<128 rows>",
                                                                  256: "gemm_pipe_kernel"}[rows_per_tile]
            assert torch.equal(out[sl].view(torch.int16), dense.view(torch.int16)), x
    finally:
        lib.sglq_debug_force_tile(0)
        lib.sglq_debug_force_splits(0)
    assert not bool((out == SENTINEL).any())


def test_grouped_mm_argument_checks(gpu):
    c = moe_case(2, [16, 16], n=128, k=128, seed=1)
    with pytest.raises(RuntimeError, match="problem_sizes must be int32"):
        run_grouped(gpu, c, torch.bfloat16, problem_sizes=c["problem_sizes"].to(torch.int64))
    with pytest.raises(RuntimeError, match="must match expert_offsets"):
        run_grouped(gpu, c, torch.bfloat16, expert_offsets=torch.zeros(3, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="output must be bfloat16 or half"):
        run_grouped(gpu, c, torch.float32)
    # sizes that claim more rows than there are: clamped to the tensor, nothing outside is touched
    sizes = torch.tensor([[16, 128, 128], [1 << 20, 128, 128]], dtype=torch.int32)
    out = run_grouped(gpu, c, torch.bfloat16, problem_sizes=sizes).cpu()
    check_against_oracle(c, out, [16, 16], torch.bfloat16)
    # no experts, no rows
    empty = moe_case(2, [0, 0], n=128, k=128, seed=1)
    assert run_grouped(gpu, empty, torch.bfloat16).shape == (0, 128)
