"""The operators enqueue kernels on the caller's stream and nothing else (no allocation inside
the library, no host synchronisation, no memset), so a quantize -> GEMM sequence can be captured
into a HIP graph, as the reference's decode path does with CUDA graphs.  Every replay must give
what eager execution gives on the same buffer contents, bit for bit."""
import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


@pytest.mark.parametrize("m", [1, 16, 48, 300])
def test_graph_replay_matches_eager(gpu, m):
    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant, sglang_per_token_group_quant_fp8, sglang_per_token_quant_fp8
    from sglang_amd.quantization.int8_kernel import per_token_group_quant_int8, per_token_quant_int8, w8a8_block_int8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_scaled_mm

    print("graph replay", m, flush=True)
    n, k = 2112, 4096
    _lib.workspace(gpu)  # the eager calls' workspace; the capture stream gets one of its own from the graph's pool
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=1))
    w8, ws8 = O.block_quant_weight_int8(O.gen_weight(n, k, seed=2))
    wq, ws, w8, ws8 = wq.to(gpu), ws.to(gpu), w8.to(gpu), ws8.to(gpu)
    sb = (torch.rand((n, 1)) * 0.01 + 0.001).to(gpu)
    bias = (torch.randn(n) * 0.1).to(torch.bfloat16).to(gpu)
    x = O.gen_activation(m, k, seed=3, outliers=True).to(gpu)
    static_scale = torch.tensor([0.05], device=gpu)

    def run(x):
        xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
        y0 = fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16)
        xq, xs = sglang_per_token_quant_fp8(x)
        y1 = fp8_scaled_mm(xq, wq.t(), xs, sb, torch.bfloat16, bias)
        xq, xs = per_token_quant_int8(x)
        y2 = int8_scaled_mm(xq, w8.t(), xs, sb, torch.bfloat16, bias)
        xq, xs = per_token_group_quant_int8(x, 128)
        y3 = w8a8_block_int8_matmul(xq, w8, xs, ws8, [128, 128], torch.bfloat16)
        xq, _ = scaled_fp8_quant(x, static_scale)
        xq_dyn, s_dyn = scaled_fp8_quant(x)  # zero-fills its scale with a fill kernel, then an atomic max
        return y0, y1, y2, y3, xq, xq_dyn, s_dyn

    run(x)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(x)
    for rep in range(3):
        x.copy_(O.gen_activation(m, k, seed=10 + rep, outliers=True).to(gpu))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run(x)  # eager work between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {rep}, output {i} differs from eager"


@pytest.mark.parametrize("rows_per_expert", [3, 40, 200])
def test_graph_replay_grouped_mm(gpu, rows_per_expert):
    """The grouped GEMM reads the experts' row counts on the device: a captured launch follows
    new routing (other problem_sizes / expert_offsets contents) on every replay."""
    from helpers import moe_case
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    print("graph replay, grouped", rows_per_expert, flush=True)
    e, n, k = 6, 512, 1024
    total = e * rows_per_expert
    c = moe_case(e, [rows_per_expert] * e, n, k, seed=rows_per_expert)
    a, b = c["a"].to(gpu), c["b"].transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    sa, sb = c["scales_a"].to(gpu), c["scales_b"].to(gpu)
    ps, eo = c["problem_sizes"].to(gpu), c["expert_offsets"].to(gpu)
    out = torch.zeros((total, n), dtype=torch.bfloat16, device=gpu)
    i64 = torch.empty((e,), dtype=torch.int64, device=gpu)
    lay = torch.zeros((e, 5), dtype=torch.int32, device=gpu)
    ws = torch.empty((1 << 16,), dtype=torch.uint8, device=gpu)

    def run(dst):
        fp8_blockwise_scaled_grouped_mm(dst, i64, i64, i64, i64, i64, a, b, sa, sb, i64, i64, i64, lay, lay, ps, eo, ws)

    run(out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(out)
    g = torch.Generator().manual_seed(1)
    for rep in range(3):
        # new routing with the same total: random cuts of the rows
        cuts = torch.cat([torch.zeros(1, dtype=torch.long), torch.sort(torch.randint(0, total + 1, (e - 1,), generator=g)).values,
                          torch.tensor([total])])
        ps.copy_(torch.stack([cuts[1:] - cuts[:-1], torch.full((e,), n), torch.full((e,), k)], dim=1).to(torch.int32))
        eo.copy_(cuts[:-1].to(torch.int32))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = torch.zeros_like(out)
        run(want)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay {rep} differs from eager"
        first = int(cuts[2])
        rows = int(cuts[3] - cuts[2])
        if rows:
            ref = O.fp8_blockwise_scaled_mm(c["a"][first:first + rows], c["b"][2], c["scales_a"][first:first + rows], c["scales_b"][2],
                                            torch.float32, acc_dtype=torch.float64)
            torch.testing.assert_close(got[first:first + rows].cpu().float(), ref, rtol=1e-2, atol=1e-2)


def test_two_streams_do_not_share_partial_sums(gpu):
    """Split-K GEMMs enqueued on two streams at the same time each use a workspace of their own
    stream, so both give what a call alone gives."""
    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    print("two streams", flush=True)
    lib = _lib.load()
    m, n, k = 300, 2112, 7168
    lib.sglq_debug_force_tile(64)  # the split-K decode kernel, four splits
    lib.sglq_debug_force_splits(4)
    try:
        wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=21))
        wq, ws = wq.to(gpu), ws.to(gpu)
        cases = []
        for seed in (22, 23):
            xq, xs = sglang_per_token_group_quant_fp8(O.gen_activation(m, k, seed=seed).to(gpu), 128, column_major_scales=True)
            alone = fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16)
            assert "splitk_reduce_kernel" in lib.sglq_debug_last_gemm_kernel().decode()
            cases.append((xq, xs, alone))
        torch.cuda.synchronize()
        streams = [torch.cuda.Stream(gpu), torch.cuda.Stream(gpu)]
        pointers = set()
        got = [[], []]
        for rep in range(20):
            for i, s in enumerate(streams):
                with torch.cuda.stream(s):
                    pointers.add(_lib.workspace(gpu)[0])
                    xq, xs, _ = cases[i]
                    got[i].append(fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16))
        torch.cuda.synchronize()
        assert len(pointers) == 2
        for i in range(2):
            for y in got[i]:
                assert torch.equal(y, cases[i][2])
    finally:
        lib.sglq_debug_force_tile(0)
        lib.sglq_debug_force_splits(0)
