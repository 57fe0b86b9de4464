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
    _lib.workspace(gpu)  # allocated before capture, as a server would at start-up
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
