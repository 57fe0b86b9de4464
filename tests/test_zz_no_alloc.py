"""The entry point that allocates nothing, sglq_fp8_blockwise_scaled_mm_noalloc, against
sglq_fp8_blockwise_scaled_mm called with a caller workspace of the same size: the outputs must be
identical bit for bit (same kernels, same split-K factors), on calls in a row that share the
library's device scratch, the later ones smaller than the first; the calls must leave the device's free
memory unchanged and replay inside a HIP graph."""
import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 32 << 20  # SGLQ_NOALLOC_SCRATCH_BYTES in include/sglq.h


def _case(m, n, k, seed, dev):
    x = O.gen_activation(m, k, seed=seed)
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=seed + 1))
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    return xq, xs, wq, ws, xq.to(dev), xs.to(dev), wq.to(dev), ws.to(dev)


def _call(lib, name, a, b, sa, sb, out, m, n, k, extra):
    fn = getattr(lib, name)
    # weight [N, K] row-major = the column-major [K, N] operand; row-major activation scales;
    # weight scales [N/128, K/128] as stored: strides (k, n) = (1, K/128)
    return fn(a.data_ptr(), k, b.data_ptr(), k, sa.data_ptr(), sa.stride(0), sa.stride(1), sb.data_ptr(), sb.stride(1), sb.stride(0),
              out.data_ptr(), n, 0, m, n, k, *extra, torch.cuda.current_stream().cuda_stream)


def test_noalloc_entry_point_matches_the_workspace_entry_point(gpu):
    from sglang_amd import _lib

    lib = _lib.load()
    assert lib.sglq_init() == 0, lib.sglq_last_error()
    workspace = torch.empty(SCRATCH_BYTES, dtype=torch.uint8, device=gpu)
    # split-K decode kernel (4 splits), then the pipelined kernel with K split over work units,
    # then a smaller split-K problem whose partial sums land on the first calls' leftovers
    shapes = [(64, 7168, 16384), (1024, 2048, 7168), (40, 2048, 16384), (64, 7168, 16384), (8, 2112, 7168)]
    for i, (m, n, k) in enumerate(shapes):
        print(f"noalloc case {i}: {m} x {n} x {k}", flush=True)
        xq, xs, wq, ws, dxq, dxs, dwq, dws = _case(m, n, k, 9000 + 10 * i, gpu)
        want = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm", dxq, dwq, dxs, dws, want, m, n, k, (workspace.data_ptr(), workspace.numel()))
        assert rc == 0, lib.sglq_last_error()
        kernel = lib.sglq_debug_last_gemm_kernel().decode()
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm_noalloc", dxq, dwq, dxs, dws, got, m, n, k, ())
        assert rc == 0, lib.sglq_last_error()
        assert lib.sglq_debug_last_gemm_kernel().decode() == kernel
        if i < 4:
            assert "splitk" in kernel, kernel  # these shapes are here because they use the scratch
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"case {i} ({kernel}) differs from the workspace entry point"
        rows = sorted(set([0, m - 1, m // 2, (m * 3) // 7]))
        ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32)
        torch.testing.assert_close(got[rows].cpu().float(), ref, rtol=1e-2, atol=1e-2)


def test_noalloc_entry_point_allocates_nothing_and_replays_in_a_graph(gpu):
    """What the entry point is for: after sglq_init() the calls leave the device's free memory as it is, and a
    split-K call captured in a HIP graph (outputs preallocated) replays with changed inputs to the bits of the
    eager call."""
    from sglang_amd import _lib

    lib = _lib.load()
    assert lib.sglq_init() == 0, lib.sglq_last_error()
    m, n, k = 64, 7168, 16384
    print(f"noalloc under capture: {m} x {n} x {k}", flush=True)
    xq, xs, wq, ws, dxq, dxs, dwq, dws = _case(m, n, k, 9100, gpu)
    xq2, xs2, _, _, dxq2, dxs2, _, _ = _case(m, 128, k, 9200, gpu)
    a_in, s_in = dxq.clone(), dxs.clone()
    eager = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(gpu)[0]
    for _ in range(3):
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm_noalloc", a_in, dwq, s_in, dws, eager, m, n, k, ())
        assert rc == 0, lib.sglq_last_error()
    assert "splitk" in lib.sglq_debug_last_gemm_kernel().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(gpu)[0] == free_before, "the calls changed the device's free memory"
    side = torch.cuda.Stream(gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = _call(lib, "sglq_fp8_blockwise_scaled_mm_noalloc", a_in, dwq, s_in, dws, got, m, n, k, ())
            assert rc == 0, lib.sglq_last_error()
    torch.cuda.current_stream(gpu).wait_stream(side)
    for rep, (src_a, src_s, ref_a, ref_s) in enumerate(((dxq, dxs, xq, xs), (dxq2, dxs2, xq2, xs2), (dxq, dxs, xq, xs))):
        a_in.copy_(src_a)
        s_in.copy_(src_s)
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm_noalloc", a_in, dwq, s_in, dws, eager, m, n, k, ())
        assert rc == 0, lib.sglq_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16)), f"replay {rep} differs from the eager call"
        rows = [0, 17, m - 1]
        ref = O.fp8_blockwise_scaled_mm(ref_a[rows], wq.t(), ref_s[rows], ws.t(), torch.float32)
        torch.testing.assert_close(got[rows].cpu().float(), ref, rtol=1e-2, atol=1e-2)


def test_noalloc_entry_point_serves_outputs_larger_than_the_scratch_unsplit(gpu):
    """More than SGLQ_NOALLOC_MAX_OUTPUTS outputs (a prefill-sized call): K is not split, the array is not used,
    and the output equals the workspace entry point's with a workspace of the scratch's size bit for bit."""
    from sglang_amd import _lib

    lib = _lib.load()
    workspace = torch.empty(SCRATCH_BYTES, dtype=torch.uint8, device=gpu)
    for i, (m, n, k) in enumerate(((4096, 2112, 1024), (1152, 4096, 8192))):
        print(f"noalloc large case {i}: {m} x {n} x {k}", flush=True)
        assert m * n > SCRATCH_BYTES // 8
        xq, xs, wq, ws, dxq, dxs, dwq, dws = _case(m, n, k, 9300 + i, gpu)
        want = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm", dxq, dwq, dxs, dws, want, m, n, k, (workspace.data_ptr(), workspace.numel()))
        assert rc == 0, lib.sglq_last_error()
        kernel = lib.sglq_debug_last_gemm_kernel().decode()
        rc = _call(lib, "sglq_fp8_blockwise_scaled_mm_noalloc", dxq, dwq, dxs, dws, got, m, n, k, ())
        assert rc == 0, lib.sglq_last_error()
        assert lib.sglq_debug_last_gemm_kernel().decode() == kernel and "splitk" not in kernel, kernel
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"large case {i} ({kernel}) differs from the workspace entry point"
        rows = sorted(set([0, m - 1, m // 2, 255, 256]))
        ref = O.fp8_blockwise_scaled_mm(xq[rows], wq.t(), xs[rows], ws.t(), torch.float32)
        torch.testing.assert_close(got[rows].cpu().float(), ref, rtol=1e-2, atol=1e-2)


def test_noalloc_entry_point_rejects_what_the_library_cannot_address(gpu):
    from sglang_amd import _lib

    lib = _lib.load()
    t = torch.zeros(4096, dtype=torch.uint8, device=gpu)
    p = t.data_ptr()
    # an operand of 2 GiB or more: refused with a message before anything is launched
    rc = lib.sglq_fp8_blockwise_scaled_mm_noalloc(p, 1 << 20, p, 1 << 20, p, 1, 1, p, 1, 1, p, 4096, 0, 4096, 4096, 1 << 20, None)
    assert rc == 2 and b"2 GiB" in lib.sglq_last_error(), lib.sglq_last_error()
    # the other checks are the workspace entry point's
    rc = lib.sglq_fp8_blockwise_scaled_mm_noalloc(p, 128, p, 128, p, 1, 1, p, 1, 1, p, 12, 0, 4, 12, 128, None)
    assert rc == 1 and b"multiples of 8" in lib.sglq_last_error()
    assert lib.sglq_fp8_blockwise_scaled_mm_noalloc(p, 128, p, 128, p, 1, 1, p, 1, 1, p, 8, 0, 0, 8, 128, None) == 0
