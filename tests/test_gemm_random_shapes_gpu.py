"""Seeded random shapes through every GEMM kernel selection: ragged M, N that is a multiple
of 8 only, K any multiple of 128 (16 for the kernels that take it), against the CPU oracle.
INT32 accumulators bit-exact; 16-bit outputs within rtol 1e-2 / atol 1e-2."""
import random

import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
RTOL, ATOL = 1e-2, 1e-2

# (force_tile code, M range, needs K % 128 == 0)
SELECTIONS = [
    (0, (1, 700), False), (128, (1, 300), False), (256, (65, 600), True), (258, (65, 600), True), (130, (65, 600), True),
    (192, (65, 600), True), (224, (65, 600), True), (257, (65, 600), True), (64, (1, 64), True),
    (16, (1, 64), True), (32, (1, 32), True),
]


def shapes_for(code, m_range, k128, count, seed):
    rng = random.Random(seed * 1000 + code)
    out = []
    for _ in range(count):
        m = rng.randint(*m_range)
        n = 8 * rng.randint(1, 150)
        k = 128 * rng.randint(1, 18) if k128 else 16 * rng.randint(1, 140)
        if code in (16, 32):
            k = 128 * rng.randint(4, 40)
        out.append((m, n, k))
    return out


@pytest.mark.parametrize("code,m_range,k128", SELECTIONS, ids=[f"tile{c[0]}" for c in SELECTIONS])
def test_random_shapes_all_kinds(gpu, code, m_range, k128):
    from sglang_amd import _lib
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32, int8_scaled_mm

    lib = _lib.load()
    lib.sglq_debug_force_tile(code)
    try:
        for (m, n, k) in shapes_for(code, m_range, k128, 12, seed=7):
            print("random shape", code, (m, n, k), flush=True)
            g = torch.Generator().manual_seed(m * 31 + n * 7 + k)
            kb, nb = (k + 127) // 128, (n + 127) // 128
            a8 = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int8)
            w8 = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int8)
            af = (torch.randn((m, k), generator=g) * 2).to(FP8)
            wf = (torch.randn((n, k), generator=g) * 0.5).to(FP8)
            sa = torch.rand((m, 1), generator=g) * 0.05 + 0.01
            sb = torch.rand((n, 1), generator=g) * 0.01 + 0.001
            bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
            # INT32 accumulators: exact
            acc = int8_mm_i32(a8.to(gpu), w8.to(gpu).t()).cpu()
            assert torch.equal(acc, O.int8_mm_i32(a8, w8.t())), (code, m, n, k)
            # per-row / per-column kinds
            ref = O.int8_scaled_mm(a8, w8.t(), sa * 0.01, sb, torch.bfloat16, bias)
            out = int8_scaled_mm(a8.to(gpu), w8.to(gpu).t(), (sa * 0.01).to(gpu), sb.to(gpu), torch.bfloat16, bias.to(gpu))
            torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=RTOL, atol=ATOL)
            ref = O.fp8_scaled_mm(af, wf.t(), sa, sb, torch.float32, None, acc_dtype=torch.float64)
            out = fp8_scaled_mm(af.to(gpu), wf.to(gpu).t(), sa.to(gpu), sb.to(gpu), torch.float16, None)
            torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
            # block-scaled kinds
            sfa = torch.rand((m, kb), generator=g) * 0.05 + 0.01
            sfb = torch.rand((nb, kb), generator=g) * 0.01 + 0.001
            ref = O.fp8_blockwise_scaled_mm(af, wf.t(), sfa, sfb.t(), torch.float32, acc_dtype=torch.float64)
            sfa_cm = sfa.t().contiguous().to(gpu).t()
            out = fp8_blockwise_scaled_mm(af.to(gpu), wf.to(gpu).t(), sfa_cm, sfb.to(gpu).t(), torch.bfloat16)
            torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
            ref = O.w8a8_block_int8_matmul(a8, w8, sfa * 0.01, sfb, torch.float32, acc_dtype=torch.float64)
            out = w8a8_block_int8_matmul(a8.to(gpu), w8.to(gpu), (sfa * 0.01).to(gpu), sfb.to(gpu), [128, 128], torch.float16)
            torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    finally:
        lib.sglq_debug_force_tile(0)


@pytest.mark.parametrize("code,m", [(0, 300), (128, 300), (256, 300), (258, 300), (130, 300), (224, 300), (192, 300), (64, 48), (16, 9), (32, 20)],
                         ids=lambda v: str(v))
def test_strided_operands(gpu, code, m):
    """mat_a a column slice of a wider tensor (row stride 2 K + 64), mat_b a slice of a wider
    [N, 3 K] weight (column stride 3 K): the kernels take the strides, nothing is copied."""
    from sglang_amd import _lib
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, int8_mm_i32

    lib = _lib.load()
    lib.sglq_debug_force_tile(code)
    try:
        n, k = 520, 2048
        g = torch.Generator().manual_seed(code * 100 + m)
        a_big = torch.randint(-128, 128, (m, 2 * k + 64), generator=g, dtype=torch.int8)
        w_big = torch.randint(-128, 128, (n, 3 * k), generator=g, dtype=torch.int8)
        a, w = a_big[:, 64 : 64 + k], w_big[:, k : 2 * k]
        ag, wg = a_big.to(gpu)[:, 64 : 64 + k], w_big.to(gpu)[:, k : 2 * k]
        assert ag.stride(0) == 2 * k + 64 and wg.t().stride(1) == 3 * k
        assert torch.equal(int8_mm_i32(ag, wg.t()).cpu(), O.int8_mm_i32(a.contiguous(), w.contiguous().t()))
        af_big = (torch.randn((m, 2 * k + 64), generator=g) * 2).to(FP8)
        wf_big = (torch.randn((n, 3 * k), generator=g) * 0.5).to(FP8)
        sfa = torch.rand((m, k // 128), generator=g) * 0.05 + 0.01
        sfb = torch.rand(((n + 127) // 128, k // 128), generator=g) * 0.01 + 0.001
        ref = O.fp8_blockwise_scaled_mm(af_big[:, 64 : 64 + k].contiguous(), wf_big[:, k : 2 * k].contiguous().t(), sfa, sfb.t(),
                                        torch.float32, acc_dtype=torch.float64)
        out = fp8_blockwise_scaled_mm(af_big.to(gpu)[:, 64 : 64 + k], wf_big.to(gpu)[:, k : 2 * k].t(),
                                      sfa.t().contiguous().to(gpu).t(), sfb.to(gpu).t(), torch.bfloat16)
        torch.testing.assert_close(out.cpu().float(), ref, rtol=RTOL, atol=ATOL)
    finally:
        lib.sglq_debug_force_tile(0)


@pytest.mark.parametrize("code", [0, 128, 130, 256, 258, 257, 224, 192, 64, 16, 32], ids=lambda v: f"tile{v}")
@pytest.mark.parametrize("mn", [(300, 520), (257, 1000), (64, 264), (9, 2112), (513, 776)], ids=lambda v: f"{v[0]}x{v[1]}")
def test_output_written_only_inside_its_rows_and_columns(gpu, code, mn):
    """The output is a [M, N] window inside a larger sentinel-filled buffer (row stride N + 24,
    guard rows above and below): through the C ABI, with and without a workspace, every kernel
    must write its window and nothing else."""
    from sglang_amd import _lib

    m, n = mn
    if (code == 32 and m > 32) or (code == 16 and m > 64) or (code == 64 and m > 512):
        pytest.skip("kernel not applicable to this M")
    k = 1024
    lib = _lib.load()
    g = torch.Generator().manual_seed(m * n + code)
    a = (torch.randn((m, k), generator=g) * 2).to(FP8)
    w = (torch.randn((n, k), generator=g) * 0.5).to(FP8)
    sfa = torch.rand((m, k // 128), generator=g) * 0.05 + 0.01
    sfb = torch.rand(((n + 127) // 128, k // 128), generator=g) * 0.01 + 0.001
    ref = O.fp8_blockwise_scaled_mm(a, w.t(), sfa, sfb.t(), torch.float32, acc_dtype=torch.float64)
    ag, wg, sag, sbg = a.to(gpu), w.to(gpu), sfa.to(gpu), sfb.to(gpu)
    ldo, guard = n + 24, 3
    ws_ptr, ws_bytes = _lib.workspace(gpu)
    lib.sglq_debug_force_tile(code)
    try:
        for use_ws in (True, False):
            print("output window", code, mn, "workspace" if use_ws else "no workspace", flush=True)
            buf = torch.full((m + 2 * guard, ldo), 768.0, dtype=torch.bfloat16, device=gpu)
            out_ptr = buf.data_ptr() + (guard * ldo + 8) * 2  # window starts 8 columns in: rows stay 16-byte aligned
            rc = lib.sglq_fp8_blockwise_scaled_mm(
                ag.data_ptr(), k, wg.data_ptr(), k, sag.data_ptr(), sag.stride(0), sag.stride(1), sbg.data_ptr(), sbg.stride(1),
                sbg.stride(0), out_ptr, ldo, 0, m, n, k, ws_ptr if use_ws else None, ws_bytes if use_ws else 0,
                _lib.stream_ptr(gpu))
            assert rc == 0, lib.sglq_last_error()
            torch.cuda.synchronize()
            host = buf.cpu().float()
            window = host[guard:guard + m, 8:8 + n]
            torch.testing.assert_close(window, ref, rtol=RTOL, atol=ATOL)
            host[guard:guard + m, 8:8 + n] = 768.0
            assert bool((host == 768.0).all()), "a kernel wrote outside the output window"
    finally:
        lib.sglq_debug_force_tile(0)
