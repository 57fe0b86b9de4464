"""GPU parity of the operators around the grouped GEMM in an MoE expert layer and of the layer
itself (python/sglang/srt/layers/moe/cutlass_moe.py:140-222): routing tables, row gathers and
the weighted combine bit for bit against the CPU oracle, SiLU-and-multiply within two units in
the last place (rarely different at all), the layer step by step on shared inputs (GEMMs within
rtol 1e-2 / atol 1e-2, everything else bit for bit)."""
import pytest
import torch

from oracle import w8a8_oracle as O
from helpers import assert_bits_equal, moe_layer_case

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
RTOL, ATOL = 1e-2, 1e-2


def say(*a):
    print(*a, flush=True)


def run_prepare(gpu, ids, num_experts, n, k, with_blockscale=True, fill=-7, shift=0):
    """`shift` moves topk_ids off its 16-byte alignment by that many elements."""
    from sglang_amd.sgl_kernel import prepare_moe_input

    i32 = lambda *shape: torch.full(shape, fill, dtype=torch.int32, device=gpu)
    if shift:
        holder = torch.full((ids.numel() + shift + 8,), 0, dtype=torch.int32)
        holder[shift:shift + ids.numel()] = ids.reshape(-1)
        ids = holder.to(gpu)[shift:shift + ids.numel()].view(ids.shape)
        assert ids.data_ptr() % 16 != 0
    offsets, rounded = i32(num_experts + 1), i32(num_experts + 1)
    ps1, ps2 = i32(num_experts, 3), i32(num_experts, 3)
    a_map, c_map = i32(ids.numel()), i32(ids.numel())
    prepare_moe_input(ids.to(gpu), offsets, ps1, ps2, a_map, c_map, num_experts, n, k,
                      blockscale_offsets=rounded if with_blockscale else None)
    return [t.cpu() for t in (offsets, rounded, ps1, ps2, a_map, c_map)]


@pytest.mark.parametrize("m,topk,num_experts", [(1, 1, 1), (1, 8, 256), (33, 2, 8), (257, 8, 64), (1000, 6, 160),
                                                (4096, 8, 256), (77, 4, 384), (300, 1, 3), (4099, 7, 8), (9000, 3, 2)])
def test_prepare_moe_input_tables(gpu, m, topk, num_experts):
    """Every table equals the oracle's, which keeps slot order inside an expert (the operator's
    documented order); ids outside [0, E) leave their output_permutation entry and the tail of
    input_permutation untouched."""
    g = torch.Generator().manual_seed(m * 31 + topk)
    ids = torch.randint(0, num_experts, (m, topk), generator=g, dtype=torch.int32)
    if m > 16:
        ids[3, 0] = -1
        ids[7, topk - 1] = num_experts       # routed to nobody
        ids[m // 2:, 0] = ids[0, 0]          # a crowded expert, longer than one sweep of the block
    say("prepare_moe_input", m, topk, num_experts)
    n, k = 768, 1024
    got = run_prepare(gpu, ids, num_experts, n, k)
    want = O.prepare_moe_input(ids, num_experts, n, k)
    names = ["expert_offsets", "blockscale_offsets", "problem_sizes1", "problem_sizes2", "input_permutation", "output_permutation"]
    for name, g_t, w_t in zip(names, got, want):
        w_t = torch.where(w_t < 0, torch.full_like(w_t, -7), w_t) if name.endswith("permutation") else w_t
        assert torch.equal(g_t, w_t.reshape(g_t.shape)), name
    # ids that do not start on a 16-byte boundary (scalar loads)
    for a, b in zip(got, run_prepare(gpu, ids, num_experts, n, k, shift=1)):
        assert torch.equal(a, b)
    # without the optional table
    got2 = run_prepare(gpu, ids, num_experts, n, k, with_blockscale=False)
    assert bool((got2[1] == -7).all())
    for a, b in zip(got[2:], got2[2:]):
        assert torch.equal(a, b)


def test_prepare_moe_input_is_the_same_on_every_run(gpu):
    ids = torch.randint(0, 32, (2048, 8), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    first = run_prepare(gpu, ids, 32, 256, 512)
    for _ in range(3):
        again = run_prepare(gpu, ids, 32, 256, 512)
        assert all(torch.equal(a, b) for a, b in zip(first, again))


@pytest.mark.parametrize("dtype,cols", [(FP8, 7168), (FP8, 100), (torch.float32, 56), (torch.float32, 1), (torch.bfloat16, 2048),
                                        (torch.bfloat16, 3), (torch.uint8, 13), (torch.int32, 4)])
def test_shuffle_rows(gpu, dtype, cols):
    """output[d] = input[map[d]] for rows of 16-byte pieces, 4-byte pieces and single bytes;
    repeated and unused source rows; map entries that name no row leave their destination alone."""
    from sglang_amd.sgl_kernel import shuffle_rows

    g = torch.Generator().manual_seed(cols)
    src_rows, dst_rows = 37, 91
    raw = torch.randint(0, 256, (src_rows, cols * torch.empty((), dtype=dtype).element_size()), generator=g, dtype=torch.uint8)
    x = raw.view(dtype) if dtype != torch.uint8 else raw
    dmap = torch.randint(0, src_rows, (dst_rows,), generator=g, dtype=torch.int32)
    say("shuffle_rows", dtype, cols)
    out = shuffle_rows(x.to(gpu), dmap.to(gpu), (dst_rows, cols)).cpu()
    assert out.dtype == dtype and out.shape == (dst_rows, cols)
    assert torch.equal(out.view(torch.uint8), O.shuffle_rows(x, dmap).view(torch.uint8))
    # fewer destination rows than map entries; an empty result
    out = shuffle_rows(x.to(gpu), dmap.to(gpu), (5, cols)).cpu()
    assert torch.equal(out.view(torch.uint8), O.shuffle_rows(x, dmap[:5]).view(torch.uint8))
    assert shuffle_rows(x.to(gpu), dmap.to(gpu), (0, cols)).shape == (0, cols)
    with pytest.raises(RuntimeError, match="one entry per output row"):
        shuffle_rows(x.to(gpu), dmap.to(gpu), (dst_rows + 1, cols))
    with pytest.raises(RuntimeError, match="int32"):
        shuffle_rows(x.to(gpu), dmap.to(gpu).long(), (dst_rows, cols))


def test_shuffle_rows_skips_entries_that_name_no_row(gpu):
    from sglang_amd import _lib

    x = torch.arange(8 * 16, dtype=torch.float32).reshape(8, 16)
    dmap = torch.tensor([3, -1, 8, 0, 7, 1 << 30], dtype=torch.int32)
    out = torch.full((6, 16), -5.0, dtype=torch.float32, device=gpu)
    xg, mg = x.to(gpu), dmap.to(gpu)
    rc = _lib.load().sglq_shuffle_rows(xg.data_ptr(), mg.data_ptr(), out.data_ptr(), 8, 6, 64, _lib.stream_ptr(gpu))
    assert rc == 0
    out = out.cpu()
    assert torch.equal(out[[0, 3, 4]], x[[3, 0, 7]])
    assert bool((out[[1, 2, 5]] == -5.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.half])
@pytest.mark.parametrize("tokens,d", [(1, 8), (5, 2048), (333, 256), (64, 4), (3, 12), (17, 7 * 8)])
def test_silu_and_mul(gpu, dtype, tokens, d):
    """T(silu(x)) * y with both roundings, against the oracle: the exponential differs between
    the host's and the device's libraries in the last bits, so the activation may land on the
    neighbouring 16-bit value, which moves the product by up to two units in the last place."""
    from sglang_amd.sgl_kernel import silu_and_mul

    g = torch.Generator().manual_seed(tokens + d)
    x = (torch.randn((tokens, 2 * d), generator=g) * 3).to(dtype)
    x[0, :4] = torch.tensor([0.0, -0.0, 30.0, -30.0], dtype=dtype)
    say("silu_and_mul", dtype, tokens, d)
    out = silu_and_mul(x.to(gpu)).cpu()
    want = O.silu_and_mul(x)
    assert out.shape == (tokens, d) and out.dtype == dtype
    ulp = (out.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert int(ulp.max()) <= 2, int(ulp.max())
    assert float((ulp != 0).float().mean()) < 0.005
    # into a caller's buffer, 3-D input
    buf = torch.empty((1, tokens, d), dtype=dtype, device=gpu)
    assert silu_and_mul(x.to(gpu).reshape(1, tokens, 2 * d), buf) is buf
    assert torch.equal(buf.cpu().reshape(tokens, d), out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.half])
@pytest.mark.parametrize("tokens,d", [(1, 128), (7, 2048), (333, 256), (4096, 384)])
def test_silu_and_mul_fused_with_group_quant(gpu, dtype, tokens, d):
    """One kernel for SiLU-and-multiply and the group quantization after it: codes and scales equal
    those of the two operators called one after the other, bit for bit (zero rows, large values
    and rows whose activation underflows included)."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import silu_and_mul
    from sglang_amd.sgl_kernel.moe import silu_and_mul_per_token_group_quant_fp8

    g = torch.Generator().manual_seed(tokens + d)
    x = (torch.randn((tokens, 2 * d), generator=g) * 3).to(dtype)
    x[0, :128] = 0
    x[tokens - 1, :64] = -40.0
    x[tokens // 2, d:d + 32] = 200.0
    say("silu_and_mul + group quant", dtype, tokens, d)
    xg = x.to(gpu)
    q2, s2 = sglang_per_token_group_quant_fp8(silu_and_mul(xg), 128)
    q1, s1 = silu_and_mul_per_token_group_quant_fp8(xg, 128)
    assert q1.shape == (tokens, d) and s1.shape == (tokens, d // 128) and s1.is_contiguous()
    assert_bits_equal(q1, q2, "codes")
    assert_bits_equal(s1, s2, "scales")
    # and the oracle's two steps on the device's activation (the exponential is the device's)
    oq, os_ = O.per_token_group_quant_fp8(silu_and_mul(xg).cpu(), 128)
    assert_bits_equal(q1, oq, "codes against the oracle")
    assert_bits_equal(s1, os_, "scales against the oracle")
    with pytest.raises(RuntimeError, match="multiple of 128"):
        silu_and_mul_per_token_group_quant_fp8(torch.zeros((2, 192), dtype=dtype, device=gpu))
    with pytest.raises(NotImplementedError):
        silu_and_mul_per_token_group_quant_fp8(torch.zeros((2, 256), dtype=torch.float32, device=gpu))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.half, torch.float32])
@pytest.mark.parametrize("m,topk,e,k", [(1, 1, 1, 128), (9, 2, 4, 256), (333, 8, 32, 384), (2048, 6, 16, 1024)])
def test_group_quant_written_to_expert_rows(gpu, dtype, m, topk, e, k):
    """One kernel for the per-token-group quantization and the two row gathers after it: on every
    row that a slot names, codes and scales equal those of the three operators called in turn, bit
    for bit; rows that no slot names (ids outside [0, E)) are not written."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import shuffle_rows
    from sglang_amd.sgl_kernel.moe import per_token_group_quant_fp8_to_expert_rows

    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn((m, k), generator=g) * 2).to(dtype)
    x[0, :128] = 0
    ids = torch.randint(0, e, (m, topk), generator=g, dtype=torch.int32)
    if m > 4:
        ids[1, 0] = -1
        ids[m - 1, topk - 1] = e
    say("group quant to expert rows", dtype, m, topk, e, k)
    offsets, _, _, _, a_map, c_map = run_prepare(gpu, ids, e, 64, k, fill=-1)
    total = int(offsets[-1])
    xg, a_map, c_map = x.to(gpu), a_map.to(gpu), c_map.to(gpu)
    q, s = sglang_per_token_group_quant_fp8(xg, 128)
    want_q, want_s = shuffle_rows(q, a_map, (m * topk, k)), shuffle_rows(s, a_map, (m * topk, k // 128))
    got_q, got_s = per_token_group_quant_fp8_to_expert_rows(xg, c_map, topk, 128)
    assert got_q.shape == (m * topk, k) and got_s.shape == (m * topk, k // 128)
    assert_bits_equal(got_q[:total], want_q[:total], "codes")
    assert_bits_equal(got_s[:total], want_s[:total], "scales")
    # nothing outside the named rows: through the C ABI into sentinel-filled buffers
    from sglang_amd import _lib
    from sglang_amd._lib import DTYPE_CODE

    out_q = torch.full((m * topk + 2, k), 0x55, dtype=torch.uint8, device=gpu)
    out_s = torch.full((m * topk + 2, k // 128), -3.0, dtype=torch.float32, device=gpu)
    rc = _lib.load().sglq_per_token_group_quant_fp8_scatter(xg.data_ptr(), DTYPE_CODE[dtype], out_q[1:].data_ptr(), out_s[1:].data_ptr(),
                                                            c_map.data_ptr(), m, k, topk, m * topk, 1e-10, _lib.stream_ptr(gpu))
    assert rc == 0
    assert torch.equal(out_q[1:1 + total], want_q[:total].view(torch.uint8))
    assert bool((out_q[0] == 0x55).all()) and bool((out_q[1 + total:] == 0x55).all())
    assert bool((out_s[0] == -3.0).all()) and bool((out_s[1 + total:] == -3.0).all())


def test_silu_and_mul_argument_checks(gpu):
    from sglang_amd.sgl_kernel import silu_and_mul

    with pytest.raises(ValueError, match="multiple of 16 bytes"):
        silu_and_mul(torch.zeros((2, 6), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(NotImplementedError):
        silu_and_mul(torch.zeros((2, 8), dtype=torch.float32, device=gpu))
    assert silu_and_mul(torch.zeros((0, 16), dtype=torch.bfloat16, device=gpu)).shape == (0, 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.half])
@pytest.mark.parametrize("m,topk,row", [(1, 1, 8), (11, 3, 64), (64, 8, 7168), (200, 6, 2048 + 8)])
def test_apply_shuffle_mul_sum(gpu, dtype, m, topk, row):
    """fp32 accumulation in slot order with one fused multiply-add per term and one rounding:
    bit for bit with the oracle, with factors and without."""
    from sglang_amd.sgl_kernel import apply_shuffle_mul_sum

    g = torch.Generator().manual_seed(m + row)
    c2 = torch.randn((m * topk, row), generator=g).to(dtype)
    c_map = torch.randperm(m * topk, generator=g).to(torch.int32)
    f = torch.rand((m, topk), generator=g).to(dtype)
    say("apply_shuffle_mul_sum", dtype, m, topk, row)
    for factors in (f, None):
        out = torch.full((m, row), 3.0, dtype=dtype, device=gpu)
        apply_shuffle_mul_sum(c2.to(gpu), out, c_map.to(gpu), None if factors is None else factors.to(gpu))
        assert_bits_equal(out.cpu().view(torch.int16), O.apply_shuffle_mul_sum(c2, c_map, factors, m).view(torch.int16),
                          f"combine {'with' if factors is not None else 'without'} factors")


def test_apply_shuffle_mul_sum_unrouted_slots_and_checks(gpu):
    from sglang_amd.sgl_kernel import apply_shuffle_mul_sum

    m, topk, row = 4, 2, 16
    c2 = torch.arange(m * topk * row, dtype=torch.float32).reshape(m * topk, row).to(torch.bfloat16)
    c_map = torch.tensor([0, -1, 2, 3, 99, 5, 6, 7], dtype=torch.int32)
    f = torch.ones((m, topk), dtype=torch.bfloat16)
    out = torch.empty((m, row), dtype=torch.bfloat16, device=gpu)
    apply_shuffle_mul_sum(c2.to(gpu), out, c_map.to(gpu), f.to(gpu))
    want = torch.stack([c2[0].float(), c2[2].float() + c2[3].float(), c2[5].float(), c2[6].float() + c2[7].float()]).to(torch.bfloat16)
    assert torch.equal(out.cpu(), want)
    with pytest.raises(RuntimeError, match="Factors must match output dtype"):
        apply_shuffle_mul_sum(c2.to(gpu), out, c_map.to(gpu), f.half().to(gpu))
    with pytest.raises(RuntimeError, match="permutation size must match"):
        apply_shuffle_mul_sum(c2.to(gpu), out, c_map[:7].to(gpu), None)
    with pytest.raises(RuntimeError, match="Half or BFloat16"):
        apply_shuffle_mul_sum(c2.float().to(gpu), out.float(), c_map.to(gpu), None)


def run_layer(gpu, c, dtype):
    """cutlass_fused_experts_fp8 with the buffers its caller allocates
    (python/sglang/test/test_cutlass_moe.py:84-121)."""
    from sglang_amd.moe.cutlass_moe import cutlass_fused_experts_fp8

    e, k, n = c["w1_q"].shape[0], c["w1_q"].shape[1], c["w2_q"].shape[1]
    col_major = lambda w: w.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    i64 = lambda v: torch.full((e,), v, dtype=torch.int64, device=gpu)
    ptrs = lambda: torch.empty((e,), dtype=torch.int64, device=gpu)
    return cutlass_fused_experts_fp8(
        c["x"].to(gpu), col_major(c["w1_q"]), col_major(c["w2_q"]), c["w1_s"].to(gpu), c["w2_s"].to(gpu),
        c["tw"].to(gpu), c["ids"].to(gpu), i64(k), i64(2 * n), i64(n), i64(k),
        torch.empty((7182 * 1024,), dtype=torch.uint8, device=gpu), ptrs(), ptrs(), ptrs(), ptrs(), ptrs(),
        torch.empty((e + 1,), dtype=torch.int32, device=gpu), torch.empty((e, 3), dtype=torch.int32, device=gpu),
        torch.empty((e, 3), dtype=torch.int32, device=gpu))


def close_as_a_layer(out, want):
    """Two runs of the layer on the same inputs differ where an intermediate 16-bit value falls on
    the other side of a rounding boundary (summation order in the GEMM, the exponential): that can
    change single FP8 codes of the second GEMM's input, each worth up to 1/8 of one activation
    times one weight in the output.  So: the GEMM tolerance on all but a few per cent of the outputs, and a bound
    on the largest difference relative to the outputs' scale."""
    out, want = out.float(), want.float()
    diff = (out - want).abs()
    outside = diff > ATOL + RTOL * want.abs()
    rms = float(want.pow(2).mean().sqrt())
    assert float(outside.float().mean()) < 0.05, float(outside.float().mean())
    assert float(diff.max()) < 0.15 * max(rms, 1e-3), (float(diff.max()), rms)


def layer_by_stages(gpu, c, dtype):
    """The layer's call sequence (cutlass_moe.py:140-222) step by step, every step checked against
    the oracle's restatement of that step ON THE DEVICE'S OWN INPUTS to it, so that no rounding
    difference carries over from one step into the next one's comparison."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import (apply_shuffle_mul_sum, fp8_blockwise_scaled_grouped_mm, prepare_moe_input, shuffle_rows,
                                       silu_and_mul)

    e, k, n = c["w1_q"].shape[0], c["w1_q"].shape[1], c["w2_q"].shape[1]
    m, topk = c["ids"].shape
    col_major = lambda w: w.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    w1, w2, s1, s2 = col_major(c["w1_q"]), col_major(c["w2_q"]), c["w1_s"].to(gpu), c["w2_s"].to(gpu)
    x, ids = c["x"].to(gpu), c["ids"].to(gpu)
    offsets = torch.empty((e + 1,), dtype=torch.int32, device=gpu)
    ps1, ps2 = torch.empty((e, 3), dtype=torch.int32, device=gpu), torch.empty((e, 3), dtype=torch.int32, device=gpu)
    a_map = torch.empty((m * topk,), dtype=torch.int32, device=gpu)
    c_map = torch.full((m * topk,), -1, dtype=torch.int32, device=gpu)
    prepare_moe_input(ids, offsets, ps1, ps2, a_map, c_map, e, n, k)
    o_off, _, o_ps1, o_ps2, o_amap, o_cmap = O.prepare_moe_input(c["ids"], e, n, k)
    total = int(o_off[-1])
    assert torch.equal(offsets.cpu(), o_off) and torch.equal(ps1.cpu(), o_ps1) and torch.equal(ps2.cpu(), o_ps2)
    assert torch.equal(a_map.cpu()[:total], o_amap[:total]) and torch.equal(c_map.cpu(), o_cmap)

    a_q, a_s = sglang_per_token_group_quant_fp8(x, 128)
    o_q, o_s = O.per_token_group_quant_fp8(c["x"], 128)
    assert_bits_equal(a_q, o_q, "activation codes")
    assert_bits_equal(a_s, o_s, "activation scales")
    rep_q, rep_s = shuffle_rows(a_q, a_map, (m * topk, k)), shuffle_rows(a_s, a_map, (m * topk, k // 128))
    assert_bits_equal(rep_q[:total], O.shuffle_rows(o_q, o_amap[:total]), "gathered codes")
    assert_bits_equal(rep_s[:total], O.shuffle_rows(o_s, o_amap[:total]), "gathered scales")

    i64 = lambda: torch.empty((e,), dtype=torch.int64, device=gpu)
    layout = lambda: torch.empty((e, 5), dtype=torch.int32, device=gpu)
    workspace = torch.empty((1 << 20,), dtype=torch.uint8, device=gpu)
    gmm = lambda out, a, b, sa, sb, ps: fp8_blockwise_scaled_grouped_mm(out, i64(), i64(), i64(), i64(), i64(), a, b, sa, sb, i64(), i64(),
                                                                        i64(), layout(), layout(), ps, offsets[:-1], workspace)
    c1 = torch.zeros((m * topk, 2 * n), dtype=dtype, device=gpu)
    gmm(c1, rep_q, w1, rep_s, s1, ps1)
    o_c1 = O.fp8_blockwise_scaled_grouped_mm(rep_q.cpu()[:total], c["w1_q"], rep_s.cpu()[:total], c["w1_s"], o_ps1, o_off[:-1], dtype)
    torch.testing.assert_close(c1.cpu()[:total].float(), o_c1.float(), rtol=RTOL, atol=ATOL)

    inter = silu_and_mul(c1)
    ulp = (inter.cpu()[:total].view(torch.int16).int() - O.silu_and_mul(c1.cpu()[:total]).view(torch.int16).int()).abs()
    assert int(ulp.max()) <= 2 and float((ulp != 0).float().mean()) < 0.005
    inter_q, inter_s = sglang_per_token_group_quant_fp8(inter, 128)
    o_iq, o_is = O.per_token_group_quant_fp8(inter.cpu()[:total], 128)
    assert_bits_equal(inter_q[:total], o_iq, "intermediate codes")
    assert_bits_equal(inter_s[:total], o_is, "intermediate scales")

    c2 = torch.zeros((m * topk, k), dtype=dtype, device=gpu)
    gmm(c2, inter_q, w2, inter_s, s2, ps2)
    o_c2 = O.fp8_blockwise_scaled_grouped_mm(inter_q.cpu()[:total], c["w2_q"], inter_s.cpu()[:total], c["w2_s"], o_ps2, o_off[:-1], dtype)
    torch.testing.assert_close(c2.cpu()[:total].float(), o_c2.float(), rtol=RTOL, atol=ATOL)

    result = torch.empty((m, k), dtype=dtype, device=gpu)
    tw = c["tw"].to(gpu).to(dtype)
    apply_shuffle_mul_sum(c2, result, c_map, tw)
    assert_bits_equal(result.view(torch.int16), O.apply_shuffle_mul_sum(c2.cpu(), o_cmap, tw.cpu(), m).view(torch.int16), "combined rows")
    return result


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.half])
@pytest.mark.parametrize("m,topk,e,n,k", [(1, 2, 4, 128, 256), (24, 2, 4, 128, 256), (64, 4, 8, 256, 512), (333, 8, 32, 256, 384),
                                          (2048, 2, 4, 256, 512)])
def test_fused_experts_layer_against_the_oracle(gpu, dtype, m, topk, e, n, k):
    """Every step of the layer against the oracle on the same inputs (codes, scales, tables and
    the combine bit for bit; the GEMMs within rtol 1e-2 / atol 1e-2); cutlass_fused_experts_fp8
    returns that chain's result bit for bit; and the oracle's end-to-end chain is close."""
    c = moe_layer_case(m, topk, e, n, k, seed=m + e, dtype=dtype)
    say("fused experts layer", dtype, m, topk, e, n, k)
    staged = layer_by_stages(gpu, c, dtype)
    out = run_layer(gpu, c, dtype)
    assert out.dtype == dtype and out.shape == (m, k)
    assert torch.equal(out.view(torch.int16), staged.view(torch.int16))
    want = O.cutlass_fused_experts_fp8(c["x"], c["w1_q"], c["w2_q"], c["w1_s"], c["w2_s"], c["tw"], c["ids"])
    close_as_a_layer(out.cpu(), want)


def test_fused_experts_layer_replays_from_a_graph(gpu):
    """Every step launches on the current stream and reads its sizes on the device: the layer can be
    captured once and replayed on new activations and a new routing."""
    from sglang_amd.moe.cutlass_moe import cutlass_fused_experts_fp8  # noqa: F401

    m, topk, e, n, k = 48, 2, 8, 128, 256
    c = moe_layer_case(m, topk, e, n, k, seed=3)
    col_major = lambda w: w.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    w1, w2, s1, s2 = col_major(c["w1_q"]), col_major(c["w2_q"]), c["w1_s"].to(gpu), c["w2_s"].to(gpu)
    x, ids, tw = c["x"].to(gpu), c["ids"].to(gpu), c["tw"].to(gpu)
    i64 = lambda v: torch.full((e,), v, dtype=torch.int64, device=gpu)
    bufs = [torch.empty((1 << 20,), dtype=torch.uint8, device=gpu)] + [torch.empty((e,), dtype=torch.int64, device=gpu) for _ in range(5)] + \
           [torch.empty((e + 1,), dtype=torch.int32, device=gpu), torch.empty((e, 3), dtype=torch.int32, device=gpu),
            torch.empty((e, 3), dtype=torch.int32, device=gpu)]
    strides = (i64(k), i64(2 * n), i64(n), i64(k))
    call = lambda: cutlass_fused_experts_fp8(x, w1, w2, s1, s2, tw, ids, *strides, *bufs)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        call()
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call()
    for seed in (4, 5, 6):
        c2 = moe_layer_case(m, topk, e, n, k, seed=seed)
        x.copy_(c2["x"].to(gpu)); ids.copy_(c2["ids"].to(gpu)); tw.copy_(c2["tw"].to(gpu))
        graph.replay()
        torch.cuda.synchronize()
        eager = call()
        assert torch.equal(out, eager), seed
        want = O.cutlass_fused_experts_fp8(c2["x"], c["w1_q"], c["w2_q"], c["w1_s"], c["w2_s"], c2["tw"], c2["ids"])
        close_as_a_layer(out.cpu(), want)


def test_fused_experts_layer_with_slots_routed_to_nobody(gpu):
    """Expert ids outside [0, E) (tokens whose expert lives on another rank): those slots add
    nothing, the rest of the token's sum is unchanged."""
    m, topk, e, n, k = 40, 2, 4, 128, 256
    c = moe_layer_case(m, topk, e, n, k, seed=12)
    c["ids"][::3, 1] = -1
    c["ids"][5, 0] = e
    out = run_layer(gpu, c, torch.bfloat16).cpu()
    want = O.cutlass_fused_experts_fp8(c["x"], c["w1_q"], c["w2_q"], c["w1_s"], c["w2_s"], c["tw"], c["ids"])
    close_as_a_layer(out, want)
