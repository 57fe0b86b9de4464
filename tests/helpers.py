"""Shared helpers for the tests: dtype plumbing between torch and the C oracle."""
import ctypes

import numpy as np
import torch

DT = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def raw_ptr(t: torch.Tensor):
    return ctypes.c_void_p(t.data_ptr())


def c_group_quant_fp8(lib, x: torch.Tensor, group: int, eps=1e-10, lo=-448.0, hi=448.0):
    x = x.contiguous()
    n = x.numel()
    q = torch.empty(n, dtype=torch.uint8)
    s = torch.empty(n // group, dtype=torch.float32)
    lib.oracle_group_quant_fp8(raw_ptr(x), DT[x.dtype], ctypes.c_int64(n // group), ctypes.c_int(group),
                               ctypes.c_float(eps), ctypes.c_float(lo), ctypes.c_float(hi), raw_ptr(q), raw_ptr(s))
    return q.reshape(x.shape), s.reshape(x.shape[:-1] + (x.shape[-1] // group,))


def c_token_quant_int8(lib, x: torch.Tensor):
    x = x.contiguous()
    rows, cols = x.numel() // x.shape[-1], x.shape[-1]
    q = torch.empty(x.shape, dtype=torch.int8)
    s = torch.empty(rows, dtype=torch.float32)
    lib.oracle_token_quant_int8(raw_ptr(x), DT[x.dtype], ctypes.c_int64(rows), ctypes.c_int64(cols), raw_ptr(q), raw_ptr(s))
    return q, s.reshape(x.shape[:-1] + (1,))


def c_token_quant_fp8(lib, x: torch.Tensor):
    x = x.contiguous()
    rows, cols = x.shape
    q = torch.empty(x.shape, dtype=torch.uint8)
    s = torch.empty(rows, dtype=torch.float32)
    lib.oracle_token_quant_fp8(raw_ptr(x), DT[x.dtype], ctypes.c_int64(rows), ctypes.c_int64(cols), raw_ptr(q), raw_ptr(s))
    return q, s.reshape(rows, 1)


def c_tensor_quant_fp8(lib, x: torch.Tensor, scale=None):
    x = x.contiguous()
    q = torch.empty(x.shape, dtype=torch.uint8)
    s = torch.zeros(1, dtype=torch.float32) if scale is None else scale.clone().float().reshape(1)
    lib.oracle_tensor_quant_fp8(raw_ptr(x), DT[x.dtype], ctypes.c_int64(x.numel()), ctypes.c_int(0 if scale is None else 1),
                                raw_ptr(q), raw_ptr(s))
    return q, s


def fp8_bits(t: torch.Tensor) -> torch.Tensor:
    return t.view(torch.uint8)


def f32_bits(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.int32)


def assert_bits_equal(got: torch.Tensor, want: torch.Tensor, what: str):
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    if got.dtype == torch.float32:
        got, want = f32_bits(got), f32_bits(want)
    elif got.dtype == torch.float8_e4m3fn:
        got, want = fp8_bits(got), fp8_bits(want)
    bad = (got != want)
    nbad = int(bad.sum())
    if nbad:
        idx = bad.nonzero()[:5].tolist()
        raise AssertionError(f"{what}: {nbad} of {got.numel()} elements differ, first at {idx}: "
                             f"got {[got[tuple(i)].item() for i in idx]} want {[want[tuple(i)].item() for i in idx]}")


FP8 = torch.float8_e4m3fn


def rows_per_tile(m: int, cap: int = 48, seed: int = 0, tile: int = 0) -> torch.Tensor:
    """Rows on which a large GEMM is compared with the oracle, chosen so that every row tile of
    every kernel is read: the first, the last and one random row of each 64-row tile up to
    M = 1024 and of each 256-row tile (the persistent kernels' tile height, which also covers
    their second-round tiles and the hand-over between consecutive tiles of a block) above,
    plus one row for each of the 16 positions inside an MFMA fragment and the rows 1 and M - 2.
    Up to `cap` rows all rows are taken.  `tile`: another tile height (the 192-row kernel)."""
    if m <= cap:
        return torch.arange(m)
    g = torch.Generator().manual_seed(1000003 * seed + m)
    tile = tile or (64 if m <= 1024 else 256)
    rows = [0, 1, m - 2, m - 1]
    for t0 in range(0, m, tile):
        t1 = min(m, t0 + tile)
        rows += [t0, t1 - 1, t0 + int(torch.randint(0, t1 - t0, (1,), generator=g))]
    for pos in range(16):  # every lane row of a 16-row fragment, each in a random fragment
        frag = int(torch.randint(0, m // 16, (1,), generator=g))
        rows.append(frag * 16 + pos)
    return torch.tensor(sorted(set(r for r in rows if 0 <= r < m)))


def moe_case(num_experts, rows_per_expert, n, k, seed, dtype=torch.bfloat16):
    """Inputs built the way the reference's grouped-GEMM test builds them
    (sgl-kernel/tests/test_fp8_blockwise_moe.py:39-63,119-190): N(0,1) activations quantized per
    token and 128 columns with amax clamped at 1e-4, N(0,1) weights quantized per 128 x 128 block,
    experts' rows stacked, K-major activation scales, [E, K/128, N/128] weight scales."""
    g = torch.Generator().manual_seed(seed)
    offsets, sizes, a_orig, b_orig, aq, asc, bq, bsc = [0], [], [], [], [], [], [], []
    for m_g in rows_per_expert:
        offsets.append(offsets[-1] + m_g)
        sizes.append([m_g, n, k])
        a = torch.randn((m_g, k), generator=g).to(dtype)
        b = torch.randn((n, k), generator=g).to(dtype)
        av = a.float().view(m_g, k // 128, 128)
        amax = av.abs().amax(dim=2).clamp(1e-4)
        aq.append((av * (448.0 / amax.unsqueeze(2))).to(FP8).view(m_g, k))
        asc.append(amax / 448.0)
        bv = b.float().view(n // 128, 128, k // 128, 128)
        bmax = bv.abs().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
        bq.append((bv * (448.0 / bmax)).to(FP8).view(n, k))
        bsc.append((bmax / 448.0).view(n // 128, k // 128).t().contiguous())  # [K/128, N/128]
        a_orig.append(a)
        b_orig.append(b)
    return dict(
        a=torch.cat(aq) if aq else torch.empty((0, k), dtype=FP8), b=torch.stack(bq).transpose(1, 2),
        scales_a=torch.cat(asc), scales_b=torch.stack(bsc),
        problem_sizes=torch.tensor(sizes, dtype=torch.int32), expert_offsets=torch.tensor(offsets[:-1], dtype=torch.int32),
        a_orig=a_orig, b_orig=b_orig)


def calc_diff(x, y):
    # the reference test's criterion (sgl-kernel/tests/test_fp8_blockwise_moe.py:29-33)
    x, y = x.double(), y.double()
    return float(1 - 2 * (x * y).sum() / (x * x + y * y).sum())


def moe_layer_case(m, topk, num_experts, n, k, seed, dtype=torch.bfloat16, w_std=0.1):
    """One MoE expert layer's inputs in the layout python/sglang/srt/layers/moe/cutlass_moe.py:30-139
    documents: x [m, k]; w1_q [E, k, 2 n] and w2_q [E, n, k] e4m3fn (transposed views of the
    [E, 2 n, k] / [E, k, n] weights, quantized per 128 x 128 block); w1_s [E, k/128, 2 n/128] and
    w2_s [E, n/128, k/128]; distinct expert ids per token and softmax weights."""
    from oracle import w8a8_oracle as O

    g = torch.Generator().manual_seed(seed)
    x = torch.randn((m, k), generator=g).to(dtype)
    w1 = torch.randn((num_experts, 2 * n, k), generator=g) * w_std
    w2 = torch.randn((num_experts, k, n), generator=g) * w_std
    q = lambda w: [O.block_quant_weight(w[i]) for i in range(w.shape[0])]
    w1q, w2q = q(w1), q(w2)
    ids = torch.stack([torch.randperm(num_experts, generator=g)[:topk] for _ in range(m)]).to(torch.int32).reshape(m, topk)
    tw = torch.softmax(torch.rand((m, topk), generator=g), dim=-1)
    return dict(
        x=x, ids=ids, tw=tw,
        w1_q=torch.stack([t[0] for t in w1q]).transpose(1, 2), w1_s=torch.stack([t[1] for t in w1q]).transpose(1, 2),
        w2_q=torch.stack([t[0] for t in w2q]).transpose(1, 2), w2_s=torch.stack([t[1] for t in w2q]).transpose(1, 2))
