#!/usr/bin/env python3
"""Writes tests/golden/w8a8_small.npz: small seeded inputs of every operator on the path and the
outputs of this repository's own CPU oracle for them (codes, scales, INT32 accumulators, fp32
and bf16 GEMM outputs), as plain numeric arrays.

    python tests/golden/make_fixtures.py

The reference holds no golden vectors for this path (its tests draw fresh random tensors) and
none of its code is run here: the fixture pins the oracle against drift, e.g. a different torch
build whose CPU float8 casts or matmuls round differently on the machine that runs the GPU tests.
Stored as raw bit patterns (uint8 / uint16 / int32) so that loading executes nothing and depends
on no dtype support in numpy."""
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
from oracle import w8a8_oracle as O  # noqa: E402

OUT = Path(__file__).resolve().parent / "w8a8_small.npz"


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def bits8(t):
    return t.contiguous().view(torch.uint8).numpy()


def bits32(t):
    return t.contiguous().view(torch.int32).numpy()


def build():
    m, k, n = 4, 256, 128
    d = {}
    x = O.gen_activation(m, k, seed=77, outliers=True)
    x[1, 128:] = 0  # an all-zero group and, for the per-token ops below, nothing special
    x[2, :] = 0     # an all-zero row
    d["x_bf16"] = bits16(x)
    # a1 group quantization, groups of 128 and of 32
    for gs in (128, 32):
        q, s = O.per_token_group_quant_fp8(x, gs)
        d[f"group{gs}_codes"], d[f"group{gs}_scales"] = bits8(q), bits32(s)
    q, s = O.per_token_group_quant_8bit(x, 128, 1e-10, -128.0, 127.0, torch.int8)
    d["group128_int8_codes"], d["group128_int8_scales"] = q.numpy(), bits32(s)
    # a2 / a3 per-token quantization
    q8, s8 = O.per_token_quant_int8(x)
    d["token_int8_codes"], d["token_int8_scales"] = q8.numpy(), bits32(s8)
    qf, sf = O.per_token_quant_fp8(x)
    d["token_fp8_codes"], d["token_fp8_scales"] = bits8(qf), bits32(sf)
    # per-tensor quantization, dynamic and static
    qt, st = O.per_tensor_quant_fp8(x)
    d["tensor_fp8_codes"], d["tensor_fp8_scale"] = bits8(qt), bits32(st)
    qs, _ = O.per_tensor_quant_fp8(x, torch.tensor([0.03125]))
    d["tensor_fp8_static_codes"] = bits8(qs)
    # a4 block-scaled FP8 GEMM
    w = O.gen_weight(n, k, seed=78)
    wq, ws = O.block_quant_weight(w)
    d["w_block_codes"], d["w_block_scales"] = bits8(wq), bits32(ws)
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    out32 = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32)
    d["block_mm_fp32"] = bits32(out32)
    d["block_mm_bf16"] = bits16(O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16))
    # a5 INT8 GEMM
    wt, s_b, bias = O.gen_int8_weight(k, n, seed=79)
    d["w_int8"], d["w_int8_scales"], d["bias_bf16"] = wt.t().contiguous().numpy(), bits32(s_b), bits16(bias)
    d["int8_acc"] = O.int8_mm_i32(q8, wt).numpy()
    d["int8_mm_bf16"] = bits16(O.int8_scaled_mm(q8, wt, s8, s_b, torch.bfloat16, bias))
    # a6 per-token / per-channel FP8 GEMM
    wq2, ws2 = O.per_tensor_quant_weight(w)
    d["w_tensor_codes"], d["w_tensor_scales"] = bits8(wq2), bits32(ws2)
    d["fp8_mm_bf16"] = bits16(O.fp8_scaled_mm(qf, wq2.t(), sf, ws2, torch.bfloat16, bias))
    d["fp8_mm_fp32"] = bits32(O.fp8_scaled_mm(qf, wq2.t(), sf, ws2, torch.float32, bias))
    # power-of-two (UE8M0) group scales: codes, exponent bytes, packed words; the block-scaled GEMM on them with a
    # weight whose block scales are rounded up to powers of two (python/sglang/srt/layers/quantization/fp8_utils.py:468-486)
    uq, ue, up = O.per_token_group_quant_fp8_ue8m0(x)
    d["group128_ue8m0_codes"], d["group128_ue8m0_exponents"] = bits8(uq), ue.numpy()
    d["group128_ue8m0_packed"] = up.contiguous().numpy()
    blocks = w.float().view(n // 128, 128, k // 128, 128)
    y = blocks.abs().amax(dim=(1, 3), keepdim=True).clamp(1e-4) / 448.0
    yb = y.view(torch.int32)
    sf = (((yb >> 23) + ((yb & 0x7FFFFF) != 0).to(torch.int32)) << 23).view(torch.float32)
    wq_u = (blocks / sf).to(torch.float8_e4m3fn).view(n, k).contiguous()
    ws_u = sf.view(n // 128, k // 128).contiguous()
    d["w_block_ue8m0_codes"], d["w_block_ue8m0_scales"] = bits8(wq_u), bits32(ws_u)
    us = torch.pow(2.0, ue.float() - 127.0)
    d["block_ue8m0_mm_fp32"] = bits32(O.fp8_blockwise_scaled_mm(uq, wq_u.t(), us, ws_u.t(), torch.float32))
    return d


if __name__ == "__main__":
    data = build()
    np.savez_compressed(OUT, **data)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(data)} arrays)")
