"""Committed golden vectors (tests/golden/w8a8_small.npz, written by tests/golden/make_fixtures.py
from this repository's CPU oracle): the oracle must reproduce them on whatever machine runs the
tests (a different torch build must not move the checker silently: codes, scales and integer
accumulators bit for bit, floating-point GEMM outputs to the rounding of the sum), and the HIP kernels must
reproduce them through the operator layer: codes, scales and INT32 accumulators bit for bit, GEMM
outputs within rtol/atol 1e-2 of the fixture's fp32 results.  Collected first on purpose."""
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent / "golden"))
import make_fixtures  # noqa: E402

from oracle import w8a8_oracle as O  # noqa: E402,F401

FIXTURE = Path(__file__).resolve().parent / "golden" / "w8a8_small.npz"
FP8 = torch.float8_e4m3fn


def load():
    with np.load(FIXTURE, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def t16(a, dtype=torch.bfloat16):
    return torch.from_numpy(a.view(np.int16).copy()).view(dtype)


def t8(a):
    return torch.from_numpy(a.copy()).view(FP8)


def f32(a):
    return torch.from_numpy(a.copy()).view(torch.float32)


def check_oracle_reproduces_the_fixture():
    want = load()
    got = make_fixtures.build()
    assert sorted(got) == sorted(want)
    for name in sorted(want):
        assert got[name].dtype == want[name].dtype and got[name].shape == want[name].shape, name
        if name.endswith("_mm_fp32") or name.endswith("_mm_bf16"):
            # floating-point GEMM outputs: the host's matmul fixes no summation order (it changes with the
            # core count), so these agree to fp32 rounding of a 256-term sum, or one unit of bf16
            g, w = (f32(got[name]), f32(want[name])) if name.endswith("fp32") else (t16(got[name]).float(), t16(want[name]).float())
            rtol = 1e-5 if name.endswith("fp32") else 2.0**-7
            torch.testing.assert_close(g, w, rtol=rtol, atol=1e-6, msg=lambda m: f"oracle output {name} is not the committed fixture's: {m}")
        else:
            assert np.array_equal(got[name], want[name]), f"oracle output {name} differs from the committed fixture"


def test_oracle_reproduces_the_fixture_on_this_machine():
    check_oracle_reproduces_the_fixture()


@pytest.mark.gpu
def test_oracle_reproduces_the_fixture_on_the_gpu_box(gpu):
    check_oracle_reproduces_the_fixture()


def same_bits(got: torch.Tensor, want: np.ndarray, what: str):
    g = got.detach().cpu().contiguous()
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[g.element_size()]
    gb = g.view(view).numpy().view(want.dtype)
    assert gb.shape == want.shape, f"{what}: shape {gb.shape} != {want.shape}"
    bad = np.argwhere(gb != want)
    assert bad.size == 0, f"{what}: {len(bad)} elements differ from the fixture, first at {bad[:4].tolist()}"


@pytest.mark.gpu
def test_quant_kernels_reproduce_the_fixture(gpu):
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant, sglang_per_token_group_quant_fp8, sglang_per_token_quant_fp8
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8, sglang_per_token_group_quant_int8

    print("golden: quant kernels", flush=True)
    z = load()
    x = t16(z["x_bf16"]).to(gpu)
    for gs in (128, 32):
        for cm in (False, True):
            q, s = sglang_per_token_group_quant_fp8(x, gs, column_major_scales=cm)
            same_bits(q, z[f"group{gs}_codes"], f"group {gs} codes")
            same_bits(s.contiguous(), z[f"group{gs}_scales"], f"group {gs} scales")
    q, s = sglang_per_token_group_quant_int8(x, 128)
    same_bits(q, z["group128_int8_codes"], "group int8 codes")
    same_bits(s, z["group128_int8_scales"], "group int8 scales")
    q, s = per_token_quant_int8(x)
    same_bits(q, z["token_int8_codes"], "token int8 codes")
    same_bits(s, z["token_int8_scales"], "token int8 scales")
    q, s = sglang_per_token_quant_fp8(x)
    same_bits(q, z["token_fp8_codes"], "token fp8 codes")
    same_bits(s, z["token_fp8_scales"], "token fp8 scales")
    q, s = scaled_fp8_quant(x)
    same_bits(q, z["tensor_fp8_codes"], "tensor fp8 codes")
    same_bits(s, z["tensor_fp8_scale"], "tensor fp8 scale")
    q, _ = scaled_fp8_quant(x, torch.tensor([0.03125], device=gpu))
    same_bits(q, z["tensor_fp8_static_codes"], "tensor fp8 static codes")


@pytest.mark.gpu
def test_gemm_kernels_reproduce_the_fixture(gpu):
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_mm_i32, int8_scaled_mm

    print("golden: GEMM kernels", flush=True)
    z = load()
    bias = t16(z["bias_bf16"]).to(gpu)
    # block-scaled FP8
    xq, xs = t8(z["group128_codes"]).to(gpu), f32(z["group128_scales"]).to(gpu)
    wq, ws = t8(z["w_block_codes"]).to(gpu), f32(z["w_block_scales"]).to(gpu)
    out = fp8_blockwise_scaled_mm(xq, wq.t(), xs.t().contiguous().t(), ws.t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), f32(z["block_mm_fp32"]), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.cpu().float(), t16(z["block_mm_bf16"]).float(), rtol=1e-2, atol=1e-2)
    # INT8: accumulators exact, output within tolerance
    a8, s8 = torch.from_numpy(z["token_int8_codes"].copy()).to(gpu), f32(z["token_int8_scales"]).to(gpu)
    w8, sb = torch.from_numpy(z["w_int8"].copy()).to(gpu), f32(z["w_int8_scales"]).to(gpu)
    same_bits(int8_mm_i32(a8, w8.t()), z["int8_acc"], "INT32 accumulators")
    out = int8_scaled_mm(a8, w8.t(), s8, sb, torch.bfloat16, bias)
    torch.testing.assert_close(out.cpu().float(), t16(z["int8_mm_bf16"]).float(), rtol=1e-2, atol=1e-2)
    # per-token / per-channel FP8
    af, sf = t8(z["token_fp8_codes"]).to(gpu), f32(z["token_fp8_scales"]).to(gpu)
    wt, wts = t8(z["w_tensor_codes"]).to(gpu), f32(z["w_tensor_scales"]).to(gpu)
    out = fp8_scaled_mm(af, wt.t(), sf, wts, torch.bfloat16, bias)
    torch.testing.assert_close(out.cpu().float(), f32(z["fp8_mm_fp32"]), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.cpu().float(), t16(z["fp8_mm_bf16"]).float(), rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
def test_power_of_two_scale_kernels_reproduce_the_fixture(gpu):
    """UE8M0 group quantization (fp32 powers of two and the packed words of scale_ue8m0=True) bit for bit,
    the block-scaled GEMM that applies such scales inside the matrix instruction within tolerance."""
    from sglang_amd.quantization.fp8_kernel import per_token_group_quant_fp8_pow2, sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    print("golden: power-of-two scales", flush=True)
    z = load()
    x = t16(z["x_bf16"]).to(gpu)
    want_s = torch.pow(2.0, torch.from_numpy(z["group128_ue8m0_exponents"].astype(np.float32)) - 127.0)
    for cm in (False, True):
        q, s = per_token_group_quant_fp8_pow2(x, 128, column_major_scales=cm)
        same_bits(q, z["group128_ue8m0_codes"], "UE8M0 codes")
        assert torch.equal(s.cpu(), want_s), "UE8M0 scales are not 2^(exponent byte - 127)"
    q, packed = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True, scale_ue8m0=True)
    same_bits(q, z["group128_ue8m0_codes"], "UE8M0 codes (packed-scale kernel)")
    assert np.array_equal(packed.cpu().contiguous().numpy(), z["group128_ue8m0_packed"]), "packed UE8M0 words differ from the fixture"
    xq, wq = t8(z["group128_ue8m0_codes"]).to(gpu), t8(z["w_block_ue8m0_codes"]).to(gpu)
    xs, ws = want_s.to(gpu), f32(z["w_block_ue8m0_scales"]).to(gpu)
    out = fp8_blockwise_scaled_mm_ue8m0(xq, wq.t(), xs.t().contiguous().t(), ws.t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), f32(z["block_ue8m0_mm_fp32"]), rtol=1e-2, atol=1e-2)
