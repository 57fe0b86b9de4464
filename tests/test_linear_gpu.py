"""End-to-end glue (quantize -> GEMM -> bias) against the oracle's same sequence."""
import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu


def test_block_fp8_linear_config0(gpu):
    """A[256,7168] with 1% x20 outliers, W[2048,7168] block-quantized, bias added by the caller."""
    from sglang_amd.quantization.fp8_utils import w8a8_block_fp8_linear

    print("block fp8 linear cfg0", flush=True)
    x = O.gen_activation(256, 7168, seed=0, outliers=True)
    wq, ws = O.block_quant_weight(O.gen_weight(2048, 7168, seed=0))
    bias = (torch.randn(2048, generator=torch.Generator().manual_seed(1)) * 0.1).to(torch.bfloat16)
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    mm = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32)
    ref = mm + bias.float()
    out = w8a8_block_fp8_linear(x.to(gpu).view(2, 128, 7168), wq.to(gpu), [128, 128], ws.to(gpu), bias=bias.to(gpu))
    assert tuple(out.shape) == (2, 128, 2048) and out.dtype == torch.bfloat16
    # the caller rounds the GEMM output to bf16 before adding the bias (fp8_utils.py:207-211):
    # allow one bf16 ulp of that intermediate on top of the path's rtol/atol of 1e-2
    tol = 1e-2 + 1e-2 * ref.abs() + mm.abs() * 2.0**-8
    err = (out.cpu().view(256, 2048).float() - ref).abs()
    assert bool((err <= tol).all()), f"max excess {(err - tol).max().item()}"


def test_int8_linear(gpu):
    from sglang_amd.quantization.w8a8_int8 import apply_w8a8_int8_linear, process_weights_after_loading

    print("int8 linear", flush=True)
    x = O.gen_activation(16, 4096, seed=1001)
    wt, s_b, bias = O.gen_int8_weight(4096, 14336, seed=1000)
    xq, xs = O.per_token_quant_int8(x)
    ref = O.int8_scaled_mm(xq, wt, xs, s_b, torch.bfloat16, bias)
    w_stored = wt.t().contiguous().to(gpu)  # [N, K] as loaded
    w_view, w_scale = process_weights_after_loading(w_stored, s_b.reshape(-1, 1).to(gpu))
    out = apply_w8a8_int8_linear(x.to(gpu), w_view, w_scale, bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_fp8_per_channel_linear(gpu):
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print("fp8 linear", flush=True)
    x = O.gen_activation(32, 4096, seed=3001)
    wq, ws = O.per_tensor_quant_weight(O.gen_weight(6144, 4096, seed=3000))
    xq, xs = O.per_token_quant_fp8(x)
    ref = O.fp8_scaled_mm(xq, wq.t(), xs, ws, torch.bfloat16)
    out = apply_fp8_linear(x.to(gpu), wq.to(gpu).t(), ws.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_fp8_static_activation_scale_linear(gpu):
    """apply_fp8_linear with a static per-tensor activation scale: static_quant_fp8 with the
    scale repeated per token (fp8_utils.py:684-689), then the per-channel GEMM."""
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print("fp8 linear, static activation scale", flush=True)
    x = O.gen_activation(48, 4096, seed=3002)
    wq, ws = O.per_tensor_quant_weight(O.gen_weight(4096, 4096, seed=3003))
    in_scale = torch.tensor([0.02], dtype=torch.float32)
    bias = (torch.randn(4096, generator=torch.Generator().manual_seed(2)) * 0.1).to(torch.bfloat16)
    xq, xs = O.static_quant_fp8(x, in_scale, repeat_scale=True)
    ref = O.fp8_scaled_mm(xq, wq.t(), xs, ws, torch.bfloat16, bias)
    out = apply_fp8_linear(x.to(gpu), wq.to(gpu).t(), ws.to(gpu), input_scale=in_scale.to(gpu), bias=bias.to(gpu))
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("mnk", [(1, 128, 128), (5, 2112, 1536), (40, 200, 1008), (127, 512, 7168), (300, 2048, 1024), (1024, 640, 2048),
                                 (4096, 1536, 512)])
def test_w8a8_block_fp8_matmul_row_major_scales(gpu, mnk):
    """w8a8_block_fp8_matmul (fp8_kernel.py:801-846,951-967): the weight and its scales as stored,
    row-major activation scales, N and K that are not multiples of 128; the same values as the
    sgl_kernel operator on transposed views, bit for bit, where that operator's K rule allows."""
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul, w8a8_block_fp8_matmul_triton
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    m, n, k = mnk
    print("w8a8_block_fp8_matmul", mnk, flush=True)
    g = torch.Generator().manual_seed(m + n + k)
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=n + k))
    xq = (torch.randn((m, k), generator=g) * 100).clamp(-448, 448).to(torch.float8_e4m3fn)
    xs = torch.rand((m, (k + 127) // 128), generator=g) * 1e-2 + 1e-3
    assert w8a8_block_fp8_matmul_triton is w8a8_block_fp8_matmul
    for dt in (torch.bfloat16, torch.float16):
        out = w8a8_block_fp8_matmul(xq.to(gpu), wq.to(gpu), xs.to(gpu), ws.to(gpu), [128, 128], dt)
        assert out.dtype == dt and tuple(out.shape) == (m, n)
        ref = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32, acc_dtype=torch.float64)
        torch.testing.assert_close(out.cpu().float(), ref, rtol=1e-2, atol=1e-2)
        if k % 128 == 0:
            xs_cm = xs.to(gpu).t().contiguous().t()
            same = fp8_blockwise_scaled_mm(xq.to(gpu), wq.to(gpu).t(), xs_cm, ws.to(gpu).t(), dt)
            assert torch.equal(out.view(torch.int16), same.view(torch.int16))
        bias = (torch.randn(n, generator=g) * 0.5).to(dt).to(gpu)
        fused = w8a8_block_fp8_matmul(xq.to(gpu), wq.to(gpu), xs.to(gpu), ws.to(gpu), [128, 128], dt, bias=bias)
        assert torch.equal(fused.view(torch.int16), (out + bias).view(torch.int16))
    # leading dimensions are kept
    out3 = w8a8_block_fp8_matmul(xq.to(gpu).view(1, m, k), wq.to(gpu), xs.to(gpu).view(1, m, -1), ws.to(gpu), [128, 128], torch.bfloat16)
    assert tuple(out3.shape) == (1, m, n)


def test_triton_path_block_fp8_linear(gpu):
    """triton_w8a8_block_fp8_linear (fp8_utils.py:289-309) against the oracle's same sequence, and
    against the column-major-scale path of the same layer bit for bit (same kernels, same sums)."""
    from sglang_amd.quantization.fp8_utils import triton_w8a8_block_fp8_linear, w8a8_block_fp8_linear

    print("triton-path block fp8 linear", flush=True)
    x = O.gen_activation(96, 2048, seed=3, outliers=True)
    wq, ws = O.block_quant_weight(O.gen_weight(1536, 2048, seed=4))
    bias = (torch.randn(1536, generator=torch.Generator().manual_seed(5)) * 0.1).to(torch.bfloat16)
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    mm = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32)
    ref = mm + bias.float()
    for b in (None, bias.to(gpu)):
        out = triton_w8a8_block_fp8_linear(x.to(gpu).view(2, 48, 2048), wq.to(gpu), [128, 128], ws.to(gpu), bias=b)
        assert tuple(out.shape) == (2, 48, 1536) and out.dtype == torch.bfloat16
        want = ref if b is not None else mm
        tol = 1e-2 + 1e-2 * want.abs() + mm.abs() * 2.0**-8
        err = (out.cpu().view(96, 1536).float() - want).abs()
        assert bool((err <= tol).all()), f"max excess {(err - tol).max().item()}"
        other = w8a8_block_fp8_linear(x.to(gpu).view(2, 48, 2048), wq.to(gpu), [128, 128], ws.to(gpu), bias=b)
        assert torch.equal(out.view(torch.int16), other.view(torch.int16))
    with pytest.raises(NotImplementedError):
        triton_w8a8_block_fp8_linear(x.to(gpu), wq.to(gpu), [64, 64], ws.to(gpu))


@pytest.mark.parametrize("m", [5, 130])
def test_deepgemm_path_block_fp8_linear(gpu, m):
    """deepgemm_w8a8_block_fp8_linear_with_fallback (fp8_utils.py:215-258): column-major activation
    scales with the row count padded to a multiple of four.  Same kernels and sums as the plain
    column-major path, so the results are equal bit for bit; fp16 inputs and an N that is not a
    multiple of 64 take the row-major path, which gives the same bits as well."""
    from sglang_amd.quantization import fp8_utils as F

    print("deepgemm-path block fp8 linear", m, flush=True)
    n, k = 1536, 2048
    x = O.gen_activation(m, k, seed=6, outliers=True)
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=7))
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(8)) * 0.1).to(torch.bfloat16)
    xq, xs = O.per_token_group_quant_fp8(x, 128)
    mm = O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.float32)
    for b in (None, bias.to(gpu)):
        out = F.deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu), wq.to(gpu), [128, 128], ws.to(gpu), bias=b)
        want = mm + bias.float() if b is not None else mm
        tol = 1e-2 + 1e-2 * want.abs() + mm.abs() * 2.0**-8
        err = (out.cpu().float() - want).abs()
        assert out.dtype == torch.bfloat16 and bool((err <= tol).all()), f"max excess {(err - tol).max().item()}"
        other = F.cutlass_w8a8_block_fp8_linear_with_fallback(x.to(gpu), wq.to(gpu), [128, 128], ws.to(gpu), bias=b)
        assert torch.equal(out.view(torch.int16), other.view(torch.int16))
    # fall-backs: fp16 activations; N = 1504 (a multiple of 4 and of 32, not of 64)
    half = F.deepgemm_w8a8_block_fp8_linear_with_fallback(x.half().to(gpu), wq.to(gpu), [128, 128], ws.to(gpu))
    assert half.dtype == torch.float16
    assert torch.equal(half, F.triton_w8a8_block_fp8_linear(x.half().to(gpu), wq.to(gpu), [128, 128], ws.to(gpu)))
    narrow = F.deepgemm_w8a8_block_fp8_linear_with_fallback(x.to(gpu), wq[:1504].contiguous().to(gpu), [128, 128], ws.to(gpu))
    assert torch.equal(narrow, out_rows(F, x.to(gpu), wq[:1504].contiguous().to(gpu), ws.to(gpu)))
    assert F.cutlass_fp8_supported() and F.cutlass_block_fp8_supported()
    assert F.dispatch_w8a8_block_fp8_linear() is F.cutlass_w8a8_block_fp8_linear_with_fallback


def out_rows(F, x, wq, ws):
    return F.triton_w8a8_block_fp8_linear(x, wq, [128, 128], ws)


def test_tensor_requant_of_block_weights_on_the_device(gpu):
    """block_quant_to_tensor_quant / channel_quant_to_tensor_quant on GPU tensors quantize with
    scaled_fp8_quant (the reference's CUDA branch, fp8_utils.py:392-396): scale = amax / 448 of
    the dequantized weight and codes that match the oracle's per-tensor quantization of it."""
    from sglang_amd.quantization import fp8_utils as F

    print("tensor requant", flush=True)
    wq, ws = O.block_quant_weight(O.gen_weight(300, 520, seed=9))
    deq = F.block_quant_dequant(wq, ws, [128, 128], torch.float32)
    q, s = F.block_quant_to_tensor_quant(wq.to(gpu), ws.to(gpu), [128, 128])
    ref_q, ref_s = O.per_tensor_quant_fp8(deq)
    assert torch.equal(s.cpu().view(-1), ref_s.view(-1))
    assert torch.equal(q.cpu().view(torch.uint8), ref_q.view(torch.uint8))
    ch = torch.rand(300, 1) * 0.01 + 0.001
    q2, s2 = F.channel_quant_to_tensor_quant(wq.to(gpu), ch.to(gpu))
    ref_q2, ref_s2 = O.per_tensor_quant_fp8(wq.float() * ch)
    assert torch.equal(s2.cpu().view(-1), ref_s2.view(-1))
    assert torch.equal(q2.cpu().view(torch.uint8), ref_q2.view(torch.uint8))


def test_fp8_linear_from_a_16_bit_checkpoint(gpu):
    """fp8.py:362-378 then apply_fp8_linear: per-channel weight quantization at load time, the
    transposed view, dynamic per-token activations.  Against the oracle's sequence on the same
    codes, and loosely against the unquantized product (FP8 keeps 3 mantissa bits)."""
    from sglang_amd.quantization.fp8 import process_weights_after_loading
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print("fp8 linear, 16-bit checkpoint", flush=True)
    m, n, k = 48, 1024, 2048
    x = O.gen_activation(m, k, seed=11)
    w = O.gen_weight(n, k, seed=12).to(torch.bfloat16)
    wt, ws, in_scale = process_weights_after_loading(w.to(gpu), is_checkpoint_fp8_serialized=False)
    assert wt.shape == (k, n) and wt.stride(0) == 1 and ws.shape == (n, 1) and in_scale is None
    out = apply_fp8_linear(x.to(gpu), wt, ws)
    xq, xs = O.per_token_quant_fp8(x)
    ref = O.fp8_scaled_mm(xq, wt.cpu(), xs, ws.cpu(), torch.float32, None)
    torch.testing.assert_close(out.cpu().float(), ref, rtol=1e-2, atol=1e-2)
    exact = x.float() @ w.float().t()
    assert ((out.cpu().float() - exact).norm() / exact.norm()).item() < 0.06


def test_requantize_fused_shards_with_max_scale(gpu):
    """utils.py:95-121 on the device: every shard ends up on the largest scale; a shard that
    already has it keeps its codes."""
    from sglang_amd.quantization.utils import requantize_with_max_scale

    print("requantize fused shards", flush=True)
    g = torch.Generator().manual_seed(13)
    codes = (torch.randn((96, 256), generator=g) * 40).clamp(-448, 448).to(torch.float8_e4m3fn)
    scales = torch.tensor([0.5, 2.0, 1.0])
    w = codes.clone().to(gpu)
    max_scale, w2 = requantize_with_max_scale(w, scales.to(gpu), [32, 32, 32])
    assert max_scale.item() == 2.0 and w2.data_ptr() == w.data_ptr()
    assert torch.equal(w2[32:64].cpu().view(torch.uint8), codes[32:64].view(torch.uint8))
    for i, s in ((0, 0.5), (2, 1.0)):
        want = (codes[32 * i:32 * i + 32].float() * s).half().float()
        q, _ = O.per_tensor_quant_fp8(want, torch.tensor([2.0]))
        assert torch.equal(w2[32 * i:32 * i + 32].cpu().view(torch.uint8), q.view(torch.uint8))
    # a fused checkpoint: the last scale was never loaded, the weight is left alone
    untouched = codes.clone().to(gpu)
    init = torch.tensor([1.5, torch.finfo(torch.float8_e4m3fn).min, torch.finfo(torch.float8_e4m3fn).min])
    m2, w3 = requantize_with_max_scale(untouched, init.to(gpu), [32, 32, 32])
    assert m2.item() == 1.5 and torch.equal(w3.cpu().view(torch.uint8), codes.view(torch.uint8))


def _fp8_linear_case(m, n, k, seed):
    x = O.gen_activation(m, k, seed=seed)
    wq, ws = O.per_tensor_quant_weight(O.gen_weight(n, k, seed=seed + 1))
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(seed + 2)) * 0.1).to(torch.bfloat16)
    return x, wq, ws, bias


def test_apply_fp8_linear_called_as_fp8_linear_method_calls_it(gpu):
    """The keyword list of Fp8LinearMethod.apply (fp8.py:480-488), dynamic activations."""
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print("fp8 linear, keyword list of fp8.py", flush=True)
    x, wq, ws, bias = _fp8_linear_case(33, 1024, 2048, 40)
    xq, xs = O.per_token_quant_fp8(x)
    ref = O.fp8_scaled_mm(xq, wq.t(), xs, ws, torch.bfloat16, bias)
    out = apply_fp8_linear(input=x.to(gpu), weight=wq.to(gpu).t(), weight_scale=ws.to(gpu), input_scale=None,
                           bias=bias.to(gpu), cutlass_fp8_supported=True, use_per_token_if_dynamic=False)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_linear_method_objects_on_a_layer(gpu):
    """W8A8Fp8LinearMethod, W8A8Int8LinearMethod and Fp8LinearMethod (block quantization) driven the
    way a linear layer drives them: process_weights_after_loading(layer), then apply(layer, x, bias)
    (linear.py:231,406,1295)."""
    import types

    from sglang_amd.quantization.fp8 import Fp8Config, Fp8LinearMethod
    from sglang_amd.quantization.w8a8_fp8 import W8A8Fp8Config, W8A8Fp8LinearMethod
    from sglang_amd.quantization.w8a8_int8 import W8A8Int8LinearMethod

    print("linear methods on a layer", flush=True)
    P = lambda t: torch.nn.Parameter(t.to(gpu), requires_grad=False)
    # W8A8 FP8 from a 16-bit checkpoint
    m, n, k = 24, 512, 1024
    x = O.gen_activation(m, k, seed=50)
    w = O.gen_weight(n, k, seed=51).to(torch.bfloat16)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(52)) * 0.1).to(torch.bfloat16)
    layer = types.SimpleNamespace(weight=P(w), weight_scale=None)
    method = W8A8Fp8LinearMethod(W8A8Fp8Config(is_checkpoint_fp8_serialized=False))
    method.process_weights_after_loading(layer)
    # load-time weight quantization runs in torch on the weight's device: torch's GPU divide is not
    # the IEEE quotient in the last place, so a few codes land on the neighbouring value (on the CPU
    # the same function equals the oracle bit for bit, tests/test_glue_signatures.py)
    wq_ref, ws_ref = O.per_token_group_quant_fp8(w, k)
    wq_dev = layer.weight.t().contiguous().cpu()
    assert (wq_dev.view(torch.uint8) != wq_ref.view(torch.uint8)).float().mean().item() < 1e-3
    torch.testing.assert_close(layer.weight_scale.cpu(), ws_ref, rtol=1e-6, atol=0)
    out = method.apply(layer, x.to(gpu).view(2, 12, k), bias.to(gpu))
    xq, xs = O.per_token_quant_fp8(x)
    ref = O.fp8_scaled_mm(xq, wq_dev.t(), xs, layer.weight_scale.cpu(), torch.bfloat16, bias)
    assert tuple(out.shape) == (2, 12, n)
    torch.testing.assert_close(out.cpu().view(m, n).float(), ref.float(), rtol=1e-2, atol=1e-2)
    # W8A8 INT8
    wt, s_b, bias8 = O.gen_int8_weight(1024, 768, seed=53)
    layer = types.SimpleNamespace(weight=P(wt.t().contiguous()), weight_scale=P(s_b.reshape(-1, 1)))
    method = W8A8Int8LinearMethod()
    method.process_weights_after_loading(layer)
    out = method.apply(layer, x.to(gpu), bias8.to(gpu))
    aq, as_ = O.per_token_quant_int8(x)
    ref = O.int8_scaled_mm(aq, wt, as_, s_b, torch.bfloat16, bias8)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    # block FP8
    wq, ws = O.block_quant_weight(O.gen_weight(n, k, seed=54))
    layer = types.SimpleNamespace(weight=P(wq), weight_scale_inv=P(ws))
    method = Fp8LinearMethod(Fp8Config(is_checkpoint_fp8_serialized=True, weight_block_size=[128, 128]))
    method.process_weights_after_loading(layer)
    out = method.apply(layer, x.to(gpu), None)
    gq, gs = O.per_token_group_quant_fp8(x, 128)
    ref = O.fp8_blockwise_scaled_mm(gq, wq.t(), gs, ws.t(), torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("per_token", [True, False])
@pytest.mark.parametrize("static", [False, True])
def test_apply_fp8_linear_compressed_tensor_branch(gpu, per_token, static):
    """compressed_tensor_quant=True (fp8_utils.py:567-596; caller
    compressed_tensors_w8a8_fp8.py:152-160): scaled_fp8_quant decides the activation scale's
    granularity; a per-tensor scale is repeated per token for the GEMM."""
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print(f"fp8 linear, compressed-tensors branch per_token={per_token} static={static}", flush=True)
    m = 20
    x, wq, ws, bias = _fp8_linear_case(m, 768, 1024, 60)
    in_scale = torch.tensor([0.015], dtype=torch.float32) if static else None
    if static:
        xq, xs = O.per_tensor_quant_fp8(x, in_scale)
        xs = xs.reshape(1, 1).expand(m, 1).contiguous()
    elif per_token:
        xq, xs = O.per_token_quant_fp8(x)
    else:
        xq, xs = O.per_tensor_quant_fp8(x)
        xs = xs.reshape(1, 1).expand(m, 1).contiguous()
    ref = O.fp8_scaled_mm(xq, wq.t(), xs, ws, torch.bfloat16, bias)
    out = apply_fp8_linear(input=x.to(gpu), weight=wq.to(gpu).t(), weight_scale=ws.to(gpu),
                           input_scale=in_scale.to(gpu) if static else None, bias=bias.to(gpu),
                           use_per_token_if_dynamic=per_token, compressed_tensor_quant=True)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_apply_fp8_linear_per_tensor_weight_scale(gpu):
    """A single weight scale (the reference's torch._scaled_mm case, fp8_utils.py:735-748) is
    repeated per channel."""
    from sglang_amd.quantization.fp8_utils import apply_fp8_linear

    print("fp8 linear, one weight scale", flush=True)
    x, wq, ws, bias = _fp8_linear_case(17, 512, 1024, 70)
    xq, xs = O.per_token_quant_fp8(x)
    ref = O.fp8_scaled_mm(xq, wq.t(), xs, ws, torch.bfloat16, bias)
    out = apply_fp8_linear(x.to(gpu), wq.to(gpu).t(), ws[:1].reshape(1).to(gpu), bias=bias.to(gpu), cutlass_fp8_supported=False)
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
