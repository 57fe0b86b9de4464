"""The glue functions must bind the argument lists that the reference's callers pass, by
position and by keyword, so that they can stand in for the reference's imports.  Each case
quotes the call site it mirrors; nothing here needs a GPU."""
import inspect
import types

import pytest
import torch

from oracle import w8a8_oracle as O
from sglang_amd.quantization import fp8 as fp8_mod
from sglang_amd.quantization import fp8_kernel, fp8_utils, int8_kernel, int8_utils, w8a8_fp8, w8a8_int8

T = object()  # stands for a tensor


def binds(fn, *args, **kwargs):
    return inspect.signature(fn).bind(*args, **kwargs).arguments


def test_apply_fp8_linear_parameter_list_is_the_references():
    # python/sglang/srt/layers/quantization/fp8_utils.py:539-550
    names = list(inspect.signature(fp8_utils.apply_fp8_linear).parameters)
    assert names == [
        "input", "weight", "weight_scale", "input_scale", "input_scale_ub", "bias", "cutlass_fp8_supported",
        "use_per_token_if_dynamic", "pad_output", "compressed_tensor_quant",
    ]
    sig = inspect.signature(fp8_utils.apply_fp8_linear)
    assert sig.parameters["use_per_token_if_dynamic"].default is False
    assert sig.parameters["compressed_tensor_quant"].default is False
    assert sig.parameters["pad_output"].default is None


def test_apply_fp8_linear_binds_fp8_linear_method_call():
    # fp8.py:480-488
    a = binds(fp8_utils.apply_fp8_linear, input=T, weight=T, weight_scale=T, input_scale=T, bias=T,
              cutlass_fp8_supported=True, use_per_token_if_dynamic=False)
    assert a["bias"] is T and a["input_scale"] is T


def test_apply_fp8_linear_binds_w8a8_fp8_linear_method_call():
    # w8a8_fp8.py:183-189
    x, w, s, b = object(), object(), object(), object()
    a = binds(fp8_utils.apply_fp8_linear, x, w, s, bias=b, cutlass_fp8_supported=True)
    assert a["input"] is x and a["weight"] is w and a["weight_scale"] is s and a["bias"] is b


def test_apply_fp8_linear_fifth_positional_is_input_scale_ub():
    # a positional call must not put a tensor meant as input_scale_ub into `bias`
    a = binds(fp8_utils.apply_fp8_linear, T, T, T, None, "ub")
    assert a["input_scale_ub"] == "ub" and "bias" not in a


def test_apply_fp8_linear_binds_compressed_tensors_call():
    # compressed_tensors/schemes/compressed_tensors_w8a8_fp8.py:152-160
    binds(fp8_utils.apply_fp8_linear, input=T, weight=T, weight_scale=T, input_scale=T, bias=T,
          use_per_token_if_dynamic=True, compressed_tensor_quant=True)


@pytest.mark.parametrize("fn_name", ["w8a8_block_fp8_linear", "cutlass_w8a8_block_fp8_linear_with_fallback",
                                     "deepgemm_w8a8_block_fp8_linear_with_fallback", "triton_w8a8_block_fp8_linear"])
def test_block_fp8_linear_binds_the_method_call(fn_name):
    # fp8.py:470-478
    fn = getattr(fp8_utils, fn_name)
    binds(fn, input=T, weight=T, block_size=[128, 128], weight_scale=T, input_scale=None, bias=T)
    assert fp8_utils.dispatch_w8a8_block_fp8_linear() is fp8_utils.cutlass_w8a8_block_fp8_linear_with_fallback


def test_quant_wrappers_bind_the_linear_functions_calls():
    # fp8_utils.py:204-206
    binds(fp8_kernel.per_token_group_quant_fp8, T, 128, column_major_scales=True)
    # fp8_utils.py:240-246
    binds(fp8_kernel.sglang_per_token_group_quant_fp8, T, 128, column_major_scales=True, scale_tma_aligned=True,
          scale_ue8m0=False)
    # fp8_utils.py:693
    binds(fp8_kernel.sglang_per_token_quant_fp8, T)
    # fp8_utils.py:686-688
    binds(fp8_kernel.static_quant_fp8, T, T, repeat_scale=True)
    # fp8_utils.py:570-574,601-606
    binds(fp8_kernel.scaled_fp8_quant, T, T, use_per_token_if_dynamic=True)
    binds(fp8_kernel.scaled_fp8_quant, T, T, num_token_padding=17, use_per_token_if_dynamic=False)
    # w8a8_int8.py:387
    binds(int8_kernel.per_token_quant_int8, T)
    assert list(inspect.signature(int8_kernel.per_token_quant_int8).parameters) == ["x", "scale_dtype", "cal_sum"]
    # int8_utils.py:11-33
    binds(int8_utils.apply_w8a8_block_int8_linear, input=T, weight=T, block_size=[128, 128], weight_scale=T,
          input_scale=None, bias=T)


def test_ue8m0_path_binds_the_reference_calls():
    # fp8_utils.py:248-250: the GEMM call of deepgemm_w8a8_block_fp8_linear_with_fallback
    a = binds(fp8_kernel.w8a8_block_fp8_matmul_deepgemm, T, T, T, T, [128, 128], output_dtype=torch.bfloat16)
    assert list(a) == ["A", "B", "As", "Bs", "block_size", "output_dtype"]
    # fp8_utils.py:424-429 (called by the loaders as requant_weight_ue8m0_inplace(weight, weight_scale_inv, weight_block_size))
    assert list(inspect.signature(fp8_utils.requant_weight_ue8m0_inplace).parameters) == ["weight", "weight_scale_inv", "weight_block_size"]
    # the flag the reference keeps in deep_gemm_wrapper (fp8_utils.py:245); off unless asked for
    assert fp8_utils.DEEPGEMM_SCALE_UE8M0 in (False, True)


def test_gemm_wrappers_bind_the_linear_functions_calls():
    import sgl_kernel
    import sgl_kernel.gemm as G

    # fp8_utils.py:207-209
    binds(sgl_kernel.fp8_blockwise_scaled_mm, T, T, T, T, out_dtype=torch.bfloat16)
    # fp8_utils.py:725-732
    binds(sgl_kernel.fp8_scaled_mm, T, T, T, T, out_dtype=torch.bfloat16, bias=T)
    # w8a8_int8.py:389-391
    binds(sgl_kernel.int8_scaled_mm, T, T, T, T, out_dtype=torch.bfloat16, bias=T)
    # sgl-kernel/python/sgl_kernel/gemm.py:13-42,100-145: positional forms
    for name, nargs in [("int8_scaled_mm", 6), ("fp8_scaled_mm", 6), ("fp8_blockwise_scaled_mm", 5),
                        ("sgl_per_token_group_quant_fp8", 8), ("sgl_per_token_group_quant_int8", 7),
                        ("sgl_per_token_quant_fp8", 3), ("sgl_per_tensor_quant_fp8", 4)]:
        binds(getattr(G, name), *([T] * nargs))
        assert getattr(sgl_kernel, name) is getattr(G, name)
        assert hasattr(torch.ops.sgl_kernel, name)


def test_linear_methods_bind_the_layers_call():
    # python/sglang/srt/layers/linear.py:231,406,1295: quant_method.apply(self, x, bias)
    for cls in (w8a8_fp8.W8A8Fp8LinearMethod, w8a8_int8.W8A8Int8LinearMethod, fp8_mod.Fp8LinearMethod):
        binds(cls.apply, "self", "layer", T, T)
        binds(cls.process_weights_after_loading, "self", "layer")


def test_w8a8_fp8_method_quantizes_a_16_bit_checkpoint_per_channel():
    # w8a8_fp8.py:114-127: every output channel of the weight is one group
    w = O.gen_weight(48, 256, seed=3).to(torch.bfloat16)
    layer = types.SimpleNamespace(weight=torch.nn.Parameter(w.clone(), requires_grad=False), weight_scale=None)
    method = w8a8_fp8.W8A8Fp8LinearMethod(w8a8_fp8.W8A8Fp8Config(is_checkpoint_fp8_serialized=False))
    method.process_weights_after_loading(layer)
    q_ref, s_ref = O.per_token_group_quant_fp8(w, 256)
    assert layer.weight.shape == (256, 48) and layer.weight.stride(0) == 1
    assert torch.equal(layer.weight.t().contiguous().view(torch.uint8), q_ref.view(torch.uint8))
    assert layer.weight_scale.shape == (48, 1) and torch.equal(layer.weight_scale.data, s_ref)
    assert layer.input_scale is None


def test_w8a8_fp8_method_keeps_an_fp8_checkpoint():
    # w8a8_fp8.py:104-111
    q = torch.randn(32, 128).to(torch.float8_e4m3fn)
    s = torch.rand(32, 1) + 0.5
    layer = types.SimpleNamespace(weight=torch.nn.Parameter(q, requires_grad=False),
                                  weight_scale=torch.nn.Parameter(s.clone(), requires_grad=False))
    cfg = w8a8_fp8.W8A8Fp8Config.from_config({"quant_method": "w8a8_fp8"})
    assert cfg.is_checkpoint_fp8_serialized
    w8a8_fp8.W8A8Fp8LinearMethod(cfg).process_weights_after_loading(layer)
    assert layer.weight.shape == (128, 32) and layer.weight.data_ptr() == q.data_ptr()
    assert torch.equal(layer.weight_scale.data, s)


def test_w8a8_int8_method_takes_the_transposed_view():
    # w8a8_int8.py:337-338
    w = torch.randint(-127, 128, (24, 64), dtype=torch.int8)
    s = torch.rand(24, 1)
    layer = types.SimpleNamespace(weight=torch.nn.Parameter(w, requires_grad=False),
                                  weight_scale=torch.nn.Parameter(s, requires_grad=False))
    w8a8_int8.W8A8Int8LinearMethod().process_weights_after_loading(layer)
    assert layer.weight.shape == (64, 24) and layer.weight.stride(0) == 1 and layer.weight.data_ptr() == w.data_ptr()
    assert torch.equal(layer.weight_scale.data, s)


def test_fp8_method_spreads_shard_scales_and_takes_the_largest_input_scale():
    # fp8.py:382-433 with per-channel GEMM scales
    q = torch.randn(48, 128).to(torch.float8_e4m3fn)
    layer = types.SimpleNamespace(
        weight=torch.nn.Parameter(q, requires_grad=False),
        weight_scale=torch.nn.Parameter(torch.tensor([0.5, 0.25, 2.0]), requires_grad=False),
        input_scale=torch.nn.Parameter(torch.tensor([0.1, 0.3, 0.2]), requires_grad=False),
        logical_widths=[16, 16, 16],
    )
    m = fp8_mod.Fp8LinearMethod(fp8_mod.Fp8Config(is_checkpoint_fp8_serialized=True, activation_scheme="static"))
    m.process_weights_after_loading(layer)
    assert layer.weight.shape == (128, 48)
    assert layer.weight_scale.shape == (48, 1)
    assert torch.equal(layer.weight_scale.data.flatten(), torch.tensor([0.5] * 16 + [0.25] * 16 + [2.0] * 16))
    assert float(layer.input_scale) == pytest.approx(0.3)


def test_fp8_config_rejects_what_the_reference_rejects():
    # fp8.py:115-135
    with pytest.raises(ValueError):
        fp8_mod.Fp8Config(activation_scheme="sometimes")
    with pytest.raises(ValueError):
        fp8_mod.Fp8Config(is_checkpoint_fp8_serialized=False, weight_block_size=[128, 128])
    with pytest.raises(ValueError):
        fp8_mod.Fp8Config(is_checkpoint_fp8_serialized=True, activation_scheme="static", weight_block_size=[128, 128])
