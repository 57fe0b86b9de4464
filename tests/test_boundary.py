"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol the header declares, the torch ops are registered under the reference's
schemas, and argument validation raises what the reference's entry points raise."""
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
FP8 = torch.float8_e4m3fn


def declared_symbols():
    text = (ROOT / "include" / "sglq.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sglq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from sglang_amd import _lib

    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 13
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/sglq.h but not exported"
    assert lib.sglq_abi_version() == 1
    assert set(_lib.SIGNATURES) <= set(names)


def test_ops_registered_with_reference_schemas():
    import sglang_amd.sgl_kernel  # noqa: F401

    want = {
        "int8_scaled_mm": ["mat_a", "mat_b", "scales_a", "scales_b", "out_dtype", "bias"],
        "fp8_scaled_mm": ["mat_a", "mat_b", "scales_a", "scales_b", "out_dtype", "bias"],
        "fp8_blockwise_scaled_mm": ["mat_a", "mat_b", "scales_a", "scales_b", "out_dtype"],
        "sgl_per_token_group_quant_fp8": ["input", "output_q", "output_s", "group_size", "eps", "fp8_min", "fp8_max", "scale_ue8m0"],
        "sgl_per_token_group_quant_int8": ["input", "output_q", "output_s", "group_size", "eps", "int8_min", "int8_max"],
        "sgl_per_token_quant_fp8": ["input", "output_q", "output_s"],
    }
    for name, args in want.items():
        schema = getattr(torch.ops.sgl_kernel, name).default._schema
        assert [a.name for a in schema.arguments] == args


def test_cpu_tensors_are_refused_by_dispatch():
    from sglang_amd.sgl_kernel import int8_scaled_mm

    a = torch.zeros(4, 16, dtype=torch.int8)
    with pytest.raises(NotImplementedError):
        int8_scaled_mm(a, a.t(), torch.ones(4), torch.ones(4), torch.bfloat16)


def test_mm_argument_validation_messages():
    from sglang_amd.sgl_kernel import gemm as G

    a = torch.zeros(4, 32, dtype=torch.int8)
    w = torch.zeros(8, 32, dtype=torch.int8)
    ok = dict(out_dtype=torch.bfloat16, elem_dtype=torch.int8, elem_name="Int8", require_cuda=False)
    G.check_mm_common(a, w.t(), **ok)
    with pytest.raises(RuntimeError, match="mat_a must be a CUDA tensor"):
        G.check_mm_common(a, w.t(), torch.bfloat16, torch.int8, "Int8")
    with pytest.raises(RuntimeError, match="mat_b must be a column major tensor"):
        G.check_mm_common(a, torch.zeros(32, 8, dtype=torch.int8), **ok)
    with pytest.raises(RuntimeError, match="mat_a must be a row major tensor"):
        G.check_mm_common(torch.zeros(32, 4, dtype=torch.int8).t(), w.t(), **ok)
    with pytest.raises(RuntimeError, match="cannot be multiplied"):
        G.check_mm_common(a, torch.zeros(8, 48, dtype=torch.int8).t(), **ok)
    with pytest.raises(RuntimeError, match="multiple of 16 bytes"):
        G.check_mm_common(torch.zeros(4, 24, dtype=torch.int8), torch.zeros(8, 24, dtype=torch.int8).t(), **ok)
    with pytest.raises(RuntimeError, match="mat_a must be Int8"):
        G.check_mm_common(a.to(torch.uint8), w.t(), **ok)
    with pytest.raises(RuntimeError, match="out_dtype must be Half or BFloat16"):
        G.check_mm_common(a, w.t(), torch.float32, torch.int8, "Int8", require_cuda=False)
    with pytest.raises(RuntimeError, match="mat_a must be a 2D tensor"):
        G.check_mm_common(a[None], w.t(), **ok)

    sa, sb = torch.ones(4, 1), torch.ones(8, 1)
    G.check_rowcol_scales(a, w.t(), sa, sb, torch.bfloat16, None)
    with pytest.raises(RuntimeError, match="size of scales_a is not matched"):
        G.check_rowcol_scales(a, w.t(), torch.ones(3), sb, torch.bfloat16, None)
    with pytest.raises(RuntimeError, match="scales_b must be Float32"):
        G.check_rowcol_scales(a, w.t(), sa, sb.double(), torch.bfloat16, None)
    with pytest.raises(RuntimeError, match="bias dtype must match output dtype"):
        G.check_rowcol_scales(a, w.t(), sa, sb, torch.bfloat16, torch.zeros(8, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="size of bias is not matched"):
        G.check_rowcol_scales(a, w.t(), sa, sb, torch.bfloat16, torch.zeros(7, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="scales_a must be contiguous"):
        G.check_rowcol_scales(a, w.t(), torch.ones(4, 2)[:, 0], sb, torch.bfloat16, None)


def test_blockwise_scale_validation():
    from sglang_amd.sgl_kernel import gemm as G

    a = torch.zeros(6, 256, dtype=FP8)
    w = torch.zeros(384, 256, dtype=FP8)
    sfa = torch.zeros(2, 6).t()          # [M, K/128] M-major
    sfb = torch.zeros(3, 2).t()          # weight_scale_inv [N/128, K/128] transposed -> K-major
    G.check_blockwise_scales(a, w.t(), sfa, sfb)
    with pytest.raises(RuntimeError, match="scales_a must be M major"):
        G.check_blockwise_scales(a, w.t(), torch.zeros(6, 2), sfb)
    with pytest.raises(RuntimeError, match="scales_b must be K major"):
        G.check_blockwise_scales(a, w.t(), sfa, torch.zeros(2, 3))
    with pytest.raises(RuntimeError, match="size of scales_b is not matched"):
        G.check_blockwise_scales(a, w.t(), sfa, torch.zeros(2, 2).t())
    with pytest.raises(RuntimeError, match="size of scales_a is not matched"):
        G.check_blockwise_scales(a, w.t(), torch.zeros(3, 6).t(), sfb)
    # ceil-division: N = 136 takes two scale columns
    G.check_blockwise_scales(a, torch.zeros(136, 256, dtype=FP8).t(), sfa, torch.zeros(2, 2).t())


def test_quant_argument_validation():
    from sglang_amd.sgl_kernel import gemm as G

    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    q = torch.zeros(4, 256, dtype=FP8)
    G.check_group_quant(x, q, torch.zeros(4, 2), 128, FP8, require_cuda=False)
    G.check_group_quant(x, q, torch.zeros(2, 4).t(), 128, FP8, require_cuda=False)  # column-major scales
    with pytest.raises(RuntimeError, match="divisible by group_size"):
        G.check_group_quant(x, q, torch.zeros(4, 2), 96, FP8, require_cuda=False)
    with pytest.raises(RuntimeError, match="output_s must be a 2D tensor"):
        G.check_group_quant(x, q, torch.zeros(8), 128, FP8, require_cuda=False)
    with pytest.raises(RuntimeError, match="input must be contiguous"):
        G.check_group_quant(torch.zeros(256, 4, dtype=torch.bfloat16).t(), q, torch.zeros(4, 2), 128, FP8, require_cuda=False)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        G.check_group_quant(x, q, torch.zeros(4, 2), 128, FP8)
    with pytest.raises(RuntimeError, match="Hidden dimension must be divisible by 8, but got 12"):
        G.check_token_quant_fp8(torch.zeros(2, 12), torch.zeros(2, 12, dtype=FP8), torch.zeros(2, 1), require_cuda=False)


def test_scale_buffer_layouts_match_reference_allocator():
    from sglang_amd.quantization.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk

    s = mk((6, 512), "cpu", 128, False, False, False)
    assert tuple(s.shape) == (6, 4) and s.is_contiguous()
    s = mk((6, 512), "cpu", 128, True, False, False)
    assert tuple(s.shape) == (6, 4) and s.stride() == (1, 6)
    s = mk((6, 512), "cpu", 128, True, True, False)
    assert tuple(s.shape) == (6, 4) and s.stride() == (1, 8)
    # scale_ue8m0: int32 words of four exponent bytes, zero-filled, column stride ceil4(M) (fp8_kernel.py:308-320)
    s = mk((6, 1536), "cpu", 128, True, True, True)
    assert s.dtype == torch.int32 and tuple(s.shape) == (6, 3) and s.stride() == (1, 8) and int(s.abs().max()) == 0


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    """Entry points validate before they touch the device."""
    from sglang_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(4096, dtype=torch.uint8)
    p = buf.data_ptr()
    rc = lib.sglq_per_token_group_quant_fp8(p, 0, p, p, 4, 100, 128, 1, 1, 1e-10, -448.0, 448.0, None)
    assert rc == 1 and b"multiple of group_size" in lib.sglq_last_error()
    rc = lib.sglq_per_token_group_quant_fp8(p, 0, p, p, 4, 96, 48, 2, 1, 1e-10, -448.0, 448.0, None)
    assert rc == 2  # group size not built
    rc = lib.sglq_per_token_quant_fp8(p, 0, p, p, 4, 12, None)
    assert rc == 1 and b"divisible by 8" in lib.sglq_last_error()
    rc = lib.sglq_int8_scaled_mm(p, 24, p, 24, p, p, None, p, 8, 0, 4, 8, 24, None, 0, None)
    assert rc == 1 and b"multiple of 16" in lib.sglq_last_error()
    rc = lib.sglq_fp8_blockwise_scaled_mm(p, 128, p, 128, p, 1, 4, p, 1, 1, p, 8, 2, 4, 8, 128, None, 0, None)
    assert rc == 1 and b"out_dtype" in lib.sglq_last_error()
    rc = lib.sglq_per_tensor_quant_fp8(p, 7, p, p, 16, 0, None)
    assert rc == 2 and b"dtype" in lib.sglq_last_error()
    rc = lib.sglq_per_tensor_quant_fp8(p, 0, p, None, 16, 0, None)
    assert rc == 1 and b"scale" in lib.sglq_last_error()
    assert lib.sglq_per_tensor_quant_fp8(None, 0, None, p, 0, 1, None) == 0
    # the widened operator set
    rc = lib.sglq_static_quant_fp8(p, 0, p, None, None, 4, 16, None)
    assert rc == 1 and b"scale" in lib.sglq_last_error()
    rc = lib.sglq_static_quant_fp8(p, 9, p, p, None, 4, 16, None)
    assert rc == 2 and b"dtype" in lib.sglq_last_error()
    assert lib.sglq_static_quant_fp8(None, 0, None, p, None, 0, 16, None) == 0
    rc = lib.sglq_per_token_group_quant_fp8_ue8m0(p, 0, p, p, 4, 200, 4, 1e-10, -448.0, 448.0, None)
    assert rc == 1 and b"multiple of 128" in lib.sglq_last_error()
    rc = lib.sglq_per_token_group_quant_fp8_ue8m0(p, 0, p, p, 8, 256, 4, 1e-10, -448.0, 448.0, None)
    assert rc == 1 and b"column stride" in lib.sglq_last_error()
    # packed UE8M0 activation scales: the workspace must hold the expanded scales; K a multiple of 128
    packed = lambda k, ws_bytes: lib.sglq_fp8_blockwise_scaled_mm_ue8m0_packed(p, k, p, k, p, 1, 4, p, 1, 4, p, 16, 0, 4, 16, k, p, ws_bytes, None)
    assert packed(256, 16) == 1 and b"workspace" in lib.sglq_last_error()
    assert packed(192, 4096) == 1 and b"multiple of 128" in lib.sglq_last_error()
    # grouped GEMM: a [32, 128], 2 experts of [16, 128]; workspace too small, then K not a multiple of 128, then no output type
    grouped = lambda k, ws_bytes, dt: lib.sglq_fp8_blockwise_scaled_grouped_mm(
        p, k, p, k, 16 * k, p, 1, 1, p, 1, 1, 1, p, 16, dt, p, p, 2, 32, 16, k, p, ws_bytes, None)
    assert grouped(128, 8, 0) == 1 and b"workspace" in lib.sglq_last_error()
    assert grouped(64, 4096, 0) == 1 and b"multiple of 128" in lib.sglq_last_error()
    assert grouped(128, 4096, 2) == 1 and b"bfloat16 or half" in lib.sglq_last_error()
    assert lib.sglq_fp8_blockwise_scaled_grouped_mm(p, 128, p, 128, 2048, p, 1, 1, p, 1, 1, 1, p, 16, 0, p, p, 0, 32, 16, 128, p, 4096,
                                                    None) == 0  # no experts
    # the operators around the grouped GEMM
    assert lib.sglq_prepare_moe_input(p, p, None, p, p, p, p, 8, 0, 4, 128, 128, None) == 1 and b"bad sizes" in lib.sglq_last_error()
    assert lib.sglq_prepare_moe_input(p, None, None, p, p, p, p, 8, 2, 4, 128, 128, None) == 1 and b"null" in lib.sglq_last_error()
    assert lib.sglq_prepare_moe_input(p, p, None, p, p, p, p, 8, 2, 0, 128, 128, None) == 0  # no experts
    assert lib.sglq_shuffle_rows(p, p, p, 4, -1, 16, None) == 1 and b"negative" in lib.sglq_last_error()
    assert lib.sglq_shuffle_rows(p, None, p, 4, 4, 16, None) == 1 and b"null" in lib.sglq_last_error()
    assert lib.sglq_shuffle_rows(p, p, p, 4, 0, 16, None) == 0
    assert lib.sglq_silu_and_mul(p, 2, p, 4, 8, None) == 2 and b"Half or BFloat16" in lib.sglq_last_error()
    assert lib.sglq_silu_and_mul(None, 0, p, 4, 8, None) == 1 and b"null" in lib.sglq_last_error()
    assert lib.sglq_silu_and_mul(p, 0, p, 0, 8, None) == 0
    assert lib.sglq_silu_and_mul_group_quant_fp8(p, 0, p, p, 4, 192, 1e-10, None) == 1 and b"multiple of 128" in lib.sglq_last_error()
    assert lib.sglq_silu_and_mul_group_quant_fp8(p, 2, p, p, 4, 128, 1e-10, None) == 2 and b"Half or BFloat16" in lib.sglq_last_error()
    assert lib.sglq_silu_and_mul_group_quant_fp8(p, 0, p, None, 4, 128, 1e-10, None) == 1 and b"null" in lib.sglq_last_error()
    assert lib.sglq_silu_and_mul_group_quant_fp8(p, 0, p, p, 0, 128, 1e-10, None) == 0
    assert lib.sglq_per_token_group_quant_fp8_scatter(p, 0, p, p, p, 4, 200, 2, 8, 1e-10, None) == 1 and b"multiple of 128" in lib.sglq_last_error()
    assert lib.sglq_per_token_group_quant_fp8_scatter(p, 0, p, p, None, 4, 128, 2, 8, 1e-10, None) == 1 and b"null" in lib.sglq_last_error()
    assert lib.sglq_per_token_group_quant_fp8_scatter(p, 5, p, p, p, 4, 128, 2, 8, 1e-10, None) == 2 and b"in_dtype" in lib.sglq_last_error()
    assert lib.sglq_per_token_group_quant_fp8_scatter(p, 0, p, p, p, 0, 128, 2, 0, 1e-10, None) == 0
    assert lib.sglq_apply_shuffle_mul_sum(p, p, p, None, 0, 4, 0, 8, 8, None) == 1 and b"bad sizes" in lib.sglq_last_error()
    assert lib.sglq_apply_shuffle_mul_sum(p, p, p, None, 0, 4, 2, 12, 8, None) == 1 and b"multiples of 8" in lib.sglq_last_error()
    assert lib.sglq_apply_shuffle_mul_sum(p, p, p, None, 2, 4, 2, 8, 8, None) == 2 and b"Half or BFloat16" in lib.sglq_last_error()
    assert lib.sglq_apply_shuffle_mul_sum(p, p, p, None, 0, 0, 2, 8, 8, None) == 0
    # output rows are written in 16-byte pieces: N and ldo multiples of 8 (4 for int32), base 16-byte aligned
    assert lib.sglq_int8_scaled_mm(p, 32, p, 32, p, p, None, p, 12, 0, 4, 12, 32, None, 0, None) == 1 and b"multiples of 8" in lib.sglq_last_error()
    assert lib.sglq_fp8_scaled_mm(p, 32, p, 32, p, p, None, p, 20, 0, 4, 16, 32, None, 0, None) == 1 and b"multiples of 8" in lib.sglq_last_error()
    assert lib.sglq_fp8_blockwise_scaled_mm(p, 128, p, 128, p, 1, 4, p, 1, 1, p + 8, 8, 0, 4, 8, 128, None, 0, None) == 1 and b"16-byte aligned" in lib.sglq_last_error()
    assert lib.sglq_int8_mm_i32(p, 32, p, 32, p, 6, 4, 6, 32, None, 0, None) == 1 and b"multiples of 4" in lib.sglq_last_error()
    # empty problems are a no-op
    assert lib.sglq_int8_scaled_mm(p, 32, p, 32, p, p, None, p, 8, 0, 0, 8, 32, None, 0, None) == 0


def test_tuned_config_tables(tmp_path):
    """Per-(N, K) kernel selections (the counterpart of fp8_kernel.py:738-776): file naming, the
    closest-M rule turned into ranges, and what the library's table accepts."""
    from sglang_amd import _lib
    from sglang_amd.quantization import tuned_configs as T

    name = T.config_file_name(4096, 7168)
    assert name == "N=4096,K=7168,device_name=AMD_Instinct_MI355X,dtype=fp8_w8a8,block_shape=[128, 128].json"
    assert T.parse_file_name(name) == (4096, 7168, "AMD_Instinct_MI355X", "fp8_w8a8")
    assert T.parse_file_name("README.md") is None
    table = {1: {"tile": 16, "splits": 0}, 64: {"tile": 64, "splits": 4}, 512: {"tile": 0, "splits": 0}, 4096: {"tile": 258, "splits": 1}}
    assert T.ranges_of(table) == [(0, 32, 16, 0), (33, 288, 64, 4), (289, 2304, 0, 0), (2305, T.M_MAX, 258, 1)]
    # every M goes to its closest key, ties to the smaller one
    for m in (1, 32, 33, 288, 289, 2304, 2305, 100000):
        closest = min(sorted(table), key=lambda key: abs(key - m))
        lo_hi = [r for r in T.ranges_of(table) if r[0] <= m <= r[1]]
        assert len(lo_hi) == 1 and lo_hi[0][2] == table[closest]["tile"], m
    path = T.save_config(4096, 7168, table, tmp_path)
    assert path.name == name and T.get_w8a8_block_fp8_configs(4096, 7168, 128, 128, tmp_path) == table
    assert T.get_w8a8_block_fp8_configs(4096, 7168, 64, 64, tmp_path) is None
    assert T.get_w8a8_block_fp8_configs(1, 2, 128, 128, tmp_path) is None
    T.save_config(2048, 512, {8: {"tile": 128, "splits": 2}}, tmp_path, dtype="int8_w8a8")
    (tmp_path / "N=8,K=8,device_name=other,dtype=fp8_w8a8,block_shape=[128, 128].json").write_text('{"1": {"tile": 64, "splits": 0}}')
    try:
        assert T.load_tuned_configs(tmp_path) == 4  # three selections of the first table, one of the second; the other device's file is skipped
        lib = _lib.load()
        assert lib.sglq_tuned_add(0, 4096, 7168, 0, 10, 77, 0) == 1 and b"known kernel code" in lib.sglq_last_error()
        assert lib.sglq_tuned_add(9, 4096, 7168, 0, 10, 64, 0) == 1
        assert lib.sglq_tuned_add(0, 4096, 7168, 11, 10, 64, 0) == 1
        assert lib.sglq_tuned_clear() == 0
        for i in range(1024):
            assert lib.sglq_tuned_add(0, 128 * (i + 1), 128, 0, 10, 64, 0) == 0
        assert lib.sglq_tuned_add(0, 128, 128, 0, 10, 64, 0) == 2 and b"1024 entries" in lib.sglq_last_error()
    finally:
        T.load_tuned_configs()  # back to the tables shipped with the package


def test_shipped_tuned_tables_load_into_the_library():
    """Every table shipped under quantization/configs is accepted by the library as it stands (known kernel
    codes, split factors in range, no more entries than the table holds)."""
    from sglang_amd.quantization import tuned_configs as T

    files = [p for p in T.CONFIG_DIR.iterdir() if T.parse_file_name(p.name) is not None]
    assert len(files) >= 60
    assert 0 < T.load_tuned_configs() <= 1024
