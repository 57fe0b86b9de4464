"""The group-quant kernel evaluates x / y as a reciprocal multiply plus an exact
FMA remainder correction.  tests/csrc/exact_div_check.c searches on the CPU for an
input where that differs from the IEEE quotient in a way that could reach an
8-bit code; there must be none."""
import ctypes
import subprocess
from pathlib import Path

import pytest

SRC = Path(__file__).resolve().parent / "csrc" / "exact_div_check.c"


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    so = tmp_path_factory.mktemp("exact_div") / "exact_div_check.so"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-mfma", "-shared", "-fPIC", "-o", str(so), str(SRC), "-lm"], check=True)
    lib = ctypes.CDLL(str(so))
    lib.check_16bit_numerators.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_int64]
    lib.check_16bit_numerators.restype = ctypes.c_int64
    lib.check_random_fp32.argtypes = [ctypes.c_float, ctypes.c_int64]
    lib.check_random_fp32.restype = ctypes.c_int64
    return lib


@pytest.mark.parametrize("max8", [448.0, 127.0, 224.0])
def test_division_shortcut_is_exact(lib, max8):
    assert lib.check_16bit_numerators(0, max8, 400) == 0  # bf16 numerators
    assert lib.check_16bit_numerators(1, max8, 400) == 0  # fp16 numerators
    assert lib.check_random_fp32(max8, 2_000_000) == 0
