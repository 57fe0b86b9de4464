"""ctypes binding of libsglq.so (the C ABI declared in include/sglq.h).

There is no fallback: if the shared object is missing or a symbol cannot be
resolved, importing the operators raises."""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch

# SGLQ_LIBRARY points at another build of the same C ABI (kernel development)
LIB_PATH = Path(os.environ.get("SGLQ_LIBRARY") or Path(__file__).resolve().parent / "libsglq.so")

SGLQ_BF16, SGLQ_FP16, SGLQ_FP32, SGLQ_I32 = 0, 1, 2, 3
DTYPE_CODE = {torch.bfloat16: SGLQ_BF16, torch.float16: SGLQ_FP16, torch.float32: SGLQ_FP32}

# name -> argtypes; every function returns int.  Mirrors include/sglq.h.
_GROUP_QUANT = [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int64, c_int64, c_float, c_float, c_float, c_void_p]
_ROWCOL_MM = [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64,
              c_void_p, c_int64, c_void_p]
SIGNATURES = {
    "sglq_per_token_group_quant_fp8": _GROUP_QUANT,
    "sglq_per_token_group_quant_int8": _GROUP_QUANT,
    "sglq_per_token_quant_fp8": [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    "sglq_per_token_quant_int8": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    "sglq_per_token_group_quant_fp8_ue8m0": [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_float, c_float, c_void_p],
    "sglq_per_token_group_quant_fp8_pow2": [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_float, c_float, c_void_p],
    "sglq_per_tensor_quant_fp8": [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_void_p],
    "sglq_static_quant_fp8": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_mm": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                     c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_mm_ue8m0": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                           c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_mm_ue8m0_packed": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64,
                                                  c_int64, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_mm_noalloc": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                             c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p],
    "sglq_init": [],
    "sglq_w8a8_block_fp8_linear": [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int,
                                   c_int64, c_int64, c_int64, c_float, c_void_p, c_int64, c_void_p],
    "sglq_w8a8_int8_linear": [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64,
                              c_void_p, c_int64, c_void_p],
    "sglq_w8a8_fp8_linear": [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64,
                             c_void_p, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_mm_bias": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                          c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_fp8_blockwise_scaled_grouped_mm": [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p,
                                             c_int64, c_int64, c_int64, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int64,
                                             c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_prepare_moe_input": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                               c_int64, c_void_p],
    "sglq_shuffle_rows": [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p],
    "sglq_silu_and_mul": [c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p],
    "sglq_tuned_add": [c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_int],
    "sglq_tuned_clear": [],
    "sglq_per_token_group_quant_fp8_scatter": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_void_p],
    "sglq_silu_and_mul_group_quant_fp8": [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_float, c_void_p],
    "sglq_apply_shuffle_mul_sum": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p],
    "sglq_int8_blockwise_scaled_mm": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                      c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_int8_blockwise_scaled_mm_bias": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                           c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
    "sglq_int8_scaled_mm": _ROWCOL_MM,
    "sglq_fp8_scaled_mm": _ROWCOL_MM,
    "sglq_int8_mm_i32": [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p],
}

_lib = None


def load() -> ctypes.CDLL:
    """Load libsglq.so once; raise if it is absent (it is built by ``sglang_amd.build``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP kernels first (python -m sglang_amd.build). "
            "There is no non-HIP fallback for these operators."
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = c_int
    lib.sglq_last_error.restype = c_char_p
    lib.sglq_last_error.argtypes = []
    lib.sglq_abi_version.restype = c_int
    lib.sglq_abi_version.argtypes = []
    lib.sglq_debug_set_direct_lds.argtypes = [c_int]
    lib.sglq_debug_set_direct_lds.restype = None
    lib.sglq_debug_force_tile.argtypes = [c_int]
    lib.sglq_debug_force_tile.restype = None
    lib.sglq_debug_force_splits.argtypes = [c_int]
    lib.sglq_debug_force_splits.restype = None
    lib.sglq_debug_grouped_tile.argtypes = [c_int]
    lib.sglq_debug_grouped_tile.restype = None
    lib.sglq_debug_last_gemm_kernel.argtypes = []
    lib.sglq_debug_last_gemm_kernel.restype = ctypes.c_char_p
    lib.sglq_debug_last_gemm_hw_scaled.argtypes = []
    lib.sglq_debug_last_gemm_hw_scaled.restype = ctypes.c_int
    _lib = lib
    if os.environ.get("SGLQ_NO_TUNED_CONFIGS", "0") != "1":
        # per-(N, K) kernel selections shipped beside the package (sglang_amd/quantization/configs/)
        from .quantization.tuned_configs import load_tuned_configs

        load_tuned_configs()
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().sglq_last_error().decode("utf-8", "replace")
        if rc == 2:
            raise NotImplementedError(msg or what)
        raise RuntimeError(msg or f"{what} failed with code {rc}")


_workspaces = {}
WORKSPACE_BYTES = 64 << 20


def workspace(device: torch.device):
    """Scratch for the split-K partial sums of the GEMM kernels, one buffer per device and
    stream (two streams may run GEMMs at the same time and must not share partial sums),
    allocated on first use (the reference caches its GEMM workspaces the same way,
    sgl-kernel/python/sgl_kernel/utils.py `_get_cache_buf`).  Returns (pointer, bytes) for
    the device's current stream."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (device.type, index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None:
        buf = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf.data_ptr(), buf.numel()


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
