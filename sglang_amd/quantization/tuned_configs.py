"""Tuned kernel selections per (N, K), kept as JSON files beside the package like the
reference's tables for its Triton block-FP8 GEMM (get_w8a8_block_fp8_configs,
python/sglang/srt/layers/quantization/fp8_kernel.py:738-776; files under
python/sglang/srt/layers/quantization/configs/).

File name: ``N={N},K={K},device_name={device},dtype={dtype},block_shape=[128, 128].json`` with
dtype ``fp8_w8a8`` (block-scaled FP8), ``int8_w8a8`` (block-scaled INT8), or ``fp8_w8a8_channel`` /
``int8_w8a8_channel`` (fp8_scaled_mm / int8_scaled_mm with per-token and per-channel scales, whose kernel the
reference picks per M bucket in C++: sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:751-791, int8_gemm_kernel.cu:585-661).  Content: a mapping
from batch sizes M to ``{"tile": code, "splits": s}``, where ``code`` names a kernel as
``sglq_debug_force_tile`` does and ``s`` is the split-K factor (0 = leave it to the library).
As in the reference, a call takes the entry whose M is closest to its own; here that rule is
turned into M ranges (midpoints between neighbouring keys) once, when the table is handed to
the library.  Without a file the library's built-in selection applies."""

from __future__ import annotations

import json
import os
from pathlib import Path
from typing import Any, Dict, Iterable, List, Optional, Tuple

from .. import _lib

CONFIG_DIR = Path(__file__).resolve().parent / "configs"
DEVICE_NAME = "AMD_Instinct_MI355X"
# SGLQ_KIND_FP8_BLOCK, SGLQ_KIND_I8_BLOCK; per-token / per-channel scales: SGLQ_KIND_FP8_ROWCOL, SGLQ_KIND_I8_ROWCOL
KIND_OF_DTYPE = {"fp8_w8a8": 0, "int8_w8a8": 4, "fp8_w8a8_channel": 1, "int8_w8a8_channel": 2}
M_MAX = 1 << 30


def config_file_name(N: int, K: int, dtype: str = "fp8_w8a8", device_name: str = DEVICE_NAME) -> str:
    return f"N={N},K={K},device_name={device_name},dtype={dtype},block_shape=[128, 128].json"


def get_w8a8_block_fp8_configs(N: int, K: int, block_n: int = 128, block_k: int = 128, config_dir: Optional[os.PathLike] = None,
                               dtype: str = "fp8_w8a8") -> Optional[Dict[int, Any]]:
    """The table for (N, K) as {M: {"tile": ..., "splits": ...}}, or None if there is no file
    (fp8_kernel.py:738-776)."""
    if (block_n, block_k) != (128, 128):
        return None
    path = Path(config_dir or CONFIG_DIR) / config_file_name(N, K, dtype)
    if not path.exists():
        return None
    with open(path) as f:
        return {int(key): val for key, val in json.load(f).items()}


def ranges_of(table: Dict[int, Any]) -> List[Tuple[int, int, int, int]]:
    """[(m_lo, m_hi, tile, splits)]: every M goes to the key closest to it (ties to the smaller key)."""
    keys = sorted(table)
    out = []
    for i, m in enumerate(keys):
        lo = 0 if i == 0 else (keys[i - 1] + m) // 2 + 1
        hi = M_MAX if i == len(keys) - 1 else (m + keys[i + 1]) // 2
        out.append((lo, hi, int(table[m].get("tile", 0)), int(table[m].get("splits", 0))))
    return out


def parse_file_name(name: str) -> Optional[Tuple[int, int, str, str]]:
    """(N, K, device_name, dtype) of a table's file name, None for other files."""
    if not name.endswith(",block_shape=[128, 128].json"):
        return None
    fields = dict(part.split("=", 1) for part in name[: -len(",block_shape=[128, 128].json")].split(",") if "=" in part)
    try:
        return int(fields["N"]), int(fields["K"]), fields["device_name"], fields["dtype"]
    except (KeyError, ValueError):
        return None


def load_tuned_configs(config_dir: Optional[os.PathLike] = None, device_name: str = DEVICE_NAME) -> int:
    """Hands every table of `config_dir` for this device to the library (replacing what it held);
    returns the number of (N, K, M range) entries.  Call once at start-up."""
    lib = _lib.load()
    lib.sglq_tuned_clear()
    count = 0
    directory = Path(config_dir or CONFIG_DIR)
    if not directory.is_dir():
        return 0
    for path in sorted(directory.iterdir()):
        parsed = parse_file_name(path.name)
        if parsed is None or parsed[2] != device_name or parsed[3] not in KIND_OF_DTYPE:
            continue
        n, k, _, dtype = parsed
        with open(path) as f:
            table = {int(key): val for key, val in json.load(f).items()}
        for lo, hi, tile, splits in ranges_of(table):
            if tile == 0 and splits == 0:
                continue  # the built-in selection
            _lib.check(lib.sglq_tuned_add(KIND_OF_DTYPE[dtype], n, k, lo, hi, tile, splits), "tuned_add")
            count += 1
    return count


def save_config(N: int, K: int, table: Dict[int, Dict[str, int]], config_dir: Optional[os.PathLike] = None,
                dtype: str = "fp8_w8a8") -> Path:
    directory = Path(config_dir or CONFIG_DIR)
    directory.mkdir(parents=True, exist_ok=True)
    path = directory / config_file_name(N, K, dtype)
    with open(path, "w") as f:
        json.dump({str(m): table[m] for m in sorted(table)}, f, indent=4)
        f.write("\n")
    return path
