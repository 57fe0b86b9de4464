import ctypes
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def c_oracle():
    """The scalar C restatement (oracle/w8a8_oracle.c) as a ctypes library."""
    so = ROOT / "oracle" / "liboracle.so"
    src = ROOT / "oracle" / "w8a8_oracle.c"
    if not so.exists() or so.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(ROOT / "oracle"), "-B", "liboracle.so"], check=True, capture_output=True)
    lib = ctypes.CDLL(str(so))
    lib.oracle_e4m3fn_encode.argtypes = [ctypes.c_float]
    lib.oracle_e4m3fn_encode.restype = ctypes.c_uint8
    lib.oracle_e4m3fn_decode.argtypes = [ctypes.c_uint8]
    lib.oracle_e4m3fn_decode.restype = ctypes.c_float
    return lib


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
