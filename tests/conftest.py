import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "deepseek-v3_amd"))
sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def coracle():
    """The plain-C oracle (oracle/dsv3_oracle.c), built on demand with gcc."""
    import ctypes
    import subprocess
    so = ROOT / "oracle" / "_build" / "libdsv3_oracle.so"
    src = ROOT / "oracle" / "dsv3_oracle.c"
    if not so.exists() or so.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    lib = ctypes.CDLL(str(so))
    c = ctypes
    lib.oracle_bf16_to_f32.restype = c.c_float
    lib.oracle_bf16_to_f32.argtypes = [c.c_uint16]
    lib.oracle_f32_to_bf16.restype = c.c_uint16
    lib.oracle_f32_to_bf16.argtypes = [c.c_float]
    lib.oracle_e4m3_to_f32.restype = c.c_float
    lib.oracle_e4m3_to_f32.argtypes = [c.c_uint8]
    lib.oracle_f32_to_e4m3.restype = c.c_uint8
    lib.oracle_f32_to_e4m3.argtypes = [c.c_float]
    lib.oracle_ue8m0_round_up.restype = c.c_float
    lib.oracle_ue8m0_round_up.argtypes = [c.c_float]
    lib.oracle_act_quant.restype = None
    lib.oracle_act_quant.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int]
    lib.oracle_weight_dequant.restype = None
    lib.oracle_weight_dequant.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int64, c.c_int64, c.c_int]
    lib.oracle_fp8_gemm.restype = None
    lib.oracle_fp8_gemm.argtypes = [c.c_void_p] * 6 + [c.c_int64] * 3
    return lib
