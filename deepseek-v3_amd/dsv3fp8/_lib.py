"""ctypes binding of libdsv3fp8.so (the C ABI declared in include/dsv3_fp8.h).

The library is loaded from ``deepseek-v3_amd/lib``; there is no fallback: if it
has not been built the import fails with the command that builds it.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent.parent / "lib" / "libdsv3fp8.so"

# enum dsv3_dtype / dsv3_scale_fmt / dsv3_status (include/dsv3_fp8.h)
BF16, F16, F32 = 0, 1, 2
SCALE_FMT_NONE, SCALE_FMT_UE8M0 = 0, 1
ABSORB_Q, ABSORB_V = 0, 1
SCORE_SOFTMAX, SCORE_SIGMOID = 0, 1
OK = 0

EXPORTS = {
    "dsv3_version": (c_int, []),
    "dsv3_status_string": (c_char_p, [c_int]),
    "dsv3_act_quant": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]),
    "dsv3_weight_dequant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p]),
    "dsv3_weight_quant": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]),
    "dsv3_fp8_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                              c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "dsv3_fp8_gemm_pow2": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                   c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "dsv3_fp8_gemm_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                     c_int64, c_int64, c_int64, c_void_p]),
    "dsv3_fp8_gemm_static_max_bytes": (c_size_t, []),
    "dsv3_linear_fp8_fused": (c_int, [c_int64, c_int64, c_int64]),
    "dsv3_linear_fp8": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64,
                                c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "dsv3_fp8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "dsv3_fp8_gemm_grouped_tile_rows": (c_int, []),
    "dsv3_group_tiles": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dsv3_moe_route": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dsv3_fp8_gemm_grouped": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                      c_void_p, c_int, c_int64, c_int64, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "dsv3_fp8_gemm_grouped_pow2": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                           c_void_p, c_int, c_int64, c_int64, c_int64,
                                           c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "dsv3_fp8_gemm_grouped_swiglu_fused": (c_int, [c_int64, c_int64, c_int64, c_int64]),
    "dsv3_fp8_gemm_grouped_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                             c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                             c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "dsv3_swiglu_quant": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]),
    "dsv3_moe_combine": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int64, c_int, c_int64, c_void_p]),
    "dsv3_gate_route": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                c_int, c_float, c_void_p]),
    "dsv3_wkv_b_absorb": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                  c_int64, c_int, c_int, c_int, c_int64, c_int, c_void_p]),
}


def _load() -> ctypes.CDLL:
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP library has not been built. "
            f"Run `python {LIB_PATH.parent.parent / 'build.py'}` (needs hipcc); there is no CPU fallback.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in EXPORTS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def status_string(code: int) -> str:
    return lib.dsv3_status_string(int(code)).decode()


def check(code: int, what: str) -> None:
    if code != OK:
        raise RuntimeError(f"{what} failed: {status_string(code)} (dsv3_status {code})")
