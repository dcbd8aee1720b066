"""PyTorch-ROCm custom ops over the C ABI.

``torch.ops.dsv3fp8.{act_quant, weight_dequant, fp8_gemm}`` take and return
torch tensors; the device implementations hand raw device pointers and the
current HIP stream of the tensors' device to libdsv3fp8.so.  Only a device
("CUDA" dispatch key, which is HIP on ROCm) implementation and a shape-only Meta
implementation are registered: calling an op on CPU tensors raises.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.float32: _lib.F32}
_CODE_DTYPE = {v: k for k, v in _DTYPE_CODE.items()}
FP8 = torch.float8_e4m3fn

_libdef = torch.library.Library("dsv3fp8", "DEF")
_libdef.define("act_quant(Tensor x, int block_size, int scale_fmt) -> (Tensor, Tensor)")
_libdef.define("weight_dequant(Tensor x, Tensor s, int block_size, int out_dtype) -> Tensor")
_libdef.define("fp8_gemm(Tensor a, Tensor a_s, Tensor b, Tensor b_s, int out_dtype) -> Tensor")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"dsv3fp8: unsupported dtype {dtype} (bf16, fp16 and fp32 are implemented)") from None


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


# split-K scratch, one buffer per (device, stream): calls on one stream are ordered, so they can share it
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _workspace(t: torch.Tensor, nbytes: int, stream: int) -> torch.Tensor:
    key = (t.device.index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 22), dtype=torch.uint8, device=t.device)
        _workspaces[key] = ws
    return ws


def _act_quant_dev(x: torch.Tensor, block_size: int, scale_fmt: int):
    y = torch.empty_like(x, dtype=FP8)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32)
    with torch.cuda.device(x.device):
        rc = _lib.lib.dsv3_act_quant(x.data_ptr(), dtype_code(x.dtype), y.data_ptr(), s.data_ptr(),
                                     x.numel(), x.size(-1), block_size, scale_fmt, _stream(x))
    _lib.check(rc, "dsv3_act_quant")
    return y, s


def _act_quant_meta(x, block_size, scale_fmt):
    return (torch.empty_like(x, dtype=FP8),
            x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32))


def _weight_dequant_dev(x: torch.Tensor, s: torch.Tensor, block_size: int, out_dtype: int):
    y = torch.empty_like(x, dtype=_CODE_DTYPE[out_dtype])
    m, n = x.size()
    with torch.cuda.device(x.device):
        rc = _lib.lib.dsv3_weight_dequant(x.data_ptr(), s.data_ptr(), y.data_ptr(), out_dtype,
                                          m, n, block_size, _stream(x))
    _lib.check(rc, "dsv3_weight_dequant")
    return y


def _weight_dequant_meta(x, s, block_size, out_dtype):
    return torch.empty_like(x, dtype=_CODE_DTYPE[out_dtype])


def _fp8_gemm_dev(a, a_s, b, b_s, out_dtype: int):
    k = a.size(-1)
    m = a.numel() // k if k else 0
    n = b.size(0)
    c = a.new_empty(*a.size()[:-1], n, dtype=_CODE_DTYPE[out_dtype])
    with torch.cuda.device(a.device):
        stream = _stream(a)
        need = _lib.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k)
        ws = _workspace(a, need, stream) if need else None
        rc = _lib.lib.dsv3_fp8_gemm(a.data_ptr(), a_s.data_ptr(), b.data_ptr(), b_s.data_ptr(),
                                    c.data_ptr(), out_dtype, m, n, k,
                                    ws.data_ptr() if ws is not None else None,
                                    ws.numel() if ws is not None else 0, stream)
    _lib.check(rc, "dsv3_fp8_gemm")
    return c


def _fp8_gemm_meta(a, a_s, b, b_s, out_dtype):
    return a.new_empty(*a.size()[:-1], b.size(0), dtype=_CODE_DTYPE[out_dtype])


_libimpl = torch.library.Library("dsv3fp8", "IMPL")
_libimpl.impl("act_quant", _act_quant_dev, "CUDA")
_libimpl.impl("weight_dequant", _weight_dequant_dev, "CUDA")
_libimpl.impl("fp8_gemm", _fp8_gemm_dev, "CUDA")
_libimpl.impl("act_quant", _act_quant_meta, "Meta")
_libimpl.impl("weight_dequant", _weight_dequant_meta, "Meta")
_libimpl.impl("fp8_gemm", _fp8_gemm_meta, "Meta")
