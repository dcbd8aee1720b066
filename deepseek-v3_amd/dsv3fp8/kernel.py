"""Drop-in replacement for the reference's ``inference/kernel.py``.

Same three names, signatures, defaults, asserts and return conventions
(reference: inference/kernel.py:38-57, 89-110, 175-196); the work is done by
hand-written gfx950 kernels behind ``torch.ops.dsv3fp8``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib, ops

_SCALE_FMT = {None: _lib.SCALE_FMT_NONE, "ue8m0": _lib.SCALE_FMT_UE8M0}


def act_quant(x: torch.Tensor, block_size: int = 128,
              scale_fmt: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Block-wise dynamic quantisation of ``x`` (inference/kernel.py:38-57).

    Returns ``(y, s)``: ``y`` has the shape of ``x`` in ``torch.float8_e4m3fn``;
    ``s`` is fp32 of shape ``[*x.shape[:-1], x.size(-1) // block_size]`` holding
    ``max(amax, 1e-4) / 448`` per block (rounded up to a power of two for
    ``scale_fmt="ue8m0"``; any other value means no rounding, as in the
    reference's ``scale_fmt == "ue8m0"`` test).
    """
    assert x.is_contiguous(), 'Input tensor must be contiguous'
    assert x.size(-1) % block_size == 0, f'Last dimension size must be divisible by block_size (block_size={block_size})'
    fmt = _SCALE_FMT.get(scale_fmt, _lib.SCALE_FMT_NONE)
    return torch.ops.dsv3fp8.act_quant(x, block_size, fmt)


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """``y = x * s`` per ``block_size`` x ``block_size`` tile, in the default dtype
    (inference/kernel.py:89-110)."""
    assert x.is_contiguous() and s.is_contiguous(), 'Input tensors must be contiguous'
    assert x.dim() == 2 and s.dim() == 2, 'Input tensors must have 2 dimensions'
    return torch.ops.dsv3fp8.weight_dequant(x, s, block_size, ops.dtype_code(torch.get_default_dtype()))


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """``c = a @ b.T`` with per-128-K-block fp32 rescaling, in the default dtype
    (inference/kernel.py:175-196)."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    return torch.ops.dsv3fp8.fp8_gemm(a, a_s, b, b_s, ops.dtype_code(torch.get_default_dtype()))


def fp8_gemm_pow2(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """``fp8_gemm`` for scales that are all powers of two -- ``act_quant(..., scale_fmt="ue8m0")`` activations
    (inference/kernel.py:29-31) on a weight whose block scales are stored that way (the format of
    inference/configs/config_v3.1.json:22).  Not in the reference, whose ``fp8_gemm`` multiplies by the scales
    whatever they are; here the caller vouches for the property and the large-M kernel hands the scales to the
    matrix instruction instead of multiplying per K block."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    return torch.ops.dsv3fp8.fp8_gemm_pow2(a, a_s, b, b_s, ops.dtype_code(torch.get_default_dtype()))


def fp8_gemm_f32(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """``fp8_gemm`` with the binary32 accumulators returned unrounded (not in the
    reference; the output-type knob the reference reaches through the default dtype)."""
    assert a.is_contiguous() and b.is_contiguous(), 'Input tensors must be contiguous'
    assert a_s.is_contiguous() and b_s.is_contiguous(), 'Scaling factor tensors must be contiguous'
    return torch.ops.dsv3fp8.fp8_gemm(a, a_s, b, b_s, _lib.F32)
