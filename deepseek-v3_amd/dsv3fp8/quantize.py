"""Weight block-quantiser: bf16/fp16/fp32 weight -> (fp8 e4m3fn, fp32 scales).

Produces the on-disk format that ``weight_dequant`` / ``fp8_gemm`` consume
(reference: README_WEIGHTS.md:60-92, the ``weight`` + ``weight_scale_inv`` pair;
scale tensor shape as in inference/model.py:184-187).

``weight_quant`` is the device path (the gfx950 kernel behind ``torch.ops.dsv3fp8.weight_quant``);
``block_quant_weight`` states the same rule in plain torch ops on the tensor's own device and is what
the synthetic-input generators use (on the host the two agree bit for bit; torch's device division is not
correctly rounded, so on a GPU its scales can differ from the kernel's in the last place).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn


def block_quant_weight(w: torch.Tensor, block_size: int = 128,
                       scale_fmt: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per ``block_size`` x ``block_size`` tile: ``scale = max(amax, 1e-4) / 448`` and
    ``w8 = e4m3(w / scale)``.  Ragged edge tiles are zero-padded before the amax
    (README_WEIGHTS.md:89) and cropped afterwards.  Returns ``(w8 [m,n], scale
    [ceil(m/b), ceil(n/b)])`` with ``w ~= w8 * scale`` tile-wise."""
    assert w.dim() == 2
    m, n = w.shape
    mb, nb = -(-m // block_size), -(-n // block_size)
    wf = w.float()
    if mb * block_size != m or nb * block_size != n:
        wf = torch.nn.functional.pad(wf, (0, nb * block_size - n, 0, mb * block_size - m))
    tiles = wf.view(mb, block_size, nb, block_size)
    amax = tiles.abs().amax(dim=(1, 3)).clamp_min(1e-4)
    scale = amax / 448.0
    if scale_fmt == "ue8m0":                  # round up to a power of two (inference/kernel.py:29-31)
        bits = scale.view(torch.int32)          # next power of two, on the bits: exponent + (mantissa != 0)
        scale = (((bits >> 23) + ((bits & 0x7FFFFF) != 0).int()) << 23).view(torch.float32)
    w8 = (tiles / scale[:, None, :, None]).reshape(mb * block_size, nb * block_size)[:m, :n]
    return w8.contiguous().to(FP8), scale


def weight_quant(w: torch.Tensor, block_size: int = 128,
                 scale_fmt: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``block_quant_weight`` on the device: one pass over ``w`` (2-D, contiguous, on the GPU) by the HIP kernel.
    Returns ``(w8 [m,n] e4m3fn, scale [ceil(m/128), ceil(n/128)] fp32)``; ``scale_fmt="ue8m0"`` rounds every
    scale up to a power of two, as ``act_quant`` does."""
    from . import _lib, ops  # noqa: F401  (registers torch.ops.dsv3fp8)
    assert w.is_contiguous(), 'Input tensor must be contiguous'
    assert w.dim() == 2, 'Input tensor must have 2 dimensions'
    fmt = _lib.SCALE_FMT_UE8M0 if scale_fmt == "ue8m0" else _lib.SCALE_FMT_NONE
    return torch.ops.dsv3fp8.weight_quant(w, block_size, fmt)
