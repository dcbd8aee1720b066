"""Offline weight block-quantiser: bf16/fp32 weight -> (fp8 e4m3fn, fp32 scales).

Produces the on-disk format that ``weight_dequant`` / ``fp8_gemm`` consume
(reference: README_WEIGHTS.md:60-92, the ``weight`` + ``weight_scale_inv`` pair;
scale tensor shape as in inference/model.py:184-187).  Plain torch ops on the
tensor's own device; this is set-up code, not part of the per-token hot path.
"""
from __future__ import annotations

from typing import Tuple

import torch

FP8 = torch.float8_e4m3fn


def block_quant_weight(w: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
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
    w8 = (tiles / scale[:, None, :, None]).reshape(mb * block_size, nb * block_size)[:m, :n]
    return w8.contiguous().to(FP8), scale
