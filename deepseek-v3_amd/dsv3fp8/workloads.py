"""Seeded synthetic inputs for the benchmark and parity configurations.

Every generator draws from a ``torch.Generator`` on the requested device, so the
same code makes the small CPU cases the parity tests compare on and the
full-size on-device cases the benchmark times.  Shapes are those of the 671B
configuration (reference: inference/configs/config_671B.json, through the layer
constructors at inference/model.py:424-433, 518-520, 619-621).
"""
from __future__ import annotations

from typing import Tuple

import torch

from .quantize import block_quant_weight

FP8 = torch.float8_e4m3fn

# (K -> N) of the MLA projections used for the decode sweep
DECODE_SHAPES = {
    "wq_a": (7168, 1536),
    "wq_b": (1536, 24576),
    "wkv_a": (7168, 576),
    "wkv_b": (512, 32768),
    "wo": (16384, 7168),
}
# the sweep the benchmark times: the five projections plus wq_a and wkv_a as the one stacked GEMM that the attention
# layer launches for them (both read the same input; model.py:424-427)
DECODE_SWEEP = dict(DECODE_SHAPES, wq_a_wkv_a_stacked=(7168, 2112))
DECODE_M = (1, 8, 32, 64)
# dense MLP projections for the prefill case (K -> N), M = 4096 tokens
PREFILL_SHAPES = {"w1": (7168, 18432), "w2": (18432, 7168)}
PREFILL_M = 4096


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def activations(m: int, k: int, seed: int = 0, device="cpu", outliers: bool = False) -> torch.Tensor:
    """bf16 [m,k] ~ N(0,1); with ``outliers`` a random 1 % of the elements is multiplied by 10."""
    g = _gen(seed, device)
    x = torch.randn(m, k, generator=g, device=device, dtype=torch.float32)
    if outliers:
        mask = torch.rand(m, k, generator=g, device=device) < 0.01
        x = torch.where(mask, x * 10.0, x)
    return x.to(torch.bfloat16)


def weight(n: int, k: int, seed: int = 1, device="cpu") -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8 weight [n,k] + fp32 scales [ceil(n/128), ceil(k/128)], block-quantised from bf16 ~ N(0, 0.02)."""
    g = _gen(seed, device)
    w = (torch.randn(n, k, generator=g, device=device, dtype=torch.float32) * 0.02).to(torch.bfloat16)
    return block_quant_weight(w)


def random_fp8_weight(m: int, n: int, seed: int = 2, device="cpu") -> Tuple[torch.Tensor, torch.Tensor]:
    """Uniformly random finite e4m3fn bytes [m,n] (no 0x7f/0xff NaN) and scales ~ U(1e-4, 1e-3)."""
    g = _gen(seed, device)
    b = torch.randint(0, 256, (m, n), generator=g, device=device, dtype=torch.int16)
    b = torch.where((b & 0x7F) == 0x7F, b & 0x80, b).to(torch.uint8)
    s = torch.rand(-(-m // 128), -(-n // 128), generator=g, device=device) * 9e-4 + 1e-4
    return b.view(FP8), s.float()


def cfg1_cpu_plumbing(device="cpu"):
    """x bf16 [16,7168] ~ N(0,1); wq_a-shaped weight [1536,7168]; one seeded stream (seed 0)."""
    g = _gen(0, device)
    x = torch.randn(16, 7168, generator=g, device=device).to(torch.bfloat16)
    w = (torch.randn(1536, 7168, generator=g, device=device) * 0.02).to(torch.bfloat16)
    w8, ws = block_quant_weight(w)
    return x, w8, ws
