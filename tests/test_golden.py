"""The committed golden vectors (tests/golden/*.npz, written by make_golden.py) against
the oracle on the CPU and against the HIP path on the GPU."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle

G = Path(__file__).resolve().parent / "golden"
FP8 = torch.float8_e4m3fn


def _load(name):
    return {k: torch.from_numpy(v) for k, v in np.load(G / name, allow_pickle=False).items()}


def test_oracle_reproduces_golden():
    d = _load("act_quant.npz")
    x = d["x_bf16_bits"].view(torch.bfloat16)
    for tag, fmt in (("none", None), ("ue8m0", "ue8m0")):
        y, s = oracle.act_quant(x, 128, fmt)
        assert torch.equal(y.view(torch.uint8), d[f"y_{tag}"]) and torch.equal(s, d[f"s_{tag}"])
    d = _load("weight_dequant.npz")
    y = oracle.weight_dequant(d["w8"].view(FP8), d["s"])
    assert torch.equal(y.view(torch.int16), d["y_bf16_bits"])
    d = _load("fp8_gemm.npz")
    c = oracle.fp8_gemm_f32(d["a"].view(FP8), d["a_s"], d["b"].view(FP8), d["b_s"])
    assert torch.equal(c, d["c_f32"])


@pytest.mark.gpu
def test_hip_path_reproduces_golden():
    import dsv3fp8 as K
    d = _load("act_quant.npz")
    x = d["x_bf16_bits"].view(torch.bfloat16).cuda()
    for tag, fmt in (("none", None), ("ue8m0", "ue8m0")):
        y, s = K.act_quant(x, 128, fmt)
        assert torch.equal(y.cpu().view(torch.uint8), d[f"y_{tag}"]) and torch.equal(s.cpu(), d[f"s_{tag}"])
    d = _load("weight_dequant.npz")
    torch.set_default_dtype(torch.bfloat16)
    try:
        y = K.weight_dequant(d["w8"].view(FP8).cuda(), d["s"].cuda())
    finally:
        torch.set_default_dtype(torch.float32)
    assert torch.equal(y.cpu().view(torch.int16), d["y_bf16_bits"])
    d = _load("fp8_gemm.npz")
    c = K.fp8_gemm_f32(d["a"].view(FP8).cuda(), d["a_s"].cuda(), d["b"].view(FP8).cuda(), d["b_s"].cuda()).cpu()
    ref = d["c_f32"]
    assert (c - ref).abs().max() <= 1e-2 * ref.pow(2).mean().sqrt()
