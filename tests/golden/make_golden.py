"""Writes tests/golden/*.npz: small input/expected-output vectors of the three
kernels, computed by the torch-CPU oracle and cross-checked against the plain-C
oracle before they are written.  The reference ships no vectors for this path
(it has no tests), so these fix the oracle's behaviour against drift.

    python tests/golden/make_golden.py
"""
import ctypes
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "deepseek-v3_amd"))

from oracle import oracle  # noqa: E402


def main():
    subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    C = ctypes.CDLL(str(ROOT / "oracle" / "_build" / "libdsv3_oracle.so"))
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    g = torch.Generator().manual_seed(1234)

    # act_quant: random magnitudes per row + special rows
    x = (torch.randn(12, 256, generator=g) * torch.pow(10.0, torch.randint(-5, 3, (12, 1), generator=g).float()))
    x[0] = 0.0
    x[1, :128] = 5e-5
    x[2, 128:] = -0.0
    x[3, :8] = torch.tensor([17., 19., 21., 23., 448., -448., 2.0 ** -10, 3 * 2.0 ** -10])
    x = x.bfloat16()
    out = {}
    for fmt in (None, "ue8m0"):
        y, s = oracle.act_quant(x, 128, fmt)
        yc = torch.empty(x.numel(), dtype=torch.uint8)
        sc = torch.empty(x.numel() // 128, dtype=torch.float32)
        C.oracle_act_quant(p(x.view(torch.int16)), p(yc), p(sc), ctypes.c_int64(x.numel()), 128, int(fmt == "ue8m0"))
        assert torch.equal(yc.view(12, 256), y.view(torch.uint8)) and torch.equal(sc.view(12, 2), s)
        tag = fmt or "none"
        out[f"y_{tag}"] = y.view(torch.uint8).numpy()
        out[f"s_{tag}"] = s.numpy()
    np.savez_compressed(HERE / "act_quant.npz", x_bf16_bits=x.view(torch.int16).numpy(), **out)

    # weight_dequant: ragged [130, 272]
    w8 = torch.randint(0, 256, (130, 272), generator=g, dtype=torch.int16).to(torch.uint8)
    w8 = torch.where((w8 & 0x7F) == 0x7F, w8 & 0x80, w8)
    s = torch.rand(2, 3, generator=g) * 9e-4 + 1e-4
    y = oracle.weight_dequant(w8.view(torch.float8_e4m3fn), s)
    yc = torch.empty(130, 272, dtype=torch.int16)
    C.oracle_weight_dequant(p(w8), p(s), p(yc), ctypes.c_int64(130), ctypes.c_int64(272), 128)
    assert torch.equal(yc, y.view(torch.int16))
    np.savez_compressed(HERE / "weight_dequant.npz", w8=w8.numpy(), s=s.numpy(), y_bf16_bits=y.view(torch.int16).numpy())

    # fp8_gemm: (M,N,K) = (5,130,256), ragged N
    xa = torch.randn(5, 256, generator=g).bfloat16()
    w = (torch.randn(130, 256, generator=g) * 0.02).bfloat16()
    a, a_s = oracle.act_quant(xa)
    b, b_s = oracle.block_quant_weight(w)
    c = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    cc = torch.empty(5, 130, dtype=torch.float32)
    C.oracle_fp8_gemm(p(a.view(torch.uint8)), p(a_s), p(b.view(torch.uint8)), p(b_s), p(cc), None,
                      ctypes.c_int64(5), ctypes.c_int64(130), ctypes.c_int64(256))
    assert (cc - c).abs().max() <= 2e-6 * c.pow(2).mean().sqrt()
    np.savez_compressed(HERE / "fp8_gemm.npz", a=a.view(torch.uint8).numpy(), a_s=a_s.numpy(),
                        b=b.view(torch.uint8).numpy(), b_s=b_s.numpy(), c_f32=c.numpy())
    print("wrote", sorted(f.name for f in HERE.glob("*.npz")))


if __name__ == "__main__":
    main()
