"""Pins the oracle's number formats: the plain-C conversions (written with integer
bit manipulation) against the OCP E4M3 / bfloat16 definitions and against torch's
CPU casts -- two independent implementations that have to agree everywhere."""
import ctypes
import math

import numpy as np
import torch

from oracle import oracle

FP8 = torch.float8_e4m3fn


def _c_decode_all(coracle):
    return torch.tensor([coracle.oracle_e4m3_to_f32(b) for b in range(256)], dtype=torch.float32)


def test_e4m3_decode_known_values(coracle):
    d = _c_decode_all(coracle)
    # OCP 8-bit floating point spec, E4M3: bias 7, no inf, S.1111.111 = NaN, max 448
    assert d[0x00].item() == 0.0 and math.copysign(1, d[0x80].item()) == -1.0
    assert d[0x01].item() == 2.0 ** -9          # smallest subnormal
    assert d[0x07].item() == 7 * 2.0 ** -9      # largest subnormal
    assert d[0x08].item() == 2.0 ** -6          # smallest normal
    assert d[0x38].item() == 1.0
    assert d[0x3C].item() == 1.5
    assert d[0x7E].item() == 448.0 and d[0xFE].item() == -448.0
    assert math.isnan(d[0x7F].item()) and math.isnan(d[0xFF].item())
    # closed form for every byte
    for b in range(256):
        e, m, sgn = (b >> 3) & 15, b & 7, -1.0 if b & 0x80 else 1.0
        if e == 15 and m == 7:
            continue
        want = sgn * (m / 8 * 2.0 ** -6 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
        assert d[b].item() == want


def test_e4m3_decode_matches_torch(coracle):
    d = _c_decode_all(coracle)
    t = torch.arange(256, dtype=torch.int16).to(torch.uint8).view(FP8).float()
    nan = t.isnan()
    assert torch.equal(nan, d.isnan())
    assert torch.equal(t[~nan].view(torch.int32), d[~nan].view(torch.int32))


def _c_encode(coracle, f: torch.Tensor) -> torch.Tensor:
    enc = np.frompyfunc(lambda v: coracle.oracle_f32_to_e4m3(ctypes.c_float(v)), 1, 1)
    return torch.from_numpy(enc(f.numpy()).astype(np.uint8))


def test_e4m3_encode_known_roundings(coracle):
    enc = lambda v: coracle.oracle_f32_to_e4m3(ctypes.c_float(v))
    dec = lambda b: coracle.oracle_e4m3_to_f32(b)
    assert dec(enc(17.0)) == 16.0 and dec(enc(19.0)) == 20.0       # ties to even (grid step 2 in [16,32))
    assert dec(enc(21.0)) == 20.0 and dec(enc(23.0)) == 24.0
    assert enc(448.0) == 0x7E and enc(-448.0) == 0xFE
    assert enc(463.9) == 0x7E                                      # still rounds down to 448
    assert enc(464.0) == 0x7F and enc(1e9) == 0x7F                 # no finite encoding
    assert enc(float("inf")) == 0x7F and enc(float("nan")) & 0x7F == 0x7F
    assert enc(2.0 ** -10) == 0x00                                  # tie between 0 and 2^-9 -> even (0)
    assert enc(3 * 2.0 ** -10) == 0x02                              # tie between 1 and 2 (x 2^-9) -> even
    assert enc(2.0 ** -10 * 1.0001) == 0x01
    assert enc(-1e-30) == 0x80 and enc(-0.0) == 0x80 and enc(0.0) == 0x00
    assert enc(7.5 * 2.0 ** -9) == 0x08                             # subnormal tie carries into the first normal
    assert enc(1.0) == 0x38 and enc(1.0625) == 0x38 and enc(1.0626) == 0x39 and enc(1.1875) == 0x3A


def test_e4m3_encode_matches_torch_everywhere_it_matters(coracle):
    g = torch.Generator().manual_seed(0)
    bits = torch.arange(65536, dtype=torch.int32)
    all_bf16 = (bits << 16).view(torch.float32)                          # every bf16 value as f32
    rnd = (torch.randn(200_000, generator=g) * torch.pow(2.0, torch.randint(-14, 10, (200_000,), generator=g).float()))
    grid = torch.arange(256, dtype=torch.int16).to(torch.uint8).view(FP8).float()
    grid = grid[~grid.isnan()]
    mids = (grid[:, None] + grid[None, :]).flatten() / 2                 # includes every tie point
    near = torch.cat([torch.nextafter(mids, torch.tensor(1e9)), torch.nextafter(mids, torch.tensor(-1e9))])
    f = torch.cat([all_bf16, rnd, mids, near, torch.tensor([448.0, 463.99, -463.99, 2.0 ** -10, -2.0 ** -10])])
    f = f[f.abs() < 464.0]                                               # torch and the C code both give NaN beyond
    want = f.to(FP8).view(torch.uint8)
    got = _c_encode(coracle, f)
    assert torch.equal(got, want)


def test_e4m3_round_trip(coracle):
    for b in range(256):
        if b & 0x7F == 0x7F:
            continue
        assert coracle.oracle_f32_to_e4m3(coracle.oracle_e4m3_to_f32(b)) == b


def test_bf16_rounding_matches_torch_and_ties(coracle):
    g = torch.Generator().manual_seed(1)
    f = torch.cat([torch.randn(100_000, generator=g) * 1e3, torch.randn(1000, generator=g) * 1e-40,
                   torch.tensor([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, 3.3895e38, 3.4e38, -0.0])])
    enc = np.frompyfunc(lambda v: coracle.oracle_f32_to_bf16(ctypes.c_float(v)), 1, 1)
    got = torch.from_numpy(enc(f.numpy()).astype(np.uint16).view(np.int16))
    assert torch.equal(got, f.to(torch.bfloat16).view(torch.int16))
    assert coracle.oracle_f32_to_bf16(ctypes.c_float(1.0 + 2.0 ** -8)) == 0x3F80        # tie -> even (down)
    assert coracle.oracle_f32_to_bf16(ctypes.c_float(1.0 + 3 * 2.0 ** -8)) == 0x3F82    # tie -> even (up)
    assert coracle.oracle_f32_to_bf16(ctypes.c_float(3.4e38)) == 0x7F80                 # rounds to +inf
    for h in (0x0000, 0x8000, 0x0001, 0x3F80, 0x7F7F, 0xC2F7):
        assert coracle.oracle_f32_to_bf16(coracle.oracle_bf16_to_f32(h)) == h


def test_ue8m0_round_up(coracle):
    vals = [1.0, 1.0000001, 1.5, 2.0, 0.75, 2.2321428616578487e-07, 3.0e-3, 1e30, 2.0 ** -100]
    for v in vals:
        v32 = torch.tensor(v, dtype=torch.float32).item()
        want = 2.0 ** math.ceil(math.log2(v32))      # the reference's formula (kernel.py:30-31), in double
        assert coracle.oracle_ue8m0_round_up(ctypes.c_float(v32)) == want
        assert oracle.ue8m0_round_up(torch.tensor([v32])).item() == want
    g = torch.Generator().manual_seed(2)
    s = torch.rand(10000, generator=g) * torch.pow(2.0, torch.randint(-30, 30, (10000,), generator=g).float()) + 1e-30
    up = oracle.ue8m0_round_up(s)
    assert bool((up >= s).all()) and bool((up < 2 * s).all())
    assert bool(((up.view(torch.int32) & 0x7FFFFF) == 0).all())
    # non-finite scales (a block that holds an infinity or a NaN): exp2(ceil(log2(s))) returns them unchanged
    odd = torch.tensor([float("inf"), float("nan")])
    want = torch.exp2(torch.ceil(torch.log2(odd)))
    got = oracle.ue8m0_round_up(odd)
    assert bool(torch.isinf(got[0])) and got[0] > 0 and bool(torch.isnan(got[1]))
    assert torch.equal(torch.isnan(got), torch.isnan(want)) and torch.equal(torch.isinf(got), torch.isinf(want))
