"""Pins the torch-CPU oracle of the three kernels (oracle/oracle.py): against the
independent plain-C restatement, against closed-form known answers and invariants,
and against brute force on tiny problems.  The reference ships no tests or golden
vectors for this path, so these are what anchor parity."""
import ctypes
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle

FP8 = torch.float8_e4m3fn
ROOT = Path(__file__).resolve().parent.parent


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def c_act_quant(coracle, x, block=128, ue8m0=False):
    xb = x.contiguous().view(torch.int16)
    y = torch.empty(x.numel(), dtype=torch.uint8)
    s = torch.empty(x.numel() // block, dtype=torch.float32)
    coracle.oracle_act_quant(_ptr(xb), _ptr(y), _ptr(s), x.numel(), block, int(ue8m0))
    return y.view(x.shape), s.view(*x.shape[:-1], x.size(-1) // block)


def c_weight_dequant(coracle, w8, s, block=128):
    m, n = w8.shape
    y = torch.empty(m, n, dtype=torch.int16)
    coracle.oracle_weight_dequant(_ptr(w8.view(torch.uint8)), _ptr(s), _ptr(y), m, n, block)
    return y.view(torch.bfloat16)


def c_fp8_gemm(coracle, a, a_s, b, b_s):
    m, k = a.shape
    n = b.shape[0]
    c32 = torch.empty(m, n, dtype=torch.float32)
    c16 = torch.empty(m, n, dtype=torch.int16)
    coracle.oracle_fp8_gemm(_ptr(a.view(torch.uint8)), _ptr(a_s), _ptr(b.view(torch.uint8)), _ptr(b_s),
                            _ptr(c32), _ptr(c16), m, n, k)
    return c32, c16.view(torch.bfloat16)


# ---------------------------------------------------------------- act_quant

def _adversarial_rows():
    rows = [torch.zeros(128), torch.full((128,), -0.0), torch.full((128,), 5e-5), torch.full((128,), 3.0),
            torch.linspace(-448, 448, 128), torch.full((128,), 1e-39), torch.full((128,), 2e38)]
    r = torch.zeros(128); r[17] = -1000.0; rows.append(r)
    r = torch.tensor([17., 19., 21., 23., 2 ** -10, 3 * 2 ** -10, 448., -448.] * 16); rows.append(r)
    return torch.stack(rows).bfloat16()


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_act_quant_torch_equals_c(coracle, fmt):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(64, 1024, generator=g) * torch.pow(10.0, torch.randint(-6, 4, (64, 1), generator=g).float())).bfloat16()
    x = torch.cat([x, _adversarial_rows().repeat(1, 8)])
    y, s = oracle.act_quant(x, 128, fmt)
    yc, sc = c_act_quant(coracle, x, 128, fmt == "ue8m0")
    assert torch.equal(s.view(torch.int32), sc.view(torch.int32))
    assert torch.equal(y.view(torch.uint8), yc)


def test_act_quant_known_answers():
    y, s = oracle.act_quant(torch.zeros(2, 128).bfloat16())
    assert s[0, 0].item() == 2.2321428616578487e-07          # fp32(1e-4) / 448
    assert int(y.view(torch.uint8).max()) == 0
    y, s = oracle.act_quant(torch.full((1, 128), 3.0).bfloat16())
    assert bool((y.view(torch.uint8) == 0x7E).all())          # a constant block is all +448
    assert s.item() == torch.tensor(3.0).div(448.0).item()
    x = torch.zeros(1, 128); x[0, 9] = -7.0
    y, s = oracle.act_quant(x.bfloat16())
    assert int(y.view(torch.uint8)[0, 9]) == 0xFE and int(y.view(torch.uint8).sum()) == 0xFE
    y, _ = oracle.act_quant(torch.full((1, 128), -0.0).bfloat16())
    assert bool((y.view(torch.uint8) == 0x80).all())          # sign of zero survives


def test_act_quant_invariants():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(16, 512, generator=g).bfloat16()
    y, s = oracle.act_quant(x)
    # the amax element of each block encodes to +-448
    mag = (y.view(torch.uint8) & 0x7F).view(16, 4, 128)
    assert bool((mag.amax(-1) == 0x7E).all())
    # scaling a block by 2^k scales s by 2^k and leaves the bytes alone
    y8, s8 = oracle.act_quant((x.float() * 8).bfloat16())
    assert torch.equal(y8.view(torch.uint8), y.view(torch.uint8)) and torch.equal(s8, s * 8)
    # a block depends only on its own 128 inputs
    x2 = x.clone(); x2[:, 128:256] = 99.0
    y2, s2 = oracle.act_quant(x2)
    keep = torch.ones(512, dtype=torch.bool); keep[128:256] = False
    assert torch.equal(y2.view(torch.uint8)[:, keep], y.view(torch.uint8)[:, keep])
    # reconstruction error is at most half an e4m3 ulp at 448's binade (32/2) times s
    err = (y.float().view(16, 4, 128) * s[..., None] - x.float().view(16, 4, 128)).abs()
    assert bool((err <= 16.0 * s[..., None] * (1 + 1e-6)).all())
    # ue8m0: scales are powers of two in [s, 2s)
    _, su = oracle.act_quant(x, 128, "ue8m0")
    assert bool(((su.view(torch.int32) & 0x7FFFFF) == 0).all()) and bool((su >= s).all()) and bool((su < 2 * s).all())


def test_act_quant_rejects_what_the_reference_rejects():
    with pytest.raises(AssertionError):
        oracle.act_quant(torch.zeros(4, 100).bfloat16())
    with pytest.raises(AssertionError):
        oracle.act_quant(torch.zeros(256, 4).bfloat16().t())


def test_fast_division_claim_subsampled():
    """The kernel's x/s shortcut, enumerated on every 32nd amax (the exhaustive run is
    `oracle/_build/check_fast_division 1`, about 10 s on 8 cores)."""
    subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    r = subprocess.run([str(ROOT / "oracle" / "_build" / "check_fast_division"), "32"], capture_output=True, text=True)
    assert r.returncode == 0 and "mismatches=0" in r.stdout, r.stdout + r.stderr


# ---------------------------------------------------------------- weight_dequant

@pytest.mark.parametrize("shape", [(256, 384), (130, 272), (576, 512), (1, 1), (127, 129)])
def test_weight_dequant_torch_equals_c(coracle, shape):
    g = torch.Generator().manual_seed(shape[0])
    w8 = torch.randint(0, 256, shape, generator=g, dtype=torch.int16).to(torch.uint8)
    w8 = torch.where((w8 & 0x7F) == 0x7F, w8 & 0x80, w8).view(FP8)
    s = torch.rand(-(-shape[0] // 128), -(-shape[1] // 128), generator=g) * 9e-4 + 1e-4
    y = oracle.weight_dequant(w8, s)
    yc = c_weight_dequant(coracle, w8, s)
    assert torch.equal(y.view(torch.int16), yc.view(torch.int16))


def test_weight_dequant_known_answers():
    w8 = torch.arange(256, dtype=torch.int16).to(torch.uint8).repeat(2, 1).view(FP8)
    y = oracle.weight_dequant(w8, torch.ones(1, 2)).float()
    assert y[0, 0x38].item() == 1.0 and y[0, 0x7E].item() == 448.0 and y[0, 0x01].item() == 2.0 ** -9
    assert y[0, 0x7F].isnan() and y[0, 0xFF].isnan()
    y4 = oracle.weight_dequant(w8, torch.full((1, 2), 0.25)).float()
    ok = ~y.isnan()
    assert torch.equal(y4[ok], y[ok] * 0.25)                   # power-of-two scales are exact
    # scale indexing: block (i//128, j//128), row stride ceil(n/128)
    w8 = torch.full((300, 300), 0x38, dtype=torch.uint8).view(FP8)
    s = torch.arange(9, dtype=torch.float32).view(3, 3) + 1
    y = oracle.weight_dequant(w8, s).float()
    assert y[0, 0] == 1 and y[0, 128] == 2 and y[128, 0] == 4 and y[299, 299] == 9 and y[127, 255] == 2


def test_block_quant_round_trip_and_padding():
    g = torch.Generator().manual_seed(3)
    w = (torch.randn(200, 300, generator=g) * 0.02).bfloat16()
    w8, s = oracle.block_quant_weight(w)
    assert w8.shape == (200, 300) and s.shape == (2, 3)
    back = oracle.weight_dequant(w8, s, out_dtype=torch.float32)
    es = oracle.expand_block_scale(s, 200, 300)
    assert bool(((back - w.float()).abs() <= 16.0 * es * (1 + 1e-6)).all())
    # the ragged blocks' scales come from their real entries only (zero padding cannot raise an amax)
    assert s[1, 2].item() == pytest.approx(w[128:, 256:].float().abs().max().item() / 448.0, rel=1e-7)
    # product quantiser == oracle quantiser, bit for bit
    from dsv3fp8.quantize import block_quant_weight
    w8p, sp = block_quant_weight(w)
    assert torch.equal(w8p.view(torch.uint8), w8.view(torch.uint8)) and torch.equal(sp, s)


def test_block_quant_known_answers():
    """What pins the quantiser without restating it: weights that ARE e4m3 values times a power-of-two scale, with
    a +-448 in every block, have exactly one quantisation -- those bytes and that scale -- and the reference's
    dequantisation rule (README_WEIGHTS.md:88-90, oracle.weight_dequant) must give the weights back."""
    g = torch.Generator().manual_seed(11)
    m, n = 300, 520                                            # ragged both ways: 3 x 5 blocks
    b = torch.randint(0, 256, (m, n), generator=g, dtype=torch.int16)
    b = torch.where((b & 0x7F) == 0x7F, b & 0x80, b).to(torch.uint8)         # no NaN bytes
    mb, nb = 3, 5
    for i in range(mb):                                        # a 448 (0x7e) or -448 (0xfe) inside every block's real part
        for j in range(nb):
            b[min(i * 128 + 7 * j + 3, m - 1), min(j * 128 + 5 * i + 2, n - 1)] = 0x7E if (i + j) % 2 else 0xFE
    w8 = b.view(FP8)
    s = torch.pow(2.0, torch.randint(-12, 3, (mb, nb), generator=g).float())
    w = oracle.weight_dequant(w8, s, out_dtype=torch.float32)                # exact: 4 significant bits times 2^e
    assert torch.equal(w.bfloat16().float(), w)                              # ... and exactly representable in bf16
    for src in (w, w.bfloat16()):
        q8, qs = oracle.block_quant_weight(src)
        assert torch.equal(qs, s)
        assert torch.equal(q8.float(), w8.float())                           # (+0 and -0 bytes compare equal here)
    # an all-zero block takes the clamp: scale 1e-4 / 448, bytes zero
    q8, qs = oracle.block_quant_weight(torch.zeros(128, 256))
    assert qs[0, 0].item() == pytest.approx(1e-4 / 448, rel=1e-7) and int(q8.view(torch.uint8).max()) == 0
    # every block of a generic weight reaches the largest code, and the quantisation error is within half an e4m3
    # step (2^-4 relative for normal codes, 2^-10 * scale absolute for the subnormal ones)
    wg = (torch.randn(256, 384, generator=g) * 0.03).bfloat16()
    q8, qs = oracle.block_quant_weight(wg)
    assert bool((q8.float().abs().view(2, 128, 3, 128).amax(dim=(1, 3)) == 448).all())
    err = (oracle.weight_dequant(q8, qs, out_dtype=torch.float32) - wg.float()).abs()
    es = oracle.expand_block_scale(qs, 256, 384)
    assert bool((err <= torch.maximum(wg.float().abs() * 2.0 ** -4, es * 2.0 ** -10) * (1 + 1e-6)).all())


# ---------------------------------------------------------------- fp8_gemm

def _rand_problem(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    a, a_s = oracle.act_quant(x)
    b, b_s = oracle.block_quant_weight(w)
    return a, a_s, b, b_s


@pytest.mark.parametrize("mnk", [(3, 130, 256), (16, 576, 512), (33, 128, 1024)])
def test_fp8_gemm_torch_matches_c(coracle, mnk):
    a, a_s, b, b_s = _rand_problem(*mnk, seed=mnk[0])
    ref = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    c32, _ = c_fp8_gemm(coracle, a, a_s, b, b_s)
    rms = c32.pow(2).mean().sqrt()
    # both are binary32 evaluations of the same formula; only the order inside each 128-dot differs
    assert (ref - c32).abs().max() <= 2e-6 * rms


def test_fp8_gemm_brute_force_tiny():
    a, a_s, b, b_s = _rand_problem(3, 130, 256, seed=9)
    ref = oracle.fp8_gemm_f32(a, a_s, b, b_s).double()
    af, bf = a.double(), b.double()
    for i in range(3):
        for j in (0, 1, 64, 127, 128, 129):
            acc = 0.0
            for kb in range(2):
                dot = sum(af[i, kb * 128 + t].item() * bf[j, kb * 128 + t].item() for t in range(128))
                acc += dot * a_s[i, kb].item() * b_s[j // 128, kb].item()
            assert abs(ref[i, j].item() - acc) <= 1e-5 * max(1.0, abs(acc))


def test_fp8_gemm_exact_cases(coracle):
    """Small-integer operands and power-of-two scales: all sums are exact in binary32,
    so torch, C and the closed form agree bit for bit."""
    g = torch.Generator().manual_seed(4)
    m, n, k = 5, 140, 384
    a = torch.randint(-4, 5, (m, k), generator=g).float().to(FP8)
    b = torch.randint(-4, 5, (n, k), generator=g).float().to(FP8)
    ones_a, ones_b = torch.ones(m, 3), torch.ones(2, 3)
    ref = oracle.fp8_gemm_f32(a, ones_a, b, ones_b)
    assert torch.equal(ref, a.float() @ b.float().t())               # scales == 1: a plain matmul
    a_s = torch.pow(2.0, torch.randint(-3, 4, (m, 3), generator=g).float())
    b_s = torch.pow(2.0, torch.randint(-3, 4, (2, 3), generator=g).float())
    ref = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    want = torch.zeros(m, n)
    for kb in range(3):
        sl = slice(kb * 128, kb * 128 + 128)
        want += (a.float()[:, sl] @ b.float()[:, sl].t()) * a_s[:, kb, None] * b_s[torch.arange(n) // 128, kb][None]
    assert torch.equal(ref, want)
    c32, c16 = c_fp8_gemm(coracle, a, a_s, b, b_s)
    assert torch.equal(c32, ref)
    assert torch.equal(c16.view(torch.int16), ref.to(torch.bfloat16).view(torch.int16))


def test_fp8_gemm_ragged_n_is_a_prefix():
    a, a_s, b, b_s = _rand_problem(4, 640, 256, seed=5)
    full = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    part = oracle.fp8_gemm_f32(a, a_s, b[:576].contiguous(), b_s)      # 5 scale rows either way
    assert torch.equal(full[:, :576], part)


def _ragged_k_problem(m, n, k, seed):
    """fp8 operands with a K that is not a multiple of 128 and scale tensors of ceil(k / 128) columns (act_quant cannot
    produce such a pair, kernel.py:52; fp8_gemm's own kernel masks the tail, kernel.py:145, 158-159)."""
    g = torch.Generator().manual_seed(seed)
    kb = -(-k // 128)
    a = torch.randn(m, k, generator=g).to(FP8)
    b = (torch.randn(n, k, generator=g) * 0.5).to(FP8)
    a_s = torch.rand(m, kb, generator=g) * 0.1 + 0.01
    b_s = torch.rand(-(-n // 128), kb, generator=g) * 0.1 + 0.01
    return a, a_s, b, b_s


@pytest.mark.parametrize("mnk", [(3, 5, 1), (2, 130, 127), (4, 7, 129), (3, 200, 300), (1, 16, 7168 + 64)])
def test_fp8_gemm_masked_k_tail_equals_zero_padding(coracle, mnk):
    """A masked tail is a zero-filled tail: the result must equal, bit for bit, that of the operands padded with zero
    bytes to the next multiple of 128 (same scales) -- in the torch restatement and in the C one."""
    m, n, k = mnk
    a, a_s, b, b_s = _ragged_k_problem(m, n, k, seed=k)
    kp = -(-k // 128) * 128
    ap = torch.zeros(m, kp, dtype=torch.uint8); ap[:, :k] = a.view(torch.uint8)
    bp = torch.zeros(n, kp, dtype=torch.uint8); bp[:, :k] = b.view(torch.uint8)
    got = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    assert torch.equal(got, oracle.fp8_gemm_f32(ap.view(FP8), a_s, bp.view(FP8), b_s))
    c32, _ = c_fp8_gemm(coracle, a, a_s, b, b_s)
    c32p, _ = c_fp8_gemm(coracle, ap.view(FP8), a_s, bp.view(FP8), b_s)
    assert torch.equal(c32, c32p)
    rms = c32.pow(2).mean().sqrt()
    assert (got - c32).abs().max() <= 2e-6 * rms + 1e-30


def test_fp8_gemm_masked_k_tail_brute_force():
    a, a_s, b, b_s = _ragged_k_problem(2, 3, 200, seed=2)
    ref = oracle.fp8_gemm_f32(a, a_s, b, b_s).double()
    af, bf = a.double(), b.double()
    for i in range(2):
        for j in range(3):
            acc = sum(af[i, t].item() * bf[j, t].item() for t in range(128)) * a_s[i, 0].item() * b_s[0, 0].item()
            acc += sum(af[i, t].item() * bf[j, t].item() for t in range(128, 200)) * a_s[i, 1].item() * b_s[0, 1].item()
            assert abs(ref[i, j].item() - acc) <= 1e-5 * max(1.0, abs(acc))


def test_fp8_gemm_close_to_unquantised_product():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(8, 1024, generator=g).bfloat16()
    w = (torch.randn(256, 1024, generator=g) * 0.02).bfloat16()
    a, a_s = oracle.act_quant(x)
    b, b_s = oracle.block_quant_weight(w)
    c = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    exact = x.float() @ w.float().t()
    # also equals x_q @ dequant(w)^T up to binary32 rounding
    deq = (a.float().view(8, 8, 128) * a_s[..., None]).view(8, 1024) @ oracle.weight_dequant(b, b_s, out_dtype=torch.float32).t()
    assert (c - deq).abs().max() <= 1e-5 * exact.abs().max()
    assert (c - exact).abs().max() <= 0.08 * exact.pow(2).mean().sqrt() * 4


def test_cfg1_cpu_plumbing():
    """The CPU-plumbing configuration: x [16,7168], wq_a-shaped weight [1536,7168], seed 0."""
    from dsv3fp8 import workloads
    x, w8, ws = workloads.cfg1_cpu_plumbing()
    assert ws.shape == (12, 56)
    y = oracle.linear(x, w8, scale=ws)
    assert y.shape == (16, 1536) and y.dtype == torch.bfloat16
    exact = x.float() @ oracle.weight_dequant(w8, ws, out_dtype=torch.float32).t()
    assert (y.float() - exact).abs().max() <= 0.05 * exact.pow(2).mean().sqrt() * 4


# ---------------------------------------------------------------- gate / moe (config 5 callers)

def test_gate_invariants():
    g = torch.Generator().manual_seed(7)
    t, e, dim = 64, 256, 64
    x = torch.randn(t, dim, generator=g).bfloat16()
    gw = torch.randn(e, dim, generator=g).bfloat16()
    bias = torch.randn(e, generator=g) * 0.1
    w, idx = oracle.gate(x, gw, bias, topk=8, n_groups=8, topk_groups=4, route_scale=2.5)
    assert w.shape == (t, 8) and idx.shape == (t, 8) and w.dtype == torch.bfloat16
    assert all(len(set(r.tolist())) == 8 for r in idx)                       # 8 distinct experts
    assert all(len(set((r // 32).tolist())) <= 4 for r in idx)               # inside at most 4 groups
    assert torch.allclose(w.float().sum(-1), torch.full((t,), 2.5), atol=0.03)
    # the bias moves the selection but the weights are the unbiased sigmoid scores
    scores = torch.nn.functional.linear(x, gw).sigmoid()
    picked = scores.gather(1, idx).float()
    want = (picked / picked.sum(-1, keepdim=True) * 2.5).bfloat16()
    assert torch.allclose(w.float(), want.float(), atol=0.02)


def test_gate_route_known_answer():
    """oracle.gate_route on logits whose routing is known in closed form (model.py:577-598).  A group's score is
    the SUM OF ITS TWO largest biased scores (:589): group 0 holds the largest single value but a small pair, so a
    top-1 group score would pick {0, 3} and the expected experts would not come out; the bias moves the selection
    (:581) but the weights are the unbiased scores (:594), normalised (:596) and scaled (:597)."""
    experts, groups = 16, 4
    logits = torch.full((1, experts), -4.0)
    logits[0, 4], logits[0, 5] = 2.0, 1.0            # group 1
    logits[0, 12], logits[0, 13] = 3.0, -1.0         # group 3
    logits[0, 0] = 3.5                                # group 0: the largest value of all, nothing beside it
    bias = torch.zeros(experts); bias[5] = 0.5; bias[13] = 0.5
    sg = lambda v: float(torch.tensor(v).sigmoid())
    pair = {0: sg(3.5) + sg(-4.0), 1: sg(2.0) + sg(1.0) + 0.5, 2: 2 * sg(-4.0), 3: sg(3.0) + sg(-1.0) + 0.5}
    top1 = {0: sg(3.5), 1: sg(1.0) + 0.5, 2: sg(-4.0), 3: sg(3.0)}
    assert set(sorted(pair, key=pair.get)[-2:]) == {1, 3} and set(sorted(top1, key=top1.get)[-2:]) == {0, 1}   # the two rules differ
    w, idx = oracle.gate_route(logits.bfloat16(), bias, 3, groups, 2, 1.0, "sigmoid")
    # biased scores inside groups 1 and 3: 5 -> 1.231, 12 -> 0.953, 4 -> 0.881, 13 -> 0.769
    assert idx.tolist() == [[5, 12, 4]]
    s = torch.tensor([1.0, 3.0, 2.0]).bfloat16().sigmoid()
    assert torch.equal(w[0], (s / s.sum(-1, keepdim=True)) * 1.0)
    w25, _ = oracle.gate_route(logits.bfloat16(), bias, 3, groups, 2, 2.5, "sigmoid")
    assert torch.equal(w25[0], (s / s.sum(-1, keepdim=True)) * 2.5)


def test_moe_equals_dense_masked_brute_force():
    g = torch.Generator().manual_seed(8)
    t, e, dim, inter = 12, 4, 128, 128
    x = torch.randn(t, dim, generator=g).bfloat16()

    def expert():
        out = []
        for shape in ((inter, dim), (dim, inter), (inter, dim)):
            out += list(oracle.block_quant_weight((torch.randn(*shape, generator=g) * 0.05).bfloat16()))
        return tuple(out)
    experts = [expert() for _ in range(e)]
    shared = expert()
    idx = torch.stack([torch.randperm(e, generator=g)[:2] for _ in range(t)])
    w = torch.rand(t, 2, generator=g).bfloat16()
    y = oracle.moe(x, w, idx, experts, shared)
    dense = torch.zeros(t, dim)
    for i in range(e):
        out = oracle.mlp(x, *experts[i]).float()
        for tok in range(t):
            for slot in range(2):
                if idx[tok, slot] == i:
                    dense[tok] += (out[tok] * w[tok, slot].float())
    dense += oracle.mlp(x, *shared).float()
    assert torch.allclose(y.float(), dense, atol=0.05, rtol=0.05)
