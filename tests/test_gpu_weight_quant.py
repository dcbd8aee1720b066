"""GPU parity: the weight block-quantiser through the C ABI vs the torch-CPU oracle, bit for bit (bytes and scales).
Format: README_WEIGHTS.md:60-92 (128 x 128 blocks, ragged blocks zero-padded before the scale is taken); the rule is
the activation quantiser's (inference/kernel.py:23-35) on a square block."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    return dsv3fp8


def _check(K, w, fmt=None):
    ref8, refs = oracle.block_quant_weight(w, scale_fmt=fmt)
    q8, qs = K.weight_quant(w.cuda(), scale_fmt=fmt)
    assert q8.dtype == FP8 and qs.dtype == torch.float32
    assert q8.shape == ref8.shape and qs.shape == refs.shape
    assert torch.equal(qs.cpu(), refs)
    assert torch.equal(q8.cpu().view(torch.uint8), ref8.view(torch.uint8))
    return q8, qs


@pytest.mark.parametrize("shape", [(256, 512), (1536, 7168), (576, 7168), (130, 272), (1, 8), (128, 7168 + 16),
                                   (300, 520), (127, 129 * 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_random_vector_path(K, shape, dtype):
    g = torch.Generator().manual_seed(shape[0] + shape[1])
    w = (torch.randn(*shape, generator=g) * 0.02).to(dtype)
    _check(K, w)


@pytest.mark.parametrize("shape", [(200, 301), (5, 7), (129, 1), (64, 1027)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_row_lengths_that_are_not_multiples_of_8(K, shape, dtype):
    g = torch.Generator().manual_seed(shape[1])
    w = (torch.randn(*shape, generator=g) * 0.5).to(dtype)
    _check(K, w)


def test_magnitudes_signed_zeros_and_the_clamp(K):
    g = torch.Generator().manual_seed(5)
    # blocks whose amax spans 60 decades of binary32-representable bf16 magnitudes, one all-zero block, signed zeros
    w = torch.randn(256, 1024, generator=g)
    expo = torch.linspace(-30, 30, 8).repeat_interleave(128)[None, :]
    w = (w * torch.pow(10.0, expo)).bfloat16()
    w[:128, 128:256] = 0
    w[5, 130] = -0.0
    w[128:, 0] = -0.0
    w[200, 700] = 3.0e38
    w[130, 900] = -3.3e38
    q8, qs = _check(K, w)
    assert qs[0, 1].item() == pytest.approx(1e-4 / 448, rel=1e-7)
    assert q8.cpu().view(torch.uint8)[5, 130] == 0x80                      # -0 stays -0


def test_every_bf16_value_as_an_element(K):
    """All finite bf16 bit patterns: block b holds one sign and 16 consecutive exponents (all 128 mantissas each), a
    range the e4m3 codes of one scale can resolve, so every quotient the correction sequence for bf16 inputs can
    meet at that block's scale occurs."""
    blocks = []
    for sign in (0, 0x8000):
        for e0 in range(0, 255, 16):
            exps = torch.arange(e0, min(e0 + 16, 255))
            pats = (sign | (exps[:, None] << 7) | torch.arange(128)[None, :]).flatten()
            blocks.append(pats.repeat(-(-16384 // pats.numel()))[:16384].view(128, 128))
    bits = torch.cat(blocks, 1)
    w = ((bits + 0x8000) % 0x10000 - 0x8000).to(torch.int16).view(torch.bfloat16).contiguous()
    assert w.shape == (128, 32 * 128) and bool(w.float().isfinite().all())
    _check(K, w)
    _check(K, w.t().contiguous())


def test_known_answers_on_device(K):
    g = torch.Generator().manual_seed(11)
    m, n = 300, 520
    b = torch.randint(0, 256, (m, n), generator=g, dtype=torch.int16)
    b = torch.where((b & 0x7F) == 0x7F, b & 0x80, b).to(torch.uint8)
    for i in range(3):
        for j in range(5):
            b[min(i * 128 + 7 * j + 3, m - 1), min(j * 128 + 5 * i + 2, n - 1)] = 0x7E if (i + j) % 2 else 0xFE
    s = torch.pow(2.0, torch.randint(-12, 3, (3, 5), generator=g).float())
    w = oracle.weight_dequant(b.view(FP8), s, out_dtype=torch.float32)
    for src in (w, w.bfloat16()):
        q8, qs = K.weight_quant(src.cuda())
        assert torch.equal(qs.cpu(), s)
        assert torch.equal(q8.cpu().float(), b.view(FP8).float())


def test_full_size_round_trip(K):
    """[18432, 7168] on the device: every block reaches the largest code, weight_dequant brings the weights back to
    within half an e4m3 step, and sampled row bands equal the oracle's bytes and scales."""
    g = torch.Generator(device="cuda").manual_seed(1)
    w = (torch.randn(18432, 7168, generator=g, device="cuda") * 0.02).bfloat16()
    q8, qs = K.weight_quant(w)
    assert q8.shape == (18432, 7168) and qs.shape == (144, 56)
    assert bool((q8.float().abs().view(144, 128, 56, 128).amax(dim=(1, 3)) == 448).all())
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float32)
    try:
        back = K.weight_dequant(q8, qs)
    finally:
        torch.set_default_dtype(old)
    es = qs.repeat_interleave(128, 0).repeat_interleave(128, 1)
    err = (back - w.float()).abs()
    assert bool((err <= torch.maximum(w.float().abs() * 2.0 ** -4, es * 2.0 ** -10) * (1 + 1e-6)).all())
    for r0 in (0, 9088, 18304):                                 # three 128-row bands against the CPU oracle
        ref8, refs = oracle.block_quant_weight(w[r0:r0 + 128].cpu())
        assert torch.equal(qs[r0 // 128].cpu(), refs[0])
        assert torch.equal(q8[r0:r0 + 128].cpu().view(torch.uint8), ref8.view(torch.uint8))


@pytest.mark.parametrize("shape,dtype", [((256, 512), torch.bfloat16), ((300, 520), torch.bfloat16),
                                         ((200, 301), torch.float32), ((130, 272), torch.float16)])
def test_power_of_two_scales(K, shape, dtype):
    """scale_fmt "ue8m0": the scales are rounded up to powers of two before the division (kernel.py:29-31 applied to
    the block scale); bytes and scales equal the oracle's, and the result feeds fp8_gemm_pow2."""
    g = torch.Generator().manual_seed(shape[1])
    w = (torch.randn(*shape, generator=g) * 0.04).to(dtype)
    q8, qs = _check(K, w, "ue8m0")
    assert bool(((qs.view(torch.int32) & 0x7FFFFF) == 0).all())
    assert bool((q8.float().abs().amax() <= 448).item())
    # a power of two is kept: blocks whose amax / 448 is already 2^e
    w2 = torch.zeros(128, 256)
    w2[3, 5], w2[100, 200] = 448 * 2.0 ** -9, -448 * 2.0 ** -3
    w2[0, 0], w2[0, 130] = 2.0 ** -9, 2.0 ** -3
    p8, ps = _check(K, w2.to(dtype), "ue8m0")
    assert ps.flatten().tolist() == [2.0 ** -9, 2.0 ** -3]
    assert p8.cpu().float()[0, 0] == 1 and p8.cpu().float()[100, 200] == -448


def test_quantise_then_multiply_with_power_of_two_scales(K):
    """weight_quant(ue8m0) -> act_quant(ue8m0) -> fp8_gemm_pow2 on the device against the oracle's chain."""
    g = torch.Generator().manual_seed(9)
    w = (torch.randn(640, 1024, generator=g) * 0.03).bfloat16()
    x = torch.randn(300, 1024, generator=g).bfloat16()
    w8, ws = K.weight_quant(w.cuda(), scale_fmt="ue8m0")
    a, a_s = K.act_quant(x.cuda(), 128, "ue8m0")
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float32)
    try:
        c = K.fp8_gemm_pow2(a, a_s, w8, ws)
    finally:
        torch.set_default_dtype(old)
    r8, rs = oracle.block_quant_weight(w, scale_fmt="ue8m0")
    ra, ras = oracle.act_quant(x, 128, "ue8m0")
    ref = oracle.fp8_gemm_f32(ra, ras, r8, rs)
    assert (c.cpu() - ref).abs().max().item() <= 1e-2 * ref.pow(2).mean().sqrt().item()


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_non_finite_weights(K, fmt, dtype):
    """A NaN or an infinity in a 128 x 128 block reaches that block's scale (NaN / inf) as through act_quant; the other
    blocks are untouched.  Against the oracle: scales NaN / inf in the same places, bytes NaN codes in the same places."""
    g = torch.Generator().manual_seed(21)
    w = (torch.randn(256, 384, generator=g) * 0.02).to(dtype)
    w[3, 5] = float("nan")               # block (0, 0)
    w[130, 200] = float("inf")           # block (1, 1)
    w[200, 300] = float("-inf"); w[201, 301] = float("nan")     # block (1, 2): NaN wins
    ref8, refs = oracle.block_quant_weight(w, scale_fmt=fmt)
    q8, qs = K.weight_quant(w.cuda(), scale_fmt=fmt)
    qs, q8, ref8 = qs.cpu(), q8.cpu().view(torch.uint8), ref8.view(torch.uint8)
    assert bool(torch.isnan(refs[0, 0])) and bool(torch.isinf(refs[1, 1])) and bool(torch.isnan(refs[1, 2]))
    assert torch.equal(torch.isnan(qs), torch.isnan(refs)) and torch.equal(torch.isinf(qs), torch.isinf(refs))
    ok = torch.isfinite(refs)
    assert torch.equal(qs[ok], refs[ok])
    nan_a, nan_b = (q8 & 0x7F) == 0x7F, (ref8 & 0x7F) == 0x7F
    assert torch.equal(nan_a, nan_b) and torch.equal(q8[~nan_a], ref8[~nan_a])
