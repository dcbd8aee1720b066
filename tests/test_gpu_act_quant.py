"""GPU parity: act_quant through the C ABI vs the torch-CPU oracle, bit for bit
(reference arithmetic: inference/kernel.py:23-35)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    return dsv3fp8


def _check(K, x_cpu, block=128, fmt=None):
    y_ref, s_ref = oracle.act_quant(x_cpu, block, fmt)
    y, s = K.act_quant(x_cpu.cuda(), block, fmt)
    torch.cuda.synchronize()
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert y.shape == y_ref.shape and s.shape == s_ref.shape
    assert torch.equal(s.cpu().view(torch.int32), s_ref.view(torch.int32)), "scales differ"
    yb, rb = y.cpu().view(torch.uint8), y_ref.view(torch.uint8)
    bad = (yb != rb).nonzero()
    assert bad.numel() == 0, f"{bad.shape[0]} fp8 bytes differ, first at {bad[0].tolist()}"


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_random_with_outliers(K, fmt):
    from dsv3fp8 import workloads
    x = workloads.activations(512, 7168, seed=3, outliers=True)
    _check(K, x, 128, fmt)


@pytest.mark.parametrize("m", [1, 8, 32, 64])
def test_decode_rows(K, m):
    from dsv3fp8 import workloads
    _check(K, workloads.activations(m, 7168, seed=10 + m))
    _check(K, workloads.activations(m, 512, seed=20 + m))


def test_leading_dims_and_small(K):
    torch.manual_seed(5)
    _check(K, torch.randn(2, 3, 256).bfloat16())
    _check(K, torch.randn(128).bfloat16())
    _check(K, torch.randn(7, 128).bfloat16())


def test_all_bf16_bit_patterns(K):
    """Every finite bf16 value appears as an element, in blocks whose amax is itself
    swept over many magnitudes: 256 columns of 128-blocks x all 65280 finite patterns."""
    bits = torch.arange(0, 65536, dtype=torch.int32)
    finite = bits[(bits & 0x7F80) != 0x7F80]
    vals = finite.to(torch.int16).view(torch.bfloat16)            # [65280]
    g = torch.Generator().manual_seed(7)
    # rows of 128: a random permutation of all values, 510 rows; then rescale rows by powers of two
    perm = vals[torch.randperm(vals.numel(), generator=g)].view(-1, 128)
    _check(K, perm.contiguous())
    _check(K, perm.contiguous(), fmt="ue8m0")
    # sorted values: neighbouring magnitudes share a block, so most elements are near the amax
    srt = vals[vals.float().abs().argsort()].view(-1, 128)
    _check(K, srt.contiguous())
    _check(K, srt.contiguous(), fmt="ue8m0")


def test_adversarial_blocks(K):
    rows = []
    rows.append(torch.zeros(128))                                  # all zero -> s = 1e-4/448, y = +0
    rows.append(torch.full((128,), -0.0))                           # -0 keeps its sign (0x80)
    rows.append(torch.full((128,), 5e-5))                           # below the 1e-4 clamp
    rows.append(torch.full((128,), 3.0))                            # constant -> every byte 0x7e
    r = torch.zeros(128); r[17] = -1000.0; rows.append(r)           # single outlier
    r = torch.linspace(-448, 448, 128); rows.append(r)
    r = torch.arange(128, dtype=torch.float32) * (448.0 / 127); rows.append(r)
    # exact ties of the e4m3 grid: amax = 448 -> s = 1 and elements on half-way points
    r = torch.tensor([17., 19., 21., 23., 25., 27., 29., 31., 2 ** -10, 3 * 2 ** -10, 2 ** -9 * 1.5, 2 ** -7 * 1.0625] * 10 + [448.] * 8)
    rows.append(r)
    r = -r.clone(); rows.append(r)
    # subnormal bf16 inputs and a huge block
    r = torch.full((128,), 1e-39); r[0] = 1e-38; rows.append(r)
    r = torch.full((128,), 1e38); r[5] = 3e38; r[6] = -1e30; rows.append(r)
    x = torch.stack(rows).bfloat16()
    _check(K, x)
    _check(K, x, fmt="ue8m0")


@pytest.mark.parametrize("block", [32, 64, 256, 512])
def test_other_block_sizes(K, block):
    torch.manual_seed(block)
    x = (torch.randn(33, 1024) * torch.rand(33, 1) * 10).bfloat16()
    _check(K, x, block)


@pytest.mark.parametrize("block", [1, 2, 8, 16, 24, 100, 1024, 2048, 4096])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_any_block_size_that_divides_the_last_dimension(K, block, dtype):
    """The reference's wrapper takes every block size that divides the last dimension (inference/kernel.py:38,52);
    sizes other than 32 ... 512 run one wavefront per block."""
    torch.manual_seed(block)
    cols = block * (3 if block >= 1024 else 5)
    x = (torch.randn(9, cols) * torch.rand(9, 1) * 10).to(dtype)
    x[0, :block] = 0
    x[1, 0] = 3e4
    _check(K, x, block)
    _check(K, x, block, "ue8m0")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_other_input_dtypes(K, dtype):
    torch.manual_seed(11)
    x = (torch.randn(65, 1024) * 3).to(dtype)
    _check(K, x)
    _check(K, x, fmt="ue8m0")


def test_known_answers(K):
    y, s = K.act_quant(torch.zeros(1, 128, dtype=torch.bfloat16, device="cuda"))
    assert s.item() == pytest.approx(2.2321428616578487e-07, rel=0, abs=0)
    assert int(y.view(torch.uint8).max()) == 0
    x = torch.randn(4, 128).bfloat16()
    y1, s1 = K.act_quant(x.cuda())
    y2, s2 = K.act_quant((x.float() * 8).bfloat16().cuda())
    assert torch.equal(y1.view(torch.uint8), y2.view(torch.uint8))
    assert torch.equal(s1 * 8, s2)


def test_asserts_match_reference(K):
    with pytest.raises(AssertionError):
        K.act_quant(torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda").t())
    with pytest.raises(AssertionError):
        K.act_quant(torch.zeros(4, 100, dtype=torch.bfloat16, device="cuda"))


def test_full_size_properties(K):
    """[4096,7168] with outliers: compare a strided sample of rows with the oracle and check
    size-independent properties on the whole output (|y| <= 448, every block holds a +-448)."""
    from dsv3fp8 import workloads
    x = workloads.activations(4096, 7168, seed=0, device="cuda", outliers=True)
    y, s = K.act_quant(x)
    rows = torch.arange(0, 4096, 37)
    y_ref, s_ref = oracle.act_quant(x[rows.cuda()].cpu())
    assert torch.equal(y[rows.cuda()].cpu().view(torch.uint8), y_ref.view(torch.uint8))
    assert torch.equal(s[rows.cuda()].cpu(), s_ref)
    mag = (y.view(torch.uint8) & 0x7F).view(4096, 56, 128)
    assert int(mag.max()) == 0x7E
    assert bool((mag.amax(-1) == 0x7E).all())


def _non_finite_rows():
    g = torch.Generator().manual_seed(12)
    x = torch.randn(6, 512, generator=g).bfloat16()
    x[0, 5] = float("nan")                      # block (0, 0)
    x[1, 130] = float("inf")                    # block (1, 1)
    x[2, 300] = float("-inf"); x[2, 301] = 7.0  # block (2, 2)
    x[3, 10] = float("nan"); x[3, 11] = float("inf")   # NaN wins over infinity
    x[4, 384:512] = 0                           # an all-zero block beside normal ones
    return x


def _same_up_to_nan_sign(y, s, yr, sr):
    """Scales: NaN where the oracle has NaN, inf where it has inf, equal elsewhere; bytes: NaN codes where the oracle
    has NaN codes (0x7f and 0xff differ only in the sign of the NaN), equal elsewhere.  Returns the NaN-code mask."""
    y, yr = y.cpu().view(torch.uint8), yr.view(torch.uint8)
    s = s.cpu()
    assert torch.equal(torch.isnan(s), torch.isnan(sr)) and torch.equal(torch.isinf(s), torch.isinf(sr))
    ok = torch.isfinite(sr)
    assert torch.equal(s[ok], sr[ok])
    nan_ref, nan_got = (yr & 0x7F) == 0x7F, (y & 0x7F) == 0x7F
    assert torch.equal(nan_ref, nan_got)
    assert torch.equal(y[~nan_ref], yr[~nan_ref])
    return nan_got


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("block", [128, 16])
def test_non_finite_inputs_every_variant(K, fmt, dtype, block):
    """Both scale formats (the power-of-two rounding must leave s = NaN / inf alone), the reciprocal and the IEEE
    division paths, the vectorised and the one-wavefront-per-block kernels."""
    x = _non_finite_rows().to(dtype)
    yr, sr = oracle.act_quant(x, block, fmt)
    y, s = K.act_quant(x.cuda(), block, fmt)
    nan_got = _same_up_to_nan_sign(y, s, yr, sr)
    assert bool(torch.isnan(s[0, 0])) and bool(nan_got[0, :block].all())
    assert bool(torch.isinf(s[1, 130 // block])) and s[1, 130 // block] > 0


def test_non_finite_inputs_follow_the_ieee_evaluation(K):
    """NaN and infinity in the activations (inference/kernel.py:26-33 evaluated with torch's CPU operators, whose amax
    propagates NaN): a block with a NaN gets s = NaN and NaN codes everywhere, a block with an infinity s = inf, zeros
    for the finite elements and NaN codes for the infinite ones; blocks beside them are untouched.  Held against
    oracle.act_quant (NaN codes are compared as "is a NaN code": 0x7f and 0xff differ only in the sign of the NaN)."""
    x = _non_finite_rows()
    yr, sr = oracle.act_quant(x)
    y, s = K.act_quant(x.cuda())
    y, s = y.cpu().view(torch.uint8), s.cpu()
    yr = yr.view(torch.uint8)
    assert torch.equal(torch.isnan(s), torch.isnan(sr)) and torch.equal(torch.isinf(s), torch.isinf(sr))
    ok = torch.isfinite(sr)
    assert torch.equal(s[ok], sr[ok])
    nan_ref, nan_got = (yr & 0x7F) == 0x7F, (y & 0x7F) == 0x7F
    assert torch.equal(nan_ref, nan_got)
    assert torch.equal(y[~nan_ref], yr[~nan_ref])
    assert bool(nan_got[0, :128].all()) and not bool(nan_got[0, 128:].any())
    assert bool(torch.isinf(s[1, 1])) and int(nan_got[1].sum()) == 1 and bool(nan_got[1, 130])
    assert int(((y[1, 128:256] & 0x7F) != 0).sum()) == 1                # finite / inf = a zero of either sign
    assert bool(torch.isnan(s[3, 0])) and bool(nan_got[3, :128].all())
