"""GPU parity: weight_dequant through the C ABI vs the torch-CPU oracle, bit for bit
(reference arithmetic: inference/kernel.py:76-86)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    return dsv3fp8


def _bits(t):
    return t.view(torch.int16) if t.element_size() == 2 else t.view(torch.int32)


def _check(K, w8, s, block=128, dtype=torch.bfloat16):
    ref = oracle.weight_dequant(w8, s, block, out_dtype=dtype)
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        y = K.weight_dequant(w8.cuda(), s.cuda(), block)
    finally:
        torch.set_default_dtype(old)
    assert y.dtype == dtype and y.shape == ref.shape
    yc = y.cpu()
    nan_ref = ref.float().isnan()
    assert torch.equal(yc.float().isnan(), nan_ref)
    assert torch.equal(_bits(yc)[~nan_ref], _bits(ref)[~nan_ref])


@pytest.mark.parametrize("shape", [(256, 512), (1536, 7168), (576, 7168), (130, 272), (1, 16), (128, 7168 + 16)])
def test_random_vector_path(K, shape):
    from dsv3fp8 import workloads
    w8, s = workloads.random_fp8_weight(*shape, seed=shape[0])
    _check(K, w8, s)


@pytest.mark.parametrize("shape", [(100, 100), (129, 130), (3, 7), (257, 1000)])
def test_ragged_scalar_path(K, shape):
    from dsv3fp8 import workloads
    w8, s = workloads.random_fp8_weight(*shape, seed=shape[1])
    _check(K, w8, s)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_other_output_dtypes(K, dtype):
    from dsv3fp8 import workloads
    w8, s = workloads.random_fp8_weight(384, 640, seed=9)
    s = s * 100   # keep fp16 away from total underflow
    _check(K, w8, s, dtype=dtype)


@pytest.mark.parametrize("block", [64, 32, 100])
def test_other_block_sizes(K, block):
    g = torch.Generator().manual_seed(block)
    w8 = torch.randint(0, 0x7F, (200, 300), generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
    s = torch.rand(-(-200 // block), -(-300 // block), generator=g) + 0.5
    _check(K, w8, s, block)


def test_all_byte_values_scale_one(K):
    """s == 1: the output is the table of the 256 e4m3fn values (0x7f / 0xff are NaN)."""
    w8 = torch.arange(256, dtype=torch.int16).to(torch.uint8).repeat(128, 1).view(torch.float8_e4m3fn)  # [128,256]
    s = torch.ones(1, 2)
    _check(K, w8, s)
    y = oracle.weight_dequant(w8, s).float()     # the table itself, against the OCP E4M3 definition
    assert y[0, 0x7E].item() == 448.0 and y[0, 0x38].item() == 1.0 and y[0, 0x01].item() == 2.0 ** -9
    assert y[0, 0x7F].isnan() and y[0, 0xFF].isnan() and y[0, 0xFE].item() == -448.0


def test_tiny_scales_reach_subnormals(K):
    from dsv3fp8 import workloads
    w8, _ = workloads.random_fp8_weight(128, 256, seed=4)
    s = torch.tensor([[1e-38, 3e-41]])
    _check(K, w8, s)
    _check(K, w8, s, dtype=torch.float32)


def test_asserts_match_reference(K):
    w8 = torch.zeros(128, 128, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    s = torch.ones(1, 1, device="cuda")
    with pytest.raises(AssertionError):
        K.weight_dequant(w8.t(), s)
    with pytest.raises(AssertionError):
        K.weight_dequant(w8.view(2, 64, 128), s)


def test_full_size_sampled(K):
    """[18432,7168] fp8 -> bf16: compare sampled row blocks with the oracle."""
    from dsv3fp8 import workloads
    w8, s = workloads.random_fp8_weight(18432, 7168, seed=2, device="cuda")
    torch.set_default_dtype(torch.bfloat16)      # the reference's callers set this (generate.py:109)
    try:
        y = K.weight_dequant(w8, s)
        y2 = K.weight_dequant(w8, s * 2)
    finally:
        torch.set_default_dtype(torch.float32)
    assert y.dtype == torch.bfloat16
    for r0 in (0, 128 * 71 + 5, 18432 - 64):
        ref = oracle.weight_dequant(w8[r0 - r0 % 128: r0 - r0 % 128 + 128].cpu(), s[r0 // 128: r0 // 128 + 1].cpu())
        got = y[r0 - r0 % 128: r0 - r0 % 128 + 128].cpu()
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    # linearity in the scale: doubling s doubles y exactly
    assert torch.equal(y2.float(), y.float() * 2)
