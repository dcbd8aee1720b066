"""GPU parity of the absorbed-attention products with the FP8 weight wkv_b (dsv3_wkv_b_absorb through
torch.ops.dsv3fp8.wkv_b_absorb) and of MLA.forward on top of them, against the torch-CPU oracle of
inference/model.py:456-497.

Tolerance of the products: the dequantised weights are bit-exact (checked with one-hot inputs), the sum is
accumulated in binary32 in a different order than the oracle's and rounded once to bf16, so
|y - r| <= 2^-8 |r| + 2^-20 * sum|x_i w_i| for the unrounded float64 result r."""
import pytest
import torch

from oracle import oracle
from test_oracle_mla import _freqs, _wkv_b, small_mla_params

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn
Q, V = 0, 1


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    from dsv3fp8 import ops  # noqa: F401  (registers torch.ops.dsv3fp8)
    return dsv3fp8


def _absorb(x, w8, s, side, nope, v):
    return torch.ops.dsv3fp8.wkv_b_absorb(x, w8, s, side, nope, v)


def _check(y, x, w8, s, side, nope, v):
    heads = x.size(-2)
    wd = oracle.weight_dequant(w8, s).double().view(heads, nope + v, -1)
    xd = x.double()
    if side == Q:
        r = torch.einsum("...hd,hdc->...hc", xd, wd[:, :nope])
        mag = torch.einsum("...hd,hdc->...hc", xd.abs(), wd[:, :nope].abs())
    else:
        r = torch.einsum("...hc,hdc->...hd", xd, wd[:, nope:])
        mag = torch.einsum("...hc,hdc->...hd", xd.abs(), wd[:, nope:].abs())
    err = (y.double().cpu() - r).abs()
    bound = 2.0 ** -8 * r.abs() + 2.0 ** -20 * mag + 1e-30
    assert (err <= bound).all(), (err / bound).max()


@pytest.mark.parametrize("tokens", [1, 5, 16, 17, 33, 64, 100, 128, 200, 256, 333])
@pytest.mark.parametrize("side", [Q, V])
def test_absorb_671b_shape(K, tokens, side):
    heads, nope, v, c = 128, 128, 128, 512
    w8, s = _wkv_b(heads, nope, v, c, 10)
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn(tokens, heads, nope if side == Q else c, generator=g).bfloat16()
    y = _absorb(x.cuda(), w8.cuda(), s.cuda(), side, nope, v)
    assert y.shape == (tokens, heads, c if side == Q else v) and y.dtype == torch.bfloat16
    _check(y, x, w8, s, side, nope, v)


@pytest.mark.parametrize("heads,nope,v,c", [(3, 64, 32, 128), (5, 64, 64, 256), (2, 128, 32, 512), (1, 128, 96, 384),
                                             (3, 64, 128, 512)])
def test_absorb_other_shapes(K, heads, nope, v, c):
    """Heads whose row ranges straddle 128-row scale blocks (nope + v not a multiple of 128)."""
    w8, s = _wkv_b(heads, nope, v, c, 11)
    s = s * torch.linspace(0.5, 2.0, s.numel()).view_as(s)      # make every scale block distinct
    g = torch.Generator().manual_seed(12)
    for tokens in (7, 90):
        xq = torch.randn(tokens, heads, nope, generator=g).bfloat16()
        _check(_absorb(xq.cuda(), w8.cuda(), s.cuda(), Q, nope, v), xq, w8, s, Q, nope, v)
        if c in (128, 256, 512):
            xv = torch.randn(tokens, heads, c, generator=g).bfloat16()
            _check(_absorb(xv.cuda(), w8.cuda(), s.cuda(), V, nope, v), xv, w8, s, V, nope, v)


def test_absorb_dequantises_bit_exactly(K):
    """One-hot activations return single dequantised weights: they must equal weight_dequant's bf16 values
    exactly (same multiply, same rounding) for every e4m3 encoding; a NaN encoding poisons exactly the sums it
    takes part in."""
    heads, nope, v, c = 4, 128, 128, 512
    g = torch.Generator().manual_seed(13)
    w8 = torch.randint(0, 256, (heads * (nope + v), c), generator=g, dtype=torch.uint8)
    w8[(w8 & 0x7F) == 0x7F] = 0x7E                                           # no NaN encodings here
    w8 = w8.view(FP8)
    s = torch.rand(heads * (nope + v) // 128, c // 128, generator=g) * 1e-2 + 1e-4
    wd = oracle.weight_dequant(w8, s).view(heads, nope + v, c).float()
    eye = torch.eye(nope, dtype=torch.bfloat16).unsqueeze(1).expand(nope, heads, nope).contiguous()
    y = _absorb(eye.cuda(), w8.cuda(), s.cuda(), Q, nope, v).cpu()          # y[d, h, :] = W[h, d, :]
    assert torch.equal(y.float(), wd[:, :nope, :].permute(1, 0, 2))
    eye = torch.eye(c, dtype=torch.bfloat16).unsqueeze(1).expand(c, heads, c).contiguous()
    y = _absorb(eye.cuda(), w8.cuda(), s.cuda(), V, nope, v).cpu()          # y[c, h, d] = W[h, nope + d, c]
    assert torch.equal(y.float(), wd[:, nope:, :].permute(2, 0, 1))
    for lo, hi in ((200, 328), (0, 40)):            # 128 and 40 tokens: the kernel that splits K over its wavefronts
        y = _absorb(eye[lo:hi].contiguous().cuda(), w8.cuda(), s.cuda(), V, nope, v).cpu()
        assert torch.equal(y.float(), wd[:, nope:, lo:hi].permute(2, 0, 1))

    wn = w8.view(torch.uint8).clone().view(heads, nope + v, c)
    wn[1, 5, 7] = 0x7F
    wn[2, nope + 9, 300] = 0xFF
    wn = wn.view(-1, c).view(FP8)
    x = torch.ones(3, heads, nope, dtype=torch.bfloat16)
    nan = torch.isnan(_absorb(x.cuda(), wn.cuda(), s.cuda(), Q, nope, v).float().cpu())
    exp = torch.zeros(3, heads, c, dtype=torch.bool); exp[:, 1, 7] = True
    assert torch.equal(nan, exp)
    x = torch.ones(3, heads, c, dtype=torch.bfloat16)
    nan = torch.isnan(_absorb(x.cuda(), wn.cuda(), s.cuda(), V, nope, v).float().cpu())
    exp = torch.zeros(3, heads, v, dtype=torch.bool); exp[:, 2, 9] = True
    assert torch.equal(nan, exp)


def test_absorb_exact_integer_case(K):
    heads, nope, v, c = 8, 128, 128, 512
    g = torch.Generator().manual_seed(14)
    wi = torch.randint(-3, 4, (heads * (nope + v), c), generator=g)
    w8, s = wi.float().to(FP8), torch.ones(heads * 2, c // 128)
    xq = torch.randint(-2, 3, (40, heads, nope), generator=g).bfloat16()
    xv = torch.randint(-1, 2, (40, heads, c), generator=g).bfloat16()
    for x, side in ((xq, Q), (xv, V)):
        ref = oracle.wkv_b_absorb_f32(x, w8, s, "q" if side == Q else "v", nope, v)
        assert ref.abs().max() <= 256                                        # integers of this size are exact in bf16
        assert torch.equal(_absorb(x.cuda(), w8.cuda(), s.cuda(), side, nope, v).float().cpu(), ref)


def test_absorb_takes_the_q_nope_view(K):
    """q_nope is a slice of q [b, s, h, nope + rope]: strided tokens and heads, no copy."""
    heads, nope, rope, v, c = 16, 128, 64, 128, 512
    w8, s = _wkv_b(heads, nope, v, c, 15)
    g = torch.Generator().manual_seed(16)
    q = torch.randn(2, 9, heads, nope + rope, generator=g).bfloat16()
    q_nope = torch.split(q.cuda(), [nope, rope], dim=-1)[0]
    assert not q_nope.is_contiguous()
    y = _absorb(q_nope, w8.cuda(), s.cuda(), Q, nope, v)
    assert y.shape == (2, 9, heads, c)
    _check(y, q[..., :nope], w8, s, Q, nope, v)
    assert torch.equal(y, _absorb(q_nope.contiguous(), w8.cuda(), s.cuda(), Q, nope, v))


def test_absorb_full_size_against_dequantised_einsum(K):
    """4096 tokens, 128 heads: against torch's bf16 einsum over weight_dequant's output on the device (both
    accumulate in binary32 and round once) and, on a sample of tokens, against the oracle's bound."""
    heads, nope, v, c, tokens = 128, 128, 128, 512, 4096
    w8, s = _wkv_b(heads, nope, v, c, 17)
    w8d, sd = w8.cuda(), s.cuda()
    wd = torch.ops.dsv3fp8.weight_dequant(w8d, sd, 128, 0).view(heads, nope + v, c)      # 0: bf16
    g = torch.Generator(device="cuda").manual_seed(18)
    pick = torch.tensor([0, 1, 2047, 4095])
    for side, width in ((Q, nope), (V, c)):
        x = torch.randn(tokens, heads, width, generator=g, device="cuda").bfloat16()
        y = _absorb(x, w8d, sd, side, nope, v)
        ref = torch.einsum("mhd,hdc->mhc", x, wd[:, :nope]) if side == Q else torch.einsum("mhc,hdc->mhd", x, wd[:, nope:])
        diff = (y.float() - ref.float()).abs()
        assert (diff <= 2.0 ** -7 * ref.float().abs() + 1e-3).all()
        _check(y[pick.cuda()], x[pick.cuda()].cpu(), w8, s, side, nope, v)


def test_absorb_rejects_unsupported(K):
    w8, s = _wkv_b(2, 64, 64, 128, 19)
    x = torch.randn(3, 2, 64).bfloat16().cuda()
    with pytest.raises(AssertionError):
        _absorb(x, w8.cuda(), s.cuda(), Q, 64, 32)          # rows of wkv_b do not match heads * (nope + v)
    w8, s = _wkv_b(2, 32, 32, 128, 19)
    with pytest.raises(RuntimeError, match="shape"):
        _absorb(x[..., :32].contiguous(), w8.cuda(), s.cuda(), Q, 32, 32)   # nope_dim 32 is not implemented


# ------------------------------------------------------------------ MLA.forward

@pytest.fixture()
def M():
    from dsv3fp8 import model
    old = (model.gemm_impl, model.attn_impl, torch.get_default_dtype())
    torch.set_default_dtype(torch.bfloat16)
    model.Linear.dtype = FP8
    model.gemm_impl = "fp8"
    yield model
    model.gemm_impl, model.attn_impl = old[0], old[1]
    model.Linear.dtype = torch.bfloat16
    model.MLA.fused = True
    model.MLA.stacked_a = True
    torch.set_default_dtype(old[2])


def _build(M, p, dim, heads, q_rank, kv_rank, nope, rope, v):
    args = M.ModelArgs(dim=dim, n_heads=heads, q_lora_rank=q_rank, kv_lora_rank=kv_rank, qk_nope_head_dim=nope,
                       qk_rope_head_dim=rope, v_head_dim=v, max_batch_size=2, max_seq_len=16, original_seq_len=16)
    with torch.device("cuda"):
        layer = M.MLA(args)
    with torch.no_grad():
        for name in ("wq_a", "wq_b", "wkv_a", "wkv_b", "wo"):
            lin = getattr(layer, name)
            lin.weight.copy_(p[name][0].cuda())
            lin.scale.copy_(p[name][1].cuda())
        layer.q_norm.weight.copy_(p["q_norm"].cuda())
        layer.kv_norm.weight.copy_(p["kv_norm"].cuda())
    return layer


def _close(got, ref, tol):
    """Layer outputs are bf16 tensors produced through several bf16 and fp8 roundings that the device and the
    oracle reach by different summation orders: allow tol * rms(ref) plus two bf16 steps at the largest
    magnitude."""
    import math
    got, ref = got.float().cpu(), ref.float()
    rms = ref.pow(2).mean().sqrt().item()
    ulp = 2.0 ** (math.floor(math.log2(max(ref.abs().max().item(), 1e-30))) - 7)
    assert (got - ref).abs().max().item() <= tol * rms + 2 * ulp, ((got - ref).abs().max().item(), rms, ulp)


def test_mla_prefill_then_decode_vs_oracle(M):
    dim, heads, q_rank, kv_rank, nope, rope, v = 256, 4, 128, 128, 64, 32, 64
    p = small_mla_params(dim, heads, q_rank, kv_rank, nope, rope, v, 20)
    layer = _build(M, p, dim, heads, q_rank, kv_rank, nope, rope, v)
    assert layer.wkv_b.weight.dtype == FP8 and layer.kv_cache.dtype == torch.bfloat16
    freqs = _freqs(rope, 16)
    g = torch.Generator().manual_seed(21)
    x0 = torch.randn(2, 7, dim, generator=g).bfloat16()
    x1 = torch.randn(2, 1, dim, generator=g).bfloat16()
    mask = torch.full((7, 7), float("-inf")).triu_(1)
    kv_c, pe_c = torch.zeros(2, 16, kv_rank, dtype=torch.bfloat16), torch.zeros(2, 16, rope, dtype=torch.bfloat16)
    scale = (nope + rope) ** -0.5
    ref0 = oracle.mla(x0, 0, freqs[:7], mask, p, kv_c, pe_c, heads, nope, rope, v, kv_rank, scale)
    ref1 = oracle.mla(x1, 7, freqs[7:8], None, p, kv_c, pe_c, heads, nope, rope, v, kv_rank, scale)
    with torch.inference_mode():
        y0 = layer(x0.cuda(), 0, freqs[:7].cuda(), mask.cuda())
        y1 = layer(x1.cuda(), 7, freqs[7:8].cuda(), None)
        _close(y0, ref0, 2e-2)
        _close(y1, ref1, 2e-2)
        _close(layer.kv_cache, kv_c, 2e-2)
        # wq_a and wkv_a ran as one stacked linear; the two layers still see their own weights
        assert layer._wa is not None and layer.wkv_a.weight.data_ptr() == layer._wa[layer.q_lora_rank:].data_ptr()
        M.MLA.stacked_a = False
        layer.kv_cache.zero_(); layer.pe_cache.zero_()
        u0 = layer(x0.cuda(), 0, freqs[:7].cuda(), mask.cuda())
        u1 = layer(x1.cuda(), 7, freqs[7:8].cuda(), None)
        M.MLA.stacked_a = True
        _close(y0, u0.cpu(), 1e-2)
        _close(y1, u1.cpu(), 1e-2)
        # the fused products against the reference's dequantise-then-einsum sequence on the same device
        M.MLA.fused = False
        layer.kv_cache.zero_(); layer.pe_cache.zero_()
        z0 = layer(x0.cuda(), 0, freqs[:7].cuda(), mask.cuda())
        z1 = layer(x1.cuda(), 7, freqs[7:8].cuda(), None)
        _close(y0, z0.cpu(), 2e-2)
        _close(y1, z1.cpu(), 2e-2)


def test_mla_naive_cache_layout_vs_oracle(M):
    """attn_impl = "naive" (model.py:443-445, 470-479, 488-490): per-head key / value caches, wkv_b as an FP8 linear
    layer.  Prefill then one decode step against oracle.mla(..., attn_impl="naive"), and against the absorbed layout."""
    dim, heads, q_rank, kv_rank, nope, rope, v = 256, 4, 128, 128, 64, 32, 64
    p = small_mla_params(dim, heads, q_rank, kv_rank, nope, rope, v, 22)
    absorbed = _build(M, p, dim, heads, q_rank, kv_rank, nope, rope, v)
    M.attn_impl = "naive"
    layer = _build(M, p, dim, heads, q_rank, kv_rank, nope, rope, v)
    M.attn_impl = "absorb"
    assert layer.k_cache.shape == (2, 16, heads, nope + rope) and layer.v_cache.shape == (2, 16, heads, v)
    assert not hasattr(layer, "kv_cache")
    freqs = _freqs(rope, 16)
    g = torch.Generator().manual_seed(23)
    x0 = torch.randn(2, 7, dim, generator=g).bfloat16()
    x1 = torch.randn(2, 1, dim, generator=g).bfloat16()
    mask = torch.full((7, 7), float("-inf")).triu_(1)
    k_c = torch.zeros(2, 16, heads, nope + rope, dtype=torch.bfloat16)
    v_c = torch.zeros(2, 16, heads, v, dtype=torch.bfloat16)
    scale = (nope + rope) ** -0.5
    ref0 = oracle.mla(x0, 0, freqs[:7], mask, p, k_c, v_c, heads, nope, rope, v, kv_rank, scale, attn_impl="naive")
    ref1 = oracle.mla(x1, 7, freqs[7:8], None, p, k_c, v_c, heads, nope, rope, v, kv_rank, scale, attn_impl="naive")
    with torch.inference_mode():
        y0 = layer(x0.cuda(), 0, freqs[:7].cuda(), mask.cuda())
        y1 = layer(x1.cuda(), 7, freqs[7:8].cuda(), None)
        _close(y0, ref0, 2e-2)
        _close(y1, ref1, 2e-2)
        _close(layer.k_cache, k_c, 2e-2)
        _close(layer.v_cache, v_c, 2e-2)
        a0 = absorbed(x0.cuda(), 0, freqs[:7].cuda(), mask.cuda())
        a1 = absorbed(x1.cuda(), 7, freqs[7:8].cuda(), None)
        for yn, ya in ((y0, a0), (y1, a1)):     # the two layouts differ by one FP8 quantisation of the latent
            rel = (yn.float() - ya.float()).pow(2).mean().sqrt() / ya.float().pow(2).mean().sqrt()
            assert rel.item() < 0.08, rel.item()
    with pytest.raises(ValueError):
        M.attn_impl = "other"
        M.MLA(M.ModelArgs(dim=dim, n_heads=heads, q_lora_rank=q_rank, kv_lora_rank=kv_rank))
