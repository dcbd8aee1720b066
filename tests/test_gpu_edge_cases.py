"""Edge cases through the C ABI on the device: empty inputs for every op, and the 32-bit row-offset boundary of the
large-M kernel (a problem whose activation matrix exceeds 4 GiB must take the generic tile kernel and still be
right)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    from dsv3fp8 import ops  # noqa: F401
    return dsv3fp8


def test_empty_inputs(K):
    dev = "cuda"
    y, s = K.act_quant(torch.empty(0, 256, dtype=torch.bfloat16, device=dev))
    assert y.shape == (0, 256) and y.dtype == FP8 and s.shape == (0, 2)
    y, s = K.act_quant(torch.empty(3, 0, 128, dtype=torch.bfloat16, device=dev))
    assert y.shape == (3, 0, 128) and s.shape == (3, 0, 1)

    w8 = torch.zeros(256, 128, dtype=torch.uint8, device=dev).view(FP8)
    ws = torch.ones(2, 1, device=dev)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        d = K.weight_dequant(torch.empty(0, 128, dtype=torch.uint8, device=dev).view(FP8), torch.empty(0, 1, device=dev))
        assert d.shape == (0, 128) and d.dtype == torch.bfloat16
        a = torch.empty(0, 128, dtype=torch.uint8, device=dev).view(FP8)
        c = K.fp8_gemm(a, torch.empty(0, 1, device=dev), w8, ws)                      # no rows
        assert c.shape == (0, 256)
        a = torch.zeros(5, 128, dtype=torch.uint8, device=dev).view(FP8)
        c = K.fp8_gemm(a, torch.ones(5, 1, device=dev), w8[:0].contiguous(), ws[:0].contiguous())   # no columns
        assert c.shape == (5, 0)
    finally:
        torch.set_default_dtype(old)

    w, i = torch.ops.dsv3fp8.gate_route(torch.empty(0, 64, dtype=torch.bfloat16, device=dev), None, 4, 1, 1, 1, 1.0)
    assert w.shape == (0, 4) and i.shape == (0, 4) and i.dtype == torch.int64
    wk8 = torch.zeros(2 * 256, 512, dtype=torch.uint8, device=dev).view(FP8)
    y = torch.ops.dsv3fp8.wkv_b_absorb(torch.empty(0, 2, 128, dtype=torch.bfloat16, device=dev), wk8,
                                       torch.ones(4, 4, device=dev), 0, 128, 128)
    assert y.shape == (0, 2, 512)
    out = torch.ops.dsv3fp8.moe_route(torch.empty(0, 2, dtype=torch.int64, device=dev),
                                      torch.empty(0, 2, dtype=torch.bfloat16, device=dev), 8, False)
    assert out[0].tolist() == [0] * 8 and out[1].numel() == 0 and (out[4] == -1).all()
    y = torch.ops.dsv3fp8.moe_combine(torch.empty(0, 256, dtype=torch.bfloat16, device=dev),
                                      torch.empty(0, 2, dtype=torch.int32, device=dev),
                                      torch.empty(0, 2, dtype=torch.bfloat16, device=dev), None)
    assert y.shape == (0, 256)
    torch.cuda.synchronize()


def test_activation_matrix_beyond_4_gib(K):
    """300 000 x 16384 fp8 activations (4.9 GB): row offsets no longer fit 32 bits, which the large-M kernel relies
    on; the dispatcher must fall back, and rows at both ends and across the 4 GiB line must match the oracle."""
    from dsv3fp8 import workloads
    m, k, n = 300_000, 16384, 128
    g = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randint(0, 0x78, (m, k), generator=g, dtype=torch.uint8, device="cuda")
    a |= (torch.randint(0, 2, (m, 1), generator=g, dtype=torch.uint8, device="cuda") << 7)      # a sign per row
    a = a.view(FP8)
    a_s = torch.rand(m, k // 128, generator=g, device="cuda") * 1e-2 + 1e-3
    w8, ws = workloads.weight(n, k, seed=2)
    c = K.fp8_gemm_f32(a, a_s, w8.cuda(), ws.cuda())
    line = (1 << 32) // k                                   # first row whose byte offset needs 33 bits
    rows = torch.tensor([0, 1, 77, line - 1, line, line + 1, m - 2, m - 1])
    ref = oracle.fp8_gemm_f32(a[rows.cuda()].cpu(), a_s[rows.cuda()].cpu(), w8, ws)
    got = c[rows.cuda()].cpu()
    assert (got - ref).abs().max().item() <= 1e-2 * ref.pow(2).mean().sqrt().item()
    del a, a_s, c
    torch.cuda.empty_cache()


@pytest.mark.parametrize("m,k", [(2, 32768), (1, 61568)])
def test_few_rows_and_a_very_long_k(m, k):
    """K beyond every DeepSeek-V3 projection at one and two rows: the activation slab of the few-row kernel is capped
    at what 64 KiB of LDS holds (more K splits instead of a refused launch)."""
    import dsv3fp8 as K
    g = torch.Generator().manual_seed(k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w8, ws = oracle.block_quant_weight((torch.randn(256, k, generator=g) * 0.02).bfloat16())
    a, a_s = oracle.act_quant(x)
    ref = oracle.fp8_gemm_f32(a, a_s, w8, ws)
    got = K.fp8_gemm_f32(a.cuda(), a_s.cuda(), w8.cuda(), ws.cuda()).cpu()
    assert (got - ref).abs().max().item() <= 1e-2 * ref.pow(2).mean().sqrt().item()


def test_moe_beyond_the_grouped_limits_takes_the_expert_loop():
    """17 experts per token is more than the grouped bookkeeping handles (16): MoE.forward falls back to the
    reference's expert loop instead of raising, and an empty batch returns an empty result."""
    from dsv3fp8 import model as M
    old = (M.gemm_impl, torch.get_default_dtype(), M.Linear.dtype)
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype, M.gemm_impl = torch.float8_e4m3fn, "fp8"
    try:
        args = M.ModelArgs(dim=256, inter_dim=512, moe_inter_dim=128, n_routed_experts=32, n_shared_experts=1,
                           n_activated_experts=17, n_expert_groups=1, n_limited_groups=1, route_scale=1.0)
        with torch.device("cuda"):
            moe = M.MoE(args)
        g = torch.Generator().manual_seed(3)
        with torch.no_grad():
            moe.gate.weight.copy_((torch.randn(32, 256, generator=g) * 0.05).bfloat16().cuda())
            for lin in [l for ex in list(moe.experts) + [moe.shared_experts] for l in (ex.w1, ex.w2, ex.w3)]:
                w8, s = oracle.block_quant_weight((torch.randn(lin.out_features, lin.in_features, generator=g) * 0.05).bfloat16())
                lin.weight.copy_(w8.cuda()); lin.scale.copy_(s.cuda())
        x = torch.randn(9, 256, generator=g).bfloat16().cuda()
        with torch.inference_mode():
            assert not moe._grouped_ok(x)
            y = moe(x)
            assert y.shape == x.shape and torch.isfinite(y.float()).all()
            empty = moe(x[:0])
            assert empty.shape == (0, 256)
    finally:
        M.gemm_impl, M.Linear.dtype = old[0], old[2]
        torch.set_default_dtype(old[1])
