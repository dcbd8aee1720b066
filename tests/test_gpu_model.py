"""GPU parity of the host-side callers (dsv3fp8.model, the mirror of the reference's inference/model.py
linear()/Linear/MLP/Gate/Expert/MoE) against the torch-CPU oracle on small configurations."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


@pytest.fixture()
def M():
    from dsv3fp8 import model
    old_impl, old_dtype = model.gemm_impl, torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)          # as the reference's entry point does (generate.py:109)
    model.Linear.dtype = FP8
    yield model
    model.gemm_impl = old_impl
    model.Linear.dtype = torch.bfloat16
    model.Linear.scale_fmt = None
    torch.set_default_dtype(old_dtype)


def _fill(lin, seed):
    """Random block-quantised weight into an fp8 Linear (keeps the weight.scale attribute, like load_model)."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(lin.out_features, lin.in_features, generator=g) * 0.05).bfloat16()
    w8, s = oracle.block_quant_weight(w)
    with torch.no_grad():
        lin.weight.copy_(w8.cuda())
        lin.scale.copy_(s.cuda())
    return w8, s


def _close(got, ref, tol=2e-2):
    got, ref = got.float().cpu(), ref.float()
    rms = ref.pow(2).mean().sqrt().item()
    assert (got - ref).abs().max().item() <= tol * max(rms, 1e-6) + 2 ** -8 * ref.abs().max().item()


@pytest.mark.parametrize("impl", ["fp8", "bf16"])
def test_linear_dispatch(M, impl):
    M.gemm_impl = impl
    with torch.device("cuda"):
        lin = M.Linear(512, 384, bias=True)
    assert lin.weight.dtype == FP8 and lin.scale.shape == (3, 4) and lin.weight.scale is lin.scale
    w8, s = _fill(lin, 1)
    with torch.no_grad():
        lin.bias.copy_(torch.linspace(-1, 1, 384))
    x = torch.randn(2, 5, 512, generator=torch.Generator().manual_seed(2)).bfloat16()
    with torch.inference_mode():
        y = lin(x.cuda())
    ref = oracle.linear(x, w8, bias=lin.bias.detach().cpu(), scale=s, gemm_impl=impl)
    assert y.shape == (2, 5, 384) and y.dtype == torch.bfloat16
    _close(y, ref)


def test_wide_weights_take_f_linear(M):
    with torch.device("cuda"):
        lin = M.Linear(256, 128, dtype=torch.bfloat16)
    assert lin.scale is None
    torch.nn.init.normal_(lin.weight, std=0.05)
    x = torch.randn(4, 256, device="cuda").bfloat16()
    assert torch.equal(lin(x), torch.nn.functional.linear(x, lin.weight))


def test_scale_fmt_only_reaches_plain_linear(M):
    M.gemm_impl = "fp8"
    M.Linear.scale_fmt = "ue8m0"
    with torch.device("cuda"):
        plain, col = M.Linear(256, 128), M.ColumnParallelLinear(256, 128)
    w8, s = _fill(plain, 3)
    _fill(col, 3)
    x = torch.randn(8, 256, generator=torch.Generator().manual_seed(4)).bfloat16()
    with torch.inference_mode():
        yp, yc = plain(x.cuda()), col(x.cuda())
    _close(yp, oracle.linear(x, w8, scale=s, scale_fmt="ue8m0"), tol=1e-2)
    _close(yc, oracle.linear(x, w8, scale=s, scale_fmt=None), tol=1e-2)


def test_linear_with_power_of_two_scales_takes_the_scaled_matrix_instruction(M, monkeypatch):
    """scale_fmt = "ue8m0" on a weight whose block scales are powers of two (config_v3.1-style checkpoints) and more
    than 64 rows: linear() calls fp8_gemm_pow2; any other weight, or few rows, takes the general path."""
    M.gemm_impl = "fp8"
    M.Linear.scale_fmt = "ue8m0"
    with torch.device("cuda"):
        lin = M.Linear(512, 384)
    g = torch.Generator().manual_seed(7)
    w = (torch.randn(384, 512, generator=g) * 0.05).bfloat16().float()
    amax = w.view(3, 128, 4, 128).abs().amax(dim=(1, 3))
    s = torch.pow(2.0, torch.ceil(torch.log2(amax / 448.0)))
    w8 = (w.view(3, 128, 4, 128) / s[:, None, :, None]).reshape(384, 512).to(FP8)
    with torch.no_grad():
        lin.weight.copy_(w8.cuda()); lin.scale.copy_(s.cuda())
    calls = []
    real = M.fp8_gemm_pow2
    monkeypatch.setattr(M, "fp8_gemm_pow2", lambda *a: (calls.append(a[0].shape[0]), real(*a))[1])
    x = torch.randn(300, 512, generator=g).bfloat16()
    with torch.inference_mode():
        y = lin(x.cuda())
        y_few = lin(x[:8].cuda())
    assert calls == [300]
    _close(y, oracle.linear(x, w8, scale=s, scale_fmt="ue8m0"), tol=1e-2)
    _close(y_few, oracle.linear(x[:8], w8, scale=s, scale_fmt="ue8m0"), tol=1e-2)
    with torch.no_grad():
        lin.scale.mul_(1.5)                                   # no longer powers of two: noticed through the version
    with torch.inference_mode():
        y2 = lin(x.cuda())
    assert calls == [300]
    _close(y2, oracle.linear(x, w8, scale=s * 1.5, scale_fmt="ue8m0"), tol=1e-2)


def test_moe_layer_small(M):
    M.gemm_impl = "fp8"
    args = M.ModelArgs(dim=256, inter_dim=512, moe_inter_dim=128, n_routed_experts=8, n_shared_experts=1,
                       n_activated_experts=2, n_expert_groups=2, n_limited_groups=1, route_scale=2.5)
    with torch.device("cuda"):
        moe = M.MoE(args)
    assert moe.gate.bias is None and moe.gate.weight.dtype == torch.bfloat16
    g = torch.Generator().manual_seed(5)
    gw = (torch.randn(8, 256, generator=g) * 0.05).bfloat16()     # scores ~ N(0, 0.8): away from sigmoid saturation
    with torch.no_grad():
        moe.gate.weight.copy_(gw.cuda())
    experts = []
    for i, ex in enumerate(moe.experts):
        w1, s1 = _fill(ex.w1, 10 + 3 * i); w2, s2 = _fill(ex.w2, 11 + 3 * i); w3, s3 = _fill(ex.w3, 12 + 3 * i)
        experts.append((w1, s1, w2, s2, w3, s3))
    sh = moe.shared_experts
    shared = (*_fill(sh.w1, 90), *_fill(sh.w2, 91), *_fill(sh.w3, 92))
    x = torch.randn(3, 7, 256, generator=g).bfloat16()
    with torch.inference_mode():
        y = moe(x.cuda())
        wts, idx = moe.gate(x.view(-1, 256).cuda())
    ref_w, ref_i = oracle.gate(x.view(-1, 256), gw, None, topk=2, n_groups=2, topk_groups=1, route_scale=2.5)
    # the router's bf16 GEMM runs in a different summation order on the GPU: near-ties may flip, the bulk may not
    same = (idx.cpu().sort(-1)[0] == ref_i.sort(-1)[0]).all(-1).float().mean().item()
    assert same >= 0.8, same
    ref = oracle.moe(x, wts.cpu(), idx.cpu(), experts, shared)
    assert y.shape == x.shape
    _close(y, ref, tol=5e-2)


def test_gate_with_bias_671b_width(M):
    args = M.ModelArgs(n_routed_experts=64, n_expert_groups=8, n_limited_groups=4, n_activated_experts=8)
    with torch.device("cuda"):
        gate = M.Gate(args)
    assert gate.bias is not None and gate.bias.dtype == torch.float32
    g = torch.Generator().manual_seed(6)
    gw = (torch.randn(64, 7168, generator=g) * 0.02).bfloat16()
    gb = torch.randn(64, generator=g) * 0.1
    with torch.no_grad():
        gate.weight.copy_(gw.cuda()); gate.bias.copy_(gb.cuda())
    x = torch.randn(32, 7168, generator=g).bfloat16()
    w, idx = gate(x.cuda())
    assert w.dtype == torch.bfloat16 and idx.shape == (32, 8)
    assert all(len(set(r.tolist())) == 8 for r in idx.cpu())
    assert all(len(set((r // 8).tolist())) <= 4 for r in idx.cpu())
    assert torch.allclose(w.float().sum(-1).cpu(), torch.full((32,), 2.5, dtype=torch.float32), atol=0.05)


@pytest.mark.parametrize("tokens", [5, 300])
def test_mlp_stacked_matches_three_linears_and_oracle(M, tokens):
    """MLP.forward with w1 | w3 as one GEMM and SwiGLU fused with the re-quantisation, against the reference's
    three linears on the device and against the oracle."""
    M.gemm_impl = "fp8"
    with torch.device("cuda"):
        mlp = M.MLP(256, 384)
    w1, s1 = _fill(mlp.w1, 1); w2, s2 = _fill(mlp.w2, 2); w3, s3 = _fill(mlp.w3, 3)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(tokens, 256, generator=g).bfloat16()
    with torch.inference_mode():
        y = mlp(x.cuda())
        assert mlp._w13 is not None and mlp.w3.weight.data_ptr() == mlp._w13[384:].data_ptr()
        M.MLP.stacked = False
        try:
            y3 = mlp(x.cuda())
        finally:
            M.MLP.stacked = True
    ref = oracle.mlp(x, w1, s1, w2, s2, w3, s3)
    _close(y, ref)
    _close(y, y3.cpu(), tol=1e-2)
