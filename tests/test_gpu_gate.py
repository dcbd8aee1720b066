"""GPU parity of the router's expert selection (dsv3_gate_route through torch.ops.dsv3fp8.gate_route and
Gate.forward) against the torch-CPU oracle of inference/model.py:577-598, on the same bf16 logits.

What can and cannot be bit-exact: the selection works on sigmoid values rounded to bf16 plus an fp32 bias; the
device's expf and the host's differ by an ulp of binary32 now and then, which flips a bf16 rounding with
probability ~3e-5 per value.  So the tests demand, per token, exactly the oracle's experts in the oracle's order
and weights within one bf16 step, for all but at most 0.2 % of the tokens, and for every token a selection that is
valid by the rule (top experts of its own scores, inside the best groups).  Equal scores are compared by value, not
by index (torch.topk leaves their order open; the kernel takes the lower index)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

SOFTMAX, SIGMOID = 0, 1


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    from dsv3fp8 import ops  # noqa: F401
    return dsv3fp8


def _route(logits, bias, topk, groups, topk_groups, func, scale):
    return torch.ops.dsv3fp8.gate_route(logits.cuda(), None if bias is None else bias.cuda(), topk, groups,
                                        topk_groups, func, scale)


def _biased(logits, bias, func):
    s = logits.sigmoid() if func == SIGMOID else logits.softmax(dim=-1, dtype=torch.float32)
    return s, (s + bias if bias is not None else s)


def _compare(logits, bias, topk, groups, topk_groups, func, scale, max_bad=0.002):
    w, idx = _route(logits, bias, topk, groups, topk_groups, func, scale)
    w, idx = w.cpu(), idx.cpu()
    assert w.dtype == torch.bfloat16 and idx.dtype == torch.int64 and idx.shape == (logits.size(0), topk)
    ref_w, ref_i = oracle.gate_route(logits, bias, topk, groups, topk_groups, scale,
                                     "sigmoid" if func == SIGMOID else "softmax")
    ref_w = ref_w.to(torch.bfloat16)
    orig, sel = _biased(logits, bias, func)
    tokens, experts = logits.shape
    # tokens whose answer the rule leaves open: equal scores across the cut, among groups or among experts
    # (bf16 logits make exact ties common when there is no fp32 bias); they only get the validity checks below
    open_ = torch.zeros(tokens, dtype=torch.bool)
    masked = sel
    if groups > 1:
        gview = sel.view(tokens, groups, -1)
        gscore = gview.amax(-1) if bias is None else gview.topk(2, dim=-1)[0].sum(-1)
        gsort = gscore.sort(-1, descending=True)[0]
        if topk_groups < groups:
            open_ |= gsort[:, topk_groups - 1] == gsort[:, topk_groups]
        gsz = experts // groups
        in_ref_groups = torch.zeros(tokens, groups, dtype=torch.bool).scatter_(1, ref_i // gsz, True)
        masked = gview.masked_fill(~in_ref_groups.unsqueeze(-1), float("-inf")).flatten(1)
    if topk < experts:
        msort = masked.sort(-1, descending=True)[0]
        open_ |= msort[:, topk - 1] == msort[:, topk]
    assert open_.float().mean().item() < 0.5
    # by value: the selected (biased) scores, in order
    same = (sel.gather(1, idx).float() == sel.gather(1, ref_i).float()).all(-1) | open_
    ulp = ref_w.float().abs() * 2.0 ** -7
    if func == SOFTMAX:
        ulp = ulp + 2.0 ** -8 * ref_w.float().abs()          # softmax sums in another order
    close = ((w.float() - ref_w.float()).abs() <= ulp).all(-1) | open_
    bad = (~(same & close)).float().mean().item()
    assert bad <= max_bad, bad
    # every token: distinct experts, descending scores, inside at most topk_groups groups
    assert all(len(set(r.tolist())) == topk for r in idx)
    picked = sel.gather(1, idx).float()
    assert (picked[:, :-1] >= picked[:, 1:]).all()
    if groups > 1:
        gsz = experts // groups
        assert all(len(set((r // gsz).tolist())) <= topk_groups for r in idx)
    return w, idx


@pytest.mark.parametrize("tokens", [1, 3, 64, 4096])
def test_gate_route_671b(K, tokens):
    g = torch.Generator().manual_seed(tokens)
    logits = (torch.randn(tokens, 256, generator=g) * 1.5).bfloat16()
    bias = torch.randn(256, generator=g) * 0.1
    w, idx = _compare(logits, bias, 8, 8, 4, SIGMOID, 2.5)
    assert torch.allclose(w.float().sum(-1), torch.full((tokens,), 2.5), atol=0.05)


@pytest.mark.parametrize("experts,topk,groups,topk_groups,with_bias,func", [
    (64, 6, 1, 1, False, SOFTMAX),       # the 16B configuration: softmax, no groups, no bias
    (160, 6, 8, 3, False, SOFTMAX),      # the 236B configuration: group score = max
    (8, 2, 2, 1, False, SIGMOID),        # tiny: many equal bf16 scores
    (64, 8, 8, 4, True, SIGMOID),
    (512, 16, 16, 4, True, SIGMOID),
    (96, 5, 3, 2, True, SOFTMAX),
])
def test_gate_route_other_configs(K, experts, topk, groups, topk_groups, with_bias, func):
    g = torch.Generator().manual_seed(experts + topk)
    logits = (torch.randn(257, experts, generator=g) * 2).bfloat16()
    bias = torch.randn(experts, generator=g) * 0.2 if with_bias else None
    _compare(logits, bias, topk, groups, topk_groups, func, 1.0 if func == SOFTMAX else 16.0)


def test_gate_route_known_answer(K):
    """Logits built so that the answer is known in closed form: group 1 and group 3 hold the largest pairs; the
    bias moves the selection but not the weights."""
    experts, groups = 16, 4
    logits = torch.full((1, experts), -4.0)
    logits[0, 4], logits[0, 5] = 2.0, 1.0            # group 1
    logits[0, 12], logits[0, 13] = 3.0, -1.0         # group 3
    logits[0, 0] = 2.5                                # group 0: one large value, small pair sum with bias
    bias = torch.zeros(experts); bias[5] = 0.5; bias[13] = 0.5
    w, idx = _route(logits.bfloat16(), bias, 3, groups, 2, SIGMOID, 1.0)
    # group sums (sigmoid + bias): g0 = s(2.5)+s(-4) = 0.942, g1 = s(2)+s(1)+0.5 = 2.11, g3 = s(3)+s(-1)+0.5 = 1.72
    assert idx.cpu().tolist() == [[5, 12, 4]]        # biased: 5 -> 1.231, 12 -> 0.953, 4 -> 0.881, 13 -> 0.769
    s = torch.tensor([1.0, 3.0, 2.0]).bfloat16().sigmoid()
    exp = (s / s.sum(-1, keepdim=True)) * 1.0
    assert torch.equal(w.cpu()[0], exp)


def test_gate_forward_uses_the_kernel_and_matches_the_tensor_ops(K):
    from dsv3fp8 import model as M
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        args = M.ModelArgs()
        with torch.device("cuda"):
            gate = M.Gate(args)
        g = torch.Generator(device="cuda").manual_seed(3)
        with torch.no_grad():
            gate.weight.copy_(torch.randn(256, 7168, generator=g, device="cuda") * 0.02)
            gate.bias.copy_(torch.randn(256, generator=g, device="cuda") * 0.1)
        x = torch.randn(512, 7168, generator=g, device="cuda").bfloat16()
        w1, i1 = gate(x)
        M.Gate.fused = False
        w0, i0 = gate(x)
        M.Gate.fused = True
        # the same experts by value (equal biased scores may come out in either order)
        sel = torch.nn.functional.linear(x, gate.weight).sigmoid().float() + gate.bias
        assert (sel.gather(1, i1) == sel.gather(1, i0)).all(-1).float().mean().item() >= 0.998
        same = (i1 == i0).all(-1)
        assert same.float().mean().item() >= 0.9
        assert ((w1.float() - w0.float()).abs() <= w0.float().abs() * 2.0 ** -7)[same].all()
    finally:
        M.Gate.fused = True
        torch.set_default_dtype(old)
