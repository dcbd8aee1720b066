"""GPU parity of the grouped mixture-of-experts path (group_tiles, fp8_gemm_grouped, swiglu_quant, moe_combine
and MoE.forward on top of them) against the torch-CPU oracle of inference/model.py:601-633, 669-693."""
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle

pytestmark = pytest.mark.gpu

FP8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    from dsv3fp8 import ops  # noqa: F401  (registers torch.ops.dsv3fp8)
    return dsv3fp8


def _tables(counts, max_tiles):
    from dsv3fp8 import ops
    R = ops.grouped_tile_rows()
    tg, t0, tr = torch.ops.dsv3fp8.group_tiles(torch.tensor(counts, dtype=torch.int32, device="cuda"), max_tiles)
    return R, tg, t0, tr


@pytest.mark.parametrize("counts", [[5, 0, 300, 256, 1], [0, 0, 0], [700], list(range(0, 600, 7))])
def test_group_tiles(K, counts):
    total = sum(counts)
    R, tg, t0, tr = _tables(counts, 1)
    max_tiles = total // R + len(counts)
    R, tg, t0, tr = _tables(counts, max_tiles)
    exp, row = [], 0
    for g, c in enumerate(counts):
        for i in range(0, c, R):
            exp.append((g, row + i, min(R, c - i)))
        row += c
    got = list(zip(tg.tolist(), t0.tolist(), tr.tolist()))
    assert got[:len(exp)] == exp
    assert all(g == -1 and n == 0 for g, _, n in got[len(exp):]) and len(got) == max_tiles


def _grouped_case(counts, n, k, seed, gather):
    g = torch.Generator().manual_seed(seed)
    groups, rows = len(counts), sum(counts)
    src_rows = rows + 3 if gather else rows
    x = torch.randn(src_rows, k, generator=g).bfloat16()
    xq, xs = oracle.act_quant(x)
    w = [oracle.block_quant_weight((torch.randn(n, k, generator=g) * 0.05).bfloat16()) for _ in range(groups)]
    a_rows = torch.randint(0, src_rows, (rows,), generator=g, dtype=torch.int32) if gather else None
    return xq, xs, w, a_rows


@pytest.mark.parametrize("counts,n,k,gather", [
    ([5, 0, 300, 256, 1], 384, 512, True),
    ([129, 64], 576, 256, False),            # ragged n: 576 = 2 tiles + 64, 5 scale rows
    ([40] * 6, 256, 1152, True),             # odd number of K blocks
    ([145, 177, 200, 241, 17], 512, 384, True),   # 256-row slots with 10, 12, 13 and 16 live sub-tiles, then a small one
    ([300, 7, 250, 193, 150, 100], 256, 1536, True),   # every tile configuration, 12 K blocks: scales in three batches of four blocks
    ([1] * 9, 4096, 7168, True),             # one token of the MoE layer: the weight-streaming kernel (up to 320 rows in all)
    ([2, 0, 1, 5, 0, 3], 7168, 2048, False), # ... its second GEMM shape, ragged group sizes, no gather
    ([20, 3, 13], 200, 640, True),           # ... a slot of more than 16 rows (two passes), n not a multiple of 32
    ([36], 48, 128, False),                  # ... one K block, three passes
    ([40] * 8, 96, 256, True),               # ... 320 rows: the largest launch that takes this kernel
])
def test_fp8_gemm_grouped_vs_oracle(K, counts, n, k, gather):
    from dsv3fp8 import ops
    xq, xs, w, a_rows = _grouped_case(counts, n, k, 11, gather)
    rows = sum(counts)
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    out32 = torch.ops.dsv3fp8.fp8_gemm_grouped(xq.cuda(), xs.cuda(), a_rows.cuda() if gather else None, b, b_s, rows,
                                               tg, t0, tr, ops.dtype_code(torch.float32))
    out16 = torch.ops.dsv3fp8.fp8_gemm_grouped(xq.cuda(), xs.cuda(), a_rows.cuda() if gather else None, b, b_s, rows,
                                               tg, t0, tr, ops.dtype_code(torch.bfloat16))
    assert out32.shape == (rows, n) and out16.dtype == torch.bfloat16
    assert torch.equal(out16.float(), out32.bfloat16().float())          # bf16 output = RNE of the fp32 result
    row = 0
    for gi, c in enumerate(counts):
        if c == 0:
            continue
        idx = a_rows[row:row + c].long() if gather else torch.arange(row, row + c)
        ref = oracle.fp8_gemm_f32(xq[idx], xs[idx], w[gi][0], w[gi][1])
        err = (out32[row:row + c].cpu() - ref).abs().max().item()
        assert err <= 1e-2 * ref.pow(2).mean().sqrt().item(), (gi, err)     # tolerance of the fp32 output
        row += c


@pytest.mark.parametrize("seed", range(12))
def test_fp8_gemm_grouped_seeded_sweep(K, seed):
    """Random group sizes (empty groups, one row, several slots per group), n and k: every tile configuration, launches
    of the weight-streaming kernel (up to 320 rows in all), K ranges with and without whole batches of four scale
    blocks, ragged n.  Every group against the oracle."""
    from dsv3fp8 import ops
    r = torch.Generator().manual_seed(100 + seed)
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=r))
    small = seed % 4 == 0                                     # a launch of the weight-streaming kernel
    groups = pick(1, 7) if small else pick(3, 7)
    top = (30, 140, 200, 420)[seed % 4]                       # ... then slots of every height
    counts = [0 if pick(0, 5) == 0 else pick(1, top) for _ in range(groups)]
    counts[0] = max(counts[0], 1 if small else 330)
    n = 16 * pick(1, 40)
    k = 512 * pick(1, 4) if seed & 2 else 128 * pick(1, 16)   # whole batches of four scale blocks, or any K
    gather = bool(seed & 1)
    xq, xs, w, a_rows = _grouped_case(counts, n, k, 200 + seed, gather)
    rows = sum(counts)
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    out = torch.ops.dsv3fp8.fp8_gemm_grouped(xq.cuda(), xs.cuda(), a_rows.cuda() if gather else None, b, b_s, rows,
                                             tg, t0, tr, ops.dtype_code(torch.float32)).cpu()
    row = 0
    for gi, c in enumerate(counts):
        if c == 0:
            continue
        idx = a_rows[row:row + c].long() if gather else torch.arange(row, row + c)
        ref = oracle.fp8_gemm_f32(xq[idx], xs[idx], w[gi][0], w[gi][1])
        err = (out[row:row + c] - ref).abs().max().item()
        assert err <= 1e-2 * ref.pow(2).mean().sqrt().item(), (counts, n, k, gi, err)     # tolerance of the fp32 output
        row += c


def test_fp8_gemm_grouped_scale_batches_need_aligned_scales(K):
    """A row of a_s that is a whole number of 16-byte pieces lets the 256-row slots copy the scales of four K blocks
    at a time; the same a_s four bytes further on in memory takes the one-line copies.  Same bits either way."""
    from dsv3fp8 import ops
    counts, n, k = [300, 250, 40], 256, 1024
    xq, xs, w, a_rows = _grouped_case(counts, n, k, 13, True)
    rows = sum(counts)
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    xs_al = xs.cuda()
    xs_off = torch.empty(xs.numel() + 1, dtype=torch.float32, device="cuda")[1:].view_as(xs)
    xs_off.copy_(xs_al)
    assert xs_al.data_ptr() % 16 == 0 and xs_off.data_ptr() % 16 == 4
    outs = [torch.ops.dsv3fp8.fp8_gemm_grouped(xq.cuda(), s, a_rows.cuda(), b, b_s, rows, tg, t0, tr,
                                               ops.dtype_code(torch.float32)) for s in (xs_al, xs_off)]
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
@pytest.mark.parametrize("counts,inter,k,gather", [
    ([128, 97, 161, 0, 300, 131, 200, 256, 3, 193], 256, 512, True),     # every tile configuration: <= 128, 129-192, > 192 rows
    ([500], 128, 128, False),                                           # one column tile, one K block
    ([40, 255, 130, 64], 384, 1152, True),                              # odd number of K blocks, three column tiles
])
def test_grouped_gemm_with_swiglu_epilogue_equals_the_two_calls(K, counts, inter, k, gather, fmt):
    """dsv3_fp8_gemm_grouped_swiglu (silu(h1) * h3 and its act_quant in the epilogue of the w1 | w3 GEMM) against
    dsv3_fp8_gemm_grouped followed by dsv3_swiglu_quant: bytes and scales bit for bit, including rows whose group
    fills only part of a tile.  The two-call chain is held against the oracle elsewhere."""
    from dsv3fp8 import ops, _lib
    code_fmt = _lib.SCALE_FMT_UE8M0 if fmt == "ue8m0" else _lib.SCALE_FMT_NONE
    xq, xs, w, a_rows = _grouped_case(counts, 2 * inter, k, 500 + inter, gather)
    rows = sum(counts)
    assert ops.grouped_swiglu_fused(rows, xq.size(0), inter, k)
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    args = (xq.cuda(), xs.cuda(), a_rows.cuda() if gather else None, b, b_s, rows, tg, t0, tr)
    h = torch.ops.dsv3fp8.fp8_gemm_grouped(*args, ops.dtype_code(torch.bfloat16))
    y2, s2 = torch.ops.dsv3fp8.swiglu_quant(h, 128, code_fmt)
    y = torch.full((rows, inter), 0x7F, dtype=torch.uint8, device="cuda").view(FP8)     # poisoned outputs
    y1, s1 = torch.ops.dsv3fp8.fp8_gemm_grouped_swiglu(*args, code_fmt)
    assert y1.shape == y2.shape == (rows, inter) and s1.shape == s2.shape == (rows, inter // 128)
    assert torch.equal(s1, s2)
    assert torch.equal(y1.view(torch.uint8), y2.view(torch.uint8))
    assert bool(torch.isfinite(s1).all()) and int((y1.view(torch.uint8) & 0x7F).max()) == 0x7E
    del y
    # few rows in all: the op falls back to the two calls (the weight-streaming kernel has no such epilogue)
    small = [3, 0, 9]
    xq, xs, w, _ = _grouped_case(small, 2 * inter, k, 600, False)
    assert not ops.grouped_swiglu_fused(sum(small), xq.size(0), inter, k)
    R, tg, t0, tr = _tables(small, len(small) + 1)
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    args = (xq.cuda(), xs.cuda(), None, b, b_s, sum(small), tg, t0, tr)
    y1, s1 = torch.ops.dsv3fp8.fp8_gemm_grouped_swiglu(*args, code_fmt)
    y2, s2 = torch.ops.dsv3fp8.swiglu_quant(torch.ops.dsv3fp8.fp8_gemm_grouped(*args, ops.dtype_code(torch.bfloat16)), 128, code_fmt)
    assert torch.equal(s1, s2) and torch.equal(y1.view(torch.uint8), y2.view(torch.uint8))


def test_fp8_gemm_grouped_seeded_tables(K):
    """Twelve seeded tables mixing empty, tiny, 129-192-row, 193-256-row and multi-tile groups (every tile
    configuration of the grouped kernel, and the weight-streaming kernel when the total is small)."""
    from dsv3fp8 import ops
    gen = torch.Generator().manual_seed(77)
    kinds = [(0, 0), (1, 16), (17, 128), (129, 192), (193, 256), (257, 600)]
    for case in range(12):
        groups = int(torch.randint(1, 9, (1,), generator=gen))
        if case % 4 == 3:                                    # a small launch: at most 320 rows in all
            counts = [int(torch.randint(0, 40, (1,), generator=gen)) for _ in range(groups)]
        else:
            counts = []
            for _ in range(groups):
                lo, hi = kinds[int(torch.randint(0, len(kinds), (1,), generator=gen))]
                counts.append(int(torch.randint(lo, hi + 1, (1,), generator=gen)))
        if sum(counts) == 0:
            counts[0] = 3
        n = 8 * int(torch.randint(4, 80, (1,), generator=gen))
        k = 128 * int(torch.randint(1, 7, (1,), generator=gen))
        gather = bool(case % 2)
        xq, xs, w, a_rows = _grouped_case(counts, n, k, 300 + case, gather)
        rows = sum(counts)
        R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
        b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
        b_s = torch.stack([wi[1] for wi in w]).cuda()
        out = torch.ops.dsv3fp8.fp8_gemm_grouped(xq.cuda(), xs.cuda(), a_rows.cuda() if gather else None, b, b_s, rows,
                                                 tg, t0, tr, ops.dtype_code(torch.float32)).cpu()
        row = 0
        for gi, c in enumerate(counts):
            if c:
                idx = a_rows[row:row + c].long() if gather else torch.arange(row, row + c)
                ref = oracle.fp8_gemm_f32(xq[idx], xs[idx], w[gi][0], w[gi][1])
                err = (out[row:row + c] - ref).abs().max().item()
                assert err <= 1e-2 * ref.pow(2).mean().sqrt().item(), (case, counts, n, k, gi, err)
            row += c


@pytest.mark.parametrize("counts,n,k", [([5, 0, 300, 256, 1], 384, 512), ([145, 177, 200, 241, 17], 512, 384),
                                        ([3, 2, 9], 256, 256),
                                        ([300, 7, 150, 193, 100], 256, 1536)])   # scales in three batches of four K blocks
def test_fp8_gemm_grouped_power_of_two_scales(K, counts, n, k):
    """Scales that are powers of two on both sides: the grouped tile kernel hands them to the matrix instruction
    (every tile configuration), a small launch takes the weight-streaming kernel as before."""
    from dsv3fp8 import ops
    g = torch.Generator().manual_seed(21)
    rows = sum(counts)
    x = torch.randn(rows, k, generator=g).bfloat16()
    xq, xs = oracle.act_quant(x, 128, "ue8m0")
    w = [oracle.block_quant_weight((torch.randn(n, k, generator=g) * 0.05).bfloat16(), scale_fmt="ue8m0") for _ in counts]
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + len(counts))
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8).cuda()
    b_s = torch.stack([wi[1] for wi in w]).cuda()
    assert bool(((b_s.view(torch.int32) & 0x7FFFFF) == 0).all())
    args = (xq.cuda(), xs.cuda(), None, b, b_s, rows, tg, t0, tr, ops.dtype_code(torch.float32))
    out = torch.ops.dsv3fp8.fp8_gemm_grouped_pow2(*args).cpu()
    gen = torch.ops.dsv3fp8.fp8_gemm_grouped(*args).cpu()
    row = 0
    for gi, c in enumerate(counts):
        if c:
            ref = oracle.fp8_gemm_f32(xq[row:row + c], xs[row:row + c], w[gi][0], w[gi][1])
            rms = ref.pow(2).mean().sqrt().item()
            assert (out[row:row + c] - ref).abs().max().item() <= 1e-2 * rms
            assert (out[row:row + c] - gen[row:row + c]).abs().max().item() <= 1e-4 * rms
        row += c


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_swiglu_quant(K, fmt):
    g = torch.Generator().manual_seed(3)
    rows, inter = 37, 384
    h = (torch.randn(rows, 2 * inter, generator=g) * 2).bfloat16()
    h[0, :inter] = 0                                      # an all-zero block: s = 1e-4/448, y = 0
    h[1, 5] = 60.0                                        # silu saturates to x
    from dsv3fp8 import _lib
    y, s = torch.ops.dsv3fp8.swiglu_quant(h.cuda(), 128, _lib.SCALE_FMT_UE8M0 if fmt else _lib.SCALE_FMT_NONE)
    gref = F.silu(h[:, :inter]) * h[:, inter:]            # bf16 tensor ops, as model.py:633
    yr, sr = oracle.act_quant(gref, 128, fmt)
    assert y.shape == (rows, inter) and s.shape == (rows, inter // 128)
    # exp() of the device and of the CPU may differ in the last place: allow a bf16 ulp of g on a few elements
    same_scale = (s.cpu() == sr).float().mean().item()
    same_code = (y.cpu().view(torch.uint8) == yr.view(torch.uint8)).float().mean().item()
    assert same_scale >= 0.97 and same_code >= 0.995, (same_scale, same_code)
    deq = y.cpu().float() * s.cpu().repeat_interleave(128, 1)
    ref = yr.float() * sr.repeat_interleave(128, 1)
    assert (deq - ref).abs().max().item() <= 0.07 * ref.abs().max().item()
    # against the same chain on the device (same exp): bit-identical
    gd = F.silu(h.cuda()[:, :inter]) * h.cuda()[:, inter:]
    yd, sd = K.act_quant(gd.contiguous(), 128, fmt)
    assert torch.equal(s, sd) and torch.equal(y.view(torch.uint8), yd.view(torch.uint8))


def test_swiglu_quant_every_bf16_value(K):
    """silu over all 65536 bf16 bit patterns (times 1, and times a second factor) against F.silu on the device
    followed by the bf16 product and act_quant: the kernel's exp and division must round to the same bf16."""
    from dsv3fp8 import _lib
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(512, 128)
    x = torch.where(torch.isnan(x), torch.zeros_like(x), x)            # NaN payloads are not compared
    h3 = torch.cat([torch.ones(256, 128), torch.full((256, 128), -0.3359375)]).bfloat16()
    h = torch.cat([x, h3], dim=1).cuda().contiguous()
    y, s = torch.ops.dsv3fp8.swiglu_quant(h, 128, _lib.SCALE_FMT_NONE)
    gd = F.silu(h[:, :128]) * h[:, 128:]
    finite = torch.isfinite(gd).all(dim=1)                              # rows with +-inf quantise to NaN scales
    yd, sd = K.act_quant(gd.contiguous(), 128, None)
    assert finite.sum().item() >= 500
    assert torch.equal(s[finite], sd[finite]) and torch.equal(y.view(torch.uint8)[finite], yd.view(torch.uint8)[finite])


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_swiglu_quant_non_finite(K, fmt):
    """A NaN or an infinity in silu(h1) * h3 reaches the block's scale as it does through act_quant."""
    from dsv3fp8 import _lib
    g = torch.Generator().manual_seed(8)
    h = torch.randn(5, 512, generator=g).bfloat16()
    h[0, 3] = float("nan")                      # h1 of block (0, 0)
    h[1, 256 + 130] = float("inf")              # h3 of block (1, 1)
    h[2, 200] = float("inf")                    # silu(inf) = inf, block (2, 1)
    h[3, 7] = float("-inf")                     # silu(-inf) = -0 / NaN as F.silu gives it
    hc = h.cuda()
    y, s = torch.ops.dsv3fp8.swiglu_quant(hc, 128, _lib.SCALE_FMT_UE8M0 if fmt else _lib.SCALE_FMT_NONE)
    gd = (F.silu(hc[:, :256]) * hc[:, 256:]).contiguous()
    yd, sd = K.act_quant(gd, 128, fmt)
    assert bool(torch.isnan(sd[0, 0])) and bool(torch.isinf(sd[1, 1]))
    assert torch.equal(torch.isnan(s), torch.isnan(sd)) and torch.equal(torch.isinf(s), torch.isinf(sd))
    ok = torch.isfinite(sd)
    assert torch.equal(s[ok], sd[ok])
    yb, ydb = y.view(torch.uint8), yd.view(torch.uint8)
    nan_a, nan_b = (yb & 0x7F) == 0x7F, (ydb & 0x7F) == 0x7F
    assert torch.equal(nan_a, nan_b) and torch.equal(yb[~nan_a], ydb[~nan_a])


@pytest.mark.parametrize("with_shared", [True, False])
def test_moe_combine_bit_exact(K, with_shared):
    g = torch.Generator().manual_seed(4)
    tokens, topk, dim, experts = 33, 4, 264, 9
    scores = torch.rand(tokens, experts, generator=g)
    indices = scores.topk(topk, dim=-1)[1]
    weights = torch.rand(tokens, topk, generator=g).bfloat16()
    flat = indices.reshape(-1)
    order = torch.argsort(flat, stable=True)
    out = torch.randn(tokens * topk, dim, generator=g).bfloat16()       # expert-sorted rows
    z = torch.randn(tokens, dim, generator=g).bfloat16()
    # reference: the loop of model.py:684-693 on the CPU
    y = torch.zeros(tokens, dim, dtype=torch.bfloat16)
    row = 0
    for e in range(experts):
        idx, top = torch.where(indices == e)
        if idx.numel() == 0:
            continue
        y[idx] += out[row:row + idx.numel()] * weights[idx, top, None]
        row += idx.numel()
    ref = y + z if with_shared else y
    slot = indices.argsort(dim=1)
    pos = torch.empty_like(order)
    pos[order] = torch.arange(tokens * topk)
    rows = pos.view(tokens, topk).gather(1, slot).to(torch.int32)
    got = torch.ops.dsv3fp8.moe_combine(out.cuda(), rows.cuda(), weights.gather(1, slot).contiguous().cuda(),
                                        z.cuda() if with_shared else None)
    assert torch.equal(got.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("tokens", [300, 1, 3])           # 1 and 3 tokens: the weight-streaming grouped kernel
def test_moe_grouped_matches_expert_loop_and_oracle(K, tokens):
    from dsv3fp8 import model as M
    old = (M.gemm_impl, torch.get_default_dtype(), M.Linear.dtype)
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype = FP8
    M.gemm_impl = "fp8"
    try:
        args = M.ModelArgs(dim=256, inter_dim=512, moe_inter_dim=128, n_routed_experts=8, n_shared_experts=1,
                           n_activated_experts=2, n_expert_groups=2, n_limited_groups=1, route_scale=2.5)
        with torch.device("cuda"):
            moe = M.MoE(args)
        g = torch.Generator().manual_seed(5)
        with torch.no_grad():
            moe.gate.weight.copy_((torch.randn(8, 256, generator=g) * 0.05).bfloat16().cuda())
        experts = []

        def fill(lin, seed):
            gg = torch.Generator().manual_seed(seed)
            w8, s = oracle.block_quant_weight((torch.randn(lin.out_features, lin.in_features, generator=gg) * 0.05).bfloat16())
            with torch.no_grad():
                lin.weight.copy_(w8.cuda()); lin.scale.copy_(s.cuda())
            return w8, s
        for i, ex in enumerate(moe.experts):
            w1, s1 = fill(ex.w1, 10 + 3 * i); w2, s2 = fill(ex.w2, 11 + 3 * i); w3, s3 = fill(ex.w3, 12 + 3 * i)
            experts.append((w1, s1, w2, s2, w3, s3))
        sh = moe.shared_experts
        shared = (*fill(sh.w1, 90), *fill(sh.w2, 91), *fill(sh.w3, 92))
        x = torch.randn(tokens, 256, generator=g).bfloat16()
        with torch.inference_mode():
            M.MoE.grouped = True
            y_grouped = moe(x.cuda())                   # 300 tokens: the shared expert rides along as group 8
            assert moe._stacked is not None and moe.experts[3].w1.weight.data_ptr() == moe._stacked[0][3].data_ptr()
            assert moe._shared_stacked and moe.shared_experts.w2.weight.data_ptr() == moe._stacked[2][8].data_ptr()
            moe.fuse_swiglu_epilogue = False            # SwiGLU + act_quant as a kernel of their own: the same bits
            assert torch.equal(moe(x.cuda()), y_grouped)
            del moe.fuse_swiglu_epilogue
            moe.fold_shared_max_tokens = 0              # the shared expert as three dense linears instead
            y_unfolded = moe(x.cuda())
            del moe.fold_shared_max_tokens
            assert (y_grouped.float() - y_unfolded.float()).abs().max().item() <= 2e-2 * y_unfolded.float().pow(2).mean().sqrt().item()
            M.MoE.grouped = False
            y_loop = moe(x.cuda())                      # the reference's loop on the (now stacked) expert weights
            wts, idx = moe.gate(x.cuda())
        ref = oracle.moe(x, wts.cpu(), idx.cpu(), experts, shared)
        rms = ref.float().pow(2).mean().sqrt().item()
        # same kernels' arithmetic up to the GEMM's summation order: a bf16 ulp here and there
        assert (y_grouped.float() - y_loop.float()).abs().max().item() <= 3e-2 * rms
        assert (y_grouped.float().cpu() - ref.float()).abs().max().item() <= 5e-2 * rms + 2 ** -8 * ref.abs().max().item()
    finally:
        M.MoE.grouped = True
        M.gemm_impl, M.Linear.dtype = old[0], old[2]
        torch.set_default_dtype(old[1])


def test_moe_layer_with_power_of_two_scales(K, monkeypatch):
    """scale_fmt "ue8m0" on experts whose block scales are powers of two: the grouped GEMMs take the entry point that
    hands the scales to the matrix instruction, and the layer still agrees with the oracle's expert loop."""
    from dsv3fp8 import model as M
    old = (M.gemm_impl, torch.get_default_dtype(), M.Linear.dtype, M.Linear.scale_fmt)
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype, M.gemm_impl, M.Linear.scale_fmt = FP8, "fp8", "ue8m0"
    try:
        args = M.ModelArgs(dim=256, inter_dim=512, moe_inter_dim=128, n_routed_experts=8, n_shared_experts=1,
                           n_activated_experts=2, n_expert_groups=2, n_limited_groups=1, route_scale=2.5)
        with torch.device("cuda"):
            moe = M.MoE(args)
        g = torch.Generator().manual_seed(6)
        with torch.no_grad():
            moe.gate.weight.copy_((torch.randn(8, 256, generator=g) * 0.05).bfloat16().cuda())

        def fill(lin, seed, fmt):
            gg = torch.Generator().manual_seed(seed)
            w8, s = oracle.block_quant_weight((torch.randn(lin.out_features, lin.in_features, generator=gg) * 0.05).bfloat16(),
                                              scale_fmt=fmt)
            with torch.no_grad():
                lin.weight.copy_(w8.cuda()); lin.scale.copy_(s.cuda())
            return w8, s
        experts = []
        for i, ex in enumerate(moe.experts):
            w1, s1 = fill(ex.w1, 10 + 3 * i, "ue8m0"); w2, s2 = fill(ex.w2, 11 + 3 * i, "ue8m0"); w3, s3 = fill(ex.w3, 12 + 3 * i, "ue8m0")
            experts.append((w1, s1, w2, s2, w3, s3))
        sh = moe.shared_experts
        shared = (*fill(sh.w1, 90, "ue8m0"), *fill(sh.w2, 91, "ue8m0"), *fill(sh.w3, 92, "ue8m0"))
        calls = []
        real = torch.ops.dsv3fp8.fp8_gemm_grouped_pow2

        class Spy:
            def __call__(self, *a):
                calls.append(a[5])
                return real(*a)
        monkeypatch.setattr(M.torch.ops.dsv3fp8, "fp8_gemm_grouped_pow2", Spy(), raising=False)
        x = torch.randn(600, 256, generator=g).bfloat16()
        with torch.inference_mode():
            y = moe(x.cuda())
            wts, idx = moe.gate(x.cuda())
        assert calls == [1200, 1200]                      # 600 tokens x 2 experts, both grouped GEMMs
        ref = oracle.moe(x, wts.cpu(), idx.cpu(), experts, shared, scale_fmt="ue8m0")
        rms = ref.float().pow(2).mean().sqrt().item()
        assert (y.float().cpu() - ref.float()).abs().max().item() <= 5e-2 * rms + 2 ** -8 * ref.abs().max().item()
    finally:
        M.gemm_impl, M.Linear.dtype, M.Linear.scale_fmt = old[0], old[2], old[3]
        torch.set_default_dtype(old[1])


@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("tokens,topk,experts", [(300, 2, 8), (4096, 8, 256), (1, 4, 16), (33, 1, 5), (256, 8, 256),
                                                 (257, 8, 256), (50, 4, 700), (1000, 3, 700)])   # 700: three scan batches
def test_moe_route(K, tokens, topk, experts, shared):
    """Both routes of the bookkeeping (one workgroup up to 256 tokens, four kernels above), with and without the
    extra group that every token selects last with weight 1."""
    from dsv3fp8 import ops
    g = torch.Generator().manual_seed(7)
    scores = torch.rand(tokens, experts, generator=g)
    scores[:, experts // 2] += 0.3 * (torch.arange(tokens) % 3 == 0)            # a popular expert
    indices = scores.topk(topk, dim=-1)[1]
    weights = torch.rand(tokens, topk, generator=g).bfloat16()
    counts, a_rows, rows, w_sorted, tg, t0, tr = torch.ops.dsv3fp8.moe_route(indices.cuda(), weights.cuda(), experts, shared)
    counts, a_rows, rows, w_sorted = counts.cpu(), a_rows.cpu(), rows.cpu(), w_sorted.cpu()
    if shared:                                                                   # the reference view of the same thing
        indices = torch.cat([indices, torch.full((tokens, 1), experts)], dim=1)
        weights = torch.cat([weights, torch.ones(tokens, 1, dtype=torch.bfloat16)], dim=1)
        experts, topk = experts + 1, topk + 1
    ref_counts = torch.bincount(indices.flatten(), minlength=experts)
    assert torch.equal(counts.long(), ref_counts)
    offsets = torch.cumsum(ref_counts, 0) - ref_counts
    pairs = tokens * topk
    assert rows.shape == (tokens, topk) and a_rows.numel() == pairs
    assert sorted(rows.flatten().tolist()) == list(range(pairs))               # every row used exactly once
    for e in range(experts):                                                    # group e = the tokens that chose e
        grp = a_rows[offsets[e]:offsets[e] + ref_counts[e]].long()
        assert torch.equal(grp.sort()[0], torch.where((indices == e).any(-1))[0])
    if shared:                                                                   # the extra group is in token order
        assert torch.equal(a_rows[offsets[-1]:].long(), torch.arange(tokens))
    order = indices.argsort(dim=1)
    se = indices.gather(1, order)
    assert torch.equal(w_sorted.view(torch.int16), weights.gather(1, order).view(torch.int16))
    for j in range(topk):                                                       # rows[t, j] lies in the group of the j-th smallest expert
        r = rows[:, j].long()
        assert torch.equal(a_rows[r].long(), torch.arange(tokens))
        assert ((r >= offsets[se[:, j]]) & (r < offsets[se[:, j]] + ref_counts[se[:, j]])).all()
    # the tile table covers every group's rows in order
    R = ops.grouped_tile_rows()
    exp = [(e, int(offsets[e]) + i, min(R, int(ref_counts[e]) - i)) for e in range(experts) for i in range(0, int(ref_counts[e]), R)]
    got = list(zip(tg.tolist(), t0.tolist(), tr.tolist()))
    assert got[:len(exp)] == exp and all(x[0] == -1 for x in got[len(exp):])


def test_moe_forward_is_graph_capturable(K):
    """The grouped path issues no host synchronisation (the reference's loop needs bincount(...).tolist()): one
    forward can be captured in a HIP graph and replayed, with eager work between the replays."""
    from dsv3fp8 import model as M
    old = (M.gemm_impl, torch.get_default_dtype(), M.Linear.dtype)
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype = FP8
    M.gemm_impl = "fp8"
    try:
        args = M.ModelArgs(dim=256, inter_dim=512, moe_inter_dim=128, n_routed_experts=8, n_shared_experts=1,
                           n_activated_experts=2, n_expert_groups=2, n_limited_groups=1, route_scale=2.5)
        with torch.device("cuda"):
            moe = M.MoE(args)
        g = torch.Generator(device="cuda").manual_seed(11)
        with torch.no_grad():
            moe.gate.weight.copy_(torch.randn(8, 256, generator=g, device="cuda") * 0.05)
            for lin in [l for ex in list(moe.experts) + [moe.shared_experts] for l in (ex.w1, ex.w2, ex.w3)]:
                w8, s = oracle.block_quant_weight((torch.randn(lin.out_features, lin.in_features) * 0.05).bfloat16())
                lin.weight.copy_(w8.cuda()); lin.scale.copy_(s.cuda())
        moe.stack_experts()
        x = torch.randn(200, 256, generator=g, device="cuda").bfloat16()
        static_x = x.clone()
        with torch.inference_mode():
            eager = moe(x).clone()
            moe(static_x)                                   # warm-up outside capture (workspaces, attributes)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = moe(static_x)
            for rep in range(3):
                x2 = torch.randn(200, 256, generator=g, device="cuda").bfloat16() if rep else x
                static_x.copy_(x2)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, moe(x2)), rep      # eager work between replays, every replay checked
        assert torch.equal(eager, moe(x))
    finally:
        M.gemm_impl, M.Linear.dtype = old[0], old[2]
        torch.set_default_dtype(old[1])


# ---- the mixture-of-experts configuration at its full dimensions (256 + 1 experts, 7168 -> 2048 -> 7168, 4096 tokens)

@pytest.mark.parametrize("k,n", [(7168, 4096), (2048, 7168)])        # w1|w3 stacked and w2 of one expert
def test_fp8_gemm_grouped_tile_kernel_full_dimensions(K, k, n):
    """The grouped TILE kernel (more than 320 rows in all) on the two GEMM shapes of the layer: groups of about 128
    rows, one of 1093 rows (five tile slots), an empty one and a 131- and a 200-row one (the 192-row
    configuration).  The oracle evaluates sampled groups on sampled rows and whole 128-column blocks."""
    from dsv3fp8 import ops, workloads
    counts = [128, 97, 161, 0, 1093, 131, 200, 128, 3, 140]
    rows, groups = sum(counts), len(counts)
    gen = torch.Generator(device="cuda").manual_seed(k)
    x = torch.randn(rows + 5, k, generator=gen, device="cuda").bfloat16()
    xq, xs = K.act_quant(x)
    a_rows = torch.randint(0, rows + 5, (rows,), generator=gen, device="cuda", dtype=torch.int32)
    w = [workloads.weight(n, k, seed=100 + g, device="cuda") for g in range(groups)]
    b = torch.stack([wi[0].view(torch.uint8) for wi in w]).view(FP8)
    b_s = torch.stack([wi[1] for wi in w])
    R, tg, t0, tr = _tables(counts, rows // ops.grouped_tile_rows() + groups)
    out32 = torch.ops.dsv3fp8.fp8_gemm_grouped(xq, xs, a_rows, b, b_s, rows, tg, t0, tr, ops.dtype_code(torch.float32))
    out16 = torch.ops.dsv3fp8.fp8_gemm_grouped(xq, xs, a_rows, b, b_s, rows, tg, t0, tr, ops.dtype_code(torch.bfloat16))
    assert torch.equal(out16.float(), out32.bfloat16().float())
    assert torch.isfinite(out32).all()
    starts = [sum(counts[:g]) for g in range(groups)]
    blocks = [0, n // 256, n // 128 - 1]
    for g in (0, 2, 4, 5, 6, 8):
        c, r0 = counts[g], starts[g]
        pick = torch.unique(torch.cat([torch.arange(0, c, max(1, c // 24)), torch.tensor([c - 1])]))
        idx = a_rows[r0 + pick.cuda()].long()
        for blk in blocks:
            ref = oracle.fp8_gemm_f32(xq[idx].cpu(), xs[idx].cpu(), w[g][0][blk * 128:(blk + 1) * 128].cpu(),
                                      w[g][1][blk:blk + 1].cpu())
            got = out32[r0 + pick.cuda()][:, blk * 128:(blk + 1) * 128].cpu()
            err = (got - ref).abs().max().item()
            assert err <= 1e-2 * ref.pow(2).mean().sqrt().item(), (g, blk, err)


def test_moe_layer_full_configuration(K):
    """MoE.forward at the benchmark's dimensions: 256 routed + 1 shared expert, 7168 -> 2048 -> 7168, 4096 tokens,
    8 groups / top-4 groups / top-8 experts.  Expert e holds one of four seeded prototype weights with its scales
    multiplied by 1 + e/512, so every expert computes something else.  oracle.moe evaluates a sample of tokens (only
    the experts those tokens select are brought to the CPU); on the whole output: finite, and permuting the tokens
    permutes the output bit for bit (a token's arithmetic does not depend on where it sits in its expert's list)."""
    from dsv3fp8 import model as M, workloads
    old = (M.gemm_impl, torch.get_default_dtype(), M.Linear.dtype)
    torch.set_default_dtype(torch.bfloat16)
    M.Linear.dtype, M.gemm_impl = FP8, "fp8"
    try:
        args = M.ModelArgs()
        assert (args.n_routed_experts, args.dim, args.moe_inter_dim, args.n_activated_experts) == (256, 7168, 2048, 8)
        with torch.device("cuda"):
            moe = M.MoE(args)
        g = torch.Generator(device="cuda").manual_seed(5)
        protos = [(workloads.weight(args.moe_inter_dim, args.dim, 40 + i, "cuda"),
                   workloads.weight(args.dim, args.moe_inter_dim, 50 + i, "cuda"),
                   workloads.weight(args.moe_inter_dim, args.dim, 60 + i, "cuda")) for i in range(4)]
        with torch.no_grad():
            moe.gate.weight.copy_(torch.randn(args.n_routed_experts, args.dim, generator=g, device="cuda") * 0.02)
            moe.gate.bias.copy_(torch.randn(args.n_routed_experts, generator=g, device="cuda") * 0.02)
            for e, ex in enumerate(list(moe.experts) + [moe.shared_experts]):
                p1, p2, p3 = protos[e % 4]
                f = 1.0 + e / 512.0
                for lin, (w8, sc) in ((ex.w1, p1), (ex.w2, p2), (ex.w3, p3)):
                    lin.weight.copy_(w8)
                    lin.scale.copy_(sc * f)
        moe.stack_experts()
        tokens = 4096
        x = workloads.activations(tokens, args.dim, 6, "cuda")
        perm = torch.randperm(tokens, generator=g, device="cuda")
        with torch.inference_mode():
            y = moe(x)
            y_perm = moe(x[perm].contiguous())
            wts, idx = moe.gate(x)
        assert y.shape == x.shape and torch.isfinite(y.float()).all()
        assert torch.equal(y_perm.view(torch.int16), y[perm].view(torch.int16))
        counts = torch.bincount(idx.flatten(), minlength=args.n_routed_experts)
        assert int(counts.sum()) == tokens * 8 and int((counts > 0).sum()) > 200
        # sampled tokens, chosen greedily so that together they select many different experts: every new token adds
        # as many experts not seen so far as possible
        idx_cpu = idx.cpu()
        sample, hit = [0, 1777, 4095], set(idx_cpu[[0, 1777, 4095]].flatten().tolist())
        cand = torch.randperm(tokens, generator=torch.Generator().manual_seed(7))[:600].tolist()
        while len(sample) < 24:
            best = max(cand, key=lambda t: len(set(idx_cpu[t].tolist()) - hit))
            cand.remove(best)
            sample.append(best)
            hit |= set(idx_cpu[best].tolist())
        assert len(hit) >= 64, len(hit)
        sample = torch.tensor(sample)

        def cpu(ex):
            return tuple(t.data.cpu() for lin in (ex.w1, ex.w2, ex.w3) for t in (lin.weight, lin.scale))
        experts = [cpu(ex) if e in hit else None for e, ex in enumerate(moe.experts)]
        ref = oracle.moe(x[sample.cuda()].cpu(), wts[sample.cuda()].cpu(), idx_cpu[sample], experts,
                         cpu(moe.shared_experts))
        rms = ref.float().pow(2).mean().sqrt().item()
        err = (y[sample.cuda()].float().cpu() - ref.float()).abs().max().item()
        assert err <= 5e-2 * rms + 2 ** -8 * ref.abs().max().item(), (err, rms)

        # the first grouped GEMM by itself, expert by expert: the rows of a sampled expert against the oracle's
        # fp8_gemm with THAT expert's w1 | w3 (and scales), on the expert's own token list
        from dsv3fp8 import ops
        with torch.inference_mode():
            route = torch.ops.dsv3fp8.moe_route(idx.contiguous(), wts.contiguous(), args.n_routed_experts, False)
            _, a_rows, rows, _, tile_group, tile_row0, tile_rows = route
            xq, xs = K.act_quant(x)
            w13, s13 = (t[:args.n_routed_experts] for t in moe._stacked[:2])
            h = torch.ops.dsv3fp8.fp8_gemm_grouped(xq, xs, a_rows, w13, s13, rows.numel(), tile_group, tile_row0,
                                                   tile_rows, ops.dtype_code(torch.float32))
        starts = torch.cumsum(counts, 0) - counts
        inter = args.moe_inter_dim
        checked = 0
        for e in sorted(hit)[::3]:                               # every third of the sampled experts (>= 21 of them)
            c, r0 = int(counts[e]), int(starts[e])
            pick = torch.unique(torch.tensor([0, c // 2, c - 1])) + r0
            toks = a_rows[pick.cuda()].long()
            assert bool((idx[toks] == e).any(dim=1).all())       # the list holds tokens that selected expert e
            w1, s1, _, _, w3, s3 = experts[e]
            for half, (w8, sc) in enumerate(((w1, s1), (w3, s3))):
                ref_h = oracle.fp8_gemm_f32(xq[toks].cpu(), xs[toks].cpu(), w8[:256], sc[:2])
                got_h = h[pick.cuda()][:, half * inter: half * inter + 256].cpu()
                err_h = (got_h - ref_h).abs().max().item()
                assert err_h <= 1e-2 * ref_h.pow(2).mean().sqrt().item(), (e, half, err_h)
            checked += 1
        assert checked >= 21
    finally:
        M.gemm_impl, M.Linear.dtype = old[0], old[2]
        torch.set_default_dtype(old[1])
