"""GPU parity: fp8_gemm through the C ABI vs the fp32 CPU oracle
(reference arithmetic: inference/kernel.py:145-172).

Tolerance: max|err| <= 1e-2 * rms(ref) on the binary32 accumulator output; the
bf16 output must equal the round-to-nearest-even bf16 of the kernel's own
binary32 output bit for bit (half a bf16 ulp at the output tail is larger than
the tolerance, so the bf16 tensor is not compared with the fp32 reference)."""
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def K():
    import dsv3fp8
    return dsv3fp8


def _gemm_both(K, a, a_s, b, b_s):
    c32 = K.fp8_gemm_f32(a, a_s, b, b_s)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        c16 = K.fp8_gemm(a, a_s, b, b_s)
    finally:
        torch.set_default_dtype(old)
    return c32, c16


def _check(K, x, w8, ws, fmt=None):
    a_ref, as_ref = oracle.act_quant(x, 128, fmt)
    ref = oracle.fp8_gemm_f32(a_ref, as_ref, w8, ws)
    a, a_s = a_ref.cuda(), as_ref.cuda()
    c32, c16 = _gemm_both(K, a, a_s, w8.cuda(), ws.cuda())
    assert c32.dtype == torch.float32 and c16.dtype == torch.bfloat16
    assert c32.shape == ref.shape == c16.shape
    rms = ref.pow(2).mean().sqrt().item()
    err = (c32.cpu() - ref).abs().max().item()
    assert err <= TOL * rms, f"max|err| {err:.3e} > {TOL} * rms {rms:.3e}"
    assert torch.equal(c16.cpu().view(torch.int16), c32.cpu().to(torch.bfloat16).view(torch.int16))
    return err / rms


# the five attention projections (inference/model.py:427-433) and wq_a | wkv_a stacked into one 7168 -> 2112 weight
DECODE = [(7168, 1536), (1536, 24576), (7168, 576), (512, 32768), (16384, 7168), (7168, 2112)]


@pytest.mark.parametrize("kn", DECODE)
@pytest.mark.parametrize("m", [1, 8, 32, 64])
def test_decode_shapes(K, kn, m):
    from dsv3fp8 import workloads
    k, n = kn
    x = workloads.activations(m, k, seed=m)
    w8, ws = workloads.weight(n, k, seed=n % 97)
    _check(K, x, w8, ws)


@pytest.mark.parametrize("m,k,n", [
    (3, 7168, 1536), (12, 7168, 1536), (16, 7168, 2112),   # one sub-tile, chunks of eight K blocks, 7 K slices
    (5, 7168, 576),                                        # 9 groups: stays with the M <= 16 kernel
    (12, 1536, 24576), (16, 1536, 24576),                  # K = 12 blocks: two sub-tiles, the second padding
    (16, 512, 32768), (17, 512, 32768), (40, 512, 32768),  # K = 512: one ring round, 1 / 2 / 4 (for 3) sub-tiles
    (17, 16384, 7168), (32, 16384, 7168),                  # a 117 MB weight of 7168 rows: four consumers, 2 K slices
    (33, 16384, 7168),                                     # ... and the large-M kernel with K slices from 33 rows
    (20, 1024, 8192 + 48), (64, 2048, 1000),               # ragged N on both consumer counts
])
def test_few_rows_on_every_streaming_plan(K, m, k, n):
    """3 .. 64 rows: the activation-streaming kernel's plans (sub-tile counts, consumer counts, K slices with the
    reduce pass, padded sub-tiles) and its neighbours in the dispatcher, each against the oracle."""
    from dsv3fp8 import workloads
    x = workloads.activations(m, k, seed=m + k % 11)
    w8, ws = workloads.weight(n, k, seed=n % 89)
    _check(K, x, w8, ws)


@pytest.mark.parametrize("m", [65, 100, 128, 257, 300])
def test_mid_m(K, m):
    from dsv3fp8 import workloads
    x = workloads.activations(m, 1024, seed=m)
    w8, ws = workloads.weight(640, 1024, seed=3)
    _check(K, x, w8, ws)


@pytest.mark.parametrize("m,n,k", [
    (100, 300, 128),      # one K block: the pipeline's prologue and clamped refills only (short tiles, 3 LDS stages)
    (130, 256, 256),      # two K blocks, two short row tiles, the second with 2 rows
    (2048, 8192, 128),    # one full round of tall tiles (256 rows, 2 LDS stages), one K block
    (2050, 8192, 384),    # tall tiles with a 2-row edge tile, odd number of K blocks
    (1024, 18432, 256),   # short tiles chosen for a large problem (3 rounds of short beat 2 of tall)
])
def test_large_m_tile_heights_and_short_k(K, m, n, k):
    from dsv3fp8 import workloads
    x = workloads.activations(m, k, seed=m)
    w8, ws = workloads.weight(n, k, seed=n % 89)
    _check(K, x, w8, ws)


@pytest.mark.parametrize("m,n,k", [
    (100, 577, 7168),     # 3 tiles: the K range is cut into 7 slices of 8 blocks; ragged N
    (130, 4096, 2048),    # two row tiles (one with 2 rows), 2 slices of 8 blocks
    (128, 18432, 7168),   # 72 tiles, 3 slices of 19 + 19 + 18 blocks
    (257, 7168, 18432),   # 84 tiles, 3 slices of 48 blocks
    (65, 1536, 1152),     # 9 K blocks: too short to cut, one slice
])
def test_mid_m_split_over_k(K, m, n, k):
    """Between 65 and a few hundred rows the large-M kernel cuts the K range into slices run by separate
    workgroups (binary32 partial sums, added in a fixed order by a second kernel)."""
    from dsv3fp8 import workloads, _lib
    x = workloads.activations(m, k, seed=m)
    w8, ws = workloads.weight(n, k, seed=n % 89)
    _check(K, x, w8, ws)
    if k >= 2048:
        assert _lib.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k) >= 2 * m * n * 4


@pytest.mark.parametrize("n", [1, 15, 16, 100, 129, 576, 577, 1000])
def test_ragged_n(K, n):
    from dsv3fp8 import workloads
    for m in (5, 130):
        x = workloads.activations(m, 512, seed=n)
        w8, ws = workloads.weight(n, 512, seed=n + 1)
        _check(K, x, w8, ws)


@pytest.mark.parametrize("mnk", [(3, 5, 1), (2, 130, 127), (4, 7, 129), (70, 200, 300), (1, 576, 7168 + 64),
                                 (5, 1000, 200)])
def test_k_not_a_multiple_of_128(K, mnk):
    """The reference's kernel masks a last, partial K block (inference/kernel.py:145, 158-159; its act_quant cannot
    produce one, kernel.py:52): scale tensors of ceil(k / 128) columns, the tail zero-filled.  Against the oracle, and
    against the same problem padded with zero bytes to the next multiple of 128, which runs the regular kernels."""
    m, n, k = mnk
    g = torch.Generator().manual_seed(k)
    kb = -(-k // 128)
    a = torch.randn(m, k, generator=g).to(torch.float8_e4m3fn)
    b = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    a_s = torch.rand(m, kb, generator=g) * 0.1 + 0.01
    b_s = torch.rand(-(-n // 128), kb, generator=g) * 0.1 + 0.01
    ref = oracle.fp8_gemm_f32(a, a_s, b, b_s)
    c32, c16 = _gemm_both(K, a.cuda(), a_s.cuda(), b.cuda(), b_s.cuda())
    rms = ref.pow(2).mean().sqrt().item()
    assert (c32.cpu() - ref).abs().max().item() <= TOL * rms
    assert torch.equal(c16.cpu().view(torch.int16), c32.cpu().to(torch.bfloat16).view(torch.int16))
    kp = kb * 128
    ap = torch.zeros(m, kp, dtype=torch.uint8); ap[:, :k] = a.view(torch.uint8)
    bp = torch.zeros(n, kp, dtype=torch.uint8); bp[:, :k] = b.view(torch.uint8)
    padded = K.fp8_gemm_f32(ap.view(torch.float8_e4m3fn).cuda(), a_s.cuda(), bp.view(torch.float8_e4m3fn).cuda(), b_s.cuda())
    assert (c32 - padded).abs().max().item() <= 1e-3 * rms          # two binary32 summation orders of the same products


def test_ragged_n_equals_prefix_of_padded(K):
    """N=576 must equal the first 576 columns of the N=640 problem built from the same rows."""
    from dsv3fp8 import workloads
    x = workloads.activations(64, 7168, seed=1)
    w8, ws = workloads.weight(640, 7168, seed=2)
    a, a_s = oracle.act_quant(x)
    a, a_s = a.cuda(), a_s.cuda()
    full = K.fp8_gemm_f32(a, a_s, w8.cuda(), ws.cuda())
    part = K.fp8_gemm_f32(a, a_s, w8[:576].contiguous().cuda(), ws.cuda())
    assert torch.equal(full[:, :576], part)


def test_leading_dims(K):
    from dsv3fp8 import workloads
    x = workloads.activations(6, 256, seed=1).view(2, 3, 256)
    w8, ws = workloads.weight(192, 256, seed=2)
    _check(K, x, w8, ws)


def test_ue8m0_activation_scales(K):
    from dsv3fp8 import workloads
    x = workloads.activations(48, 2048, seed=8, outliers=True)
    w8, ws = workloads.weight(2048, 2048, seed=9)
    _check(K, x, w8, ws, fmt="ue8m0")


def test_exact_small_integers(K):
    """Small-integer fp8 values and power-of-two scales: every partial sum is exact in
    binary32, so the result is independent of summation order -> bit-exact."""
    g = torch.Generator().manual_seed(0)
    for (m, n, k) in [(3, 130, 256), (64, 256, 1024), (200, 384, 512)]:
        a = torch.randint(-4, 5, (m, k), generator=g).float().to(torch.float8_e4m3fn)
        b = torch.randint(-4, 5, (n, k), generator=g).float().to(torch.float8_e4m3fn)
        a_s = torch.pow(2.0, torch.randint(-3, 4, (m, k // 128), generator=g).float())
        b_s = torch.pow(2.0, torch.randint(-3, 4, (-(-n // 128), k // 128), generator=g).float())
        ref = oracle.fp8_gemm_f32(a, a_s, b, b_s)
        c32 = K.fp8_gemm_f32(a.cuda(), a_s.cuda(), b.cuda(), b_s.cuda())
        assert torch.equal(c32.cpu(), ref)


def test_one_hot_picks_single_products(K):
    """One-hot activation rows select single weight values times both scales."""
    k, n = 384, 160
    g = torch.Generator().manual_seed(1)
    b = torch.randint(0, 0x7F, (n, k), generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
    b_s = torch.rand(2, 3, generator=g) + 0.5
    a = torch.zeros(16, k)
    cols = torch.randint(0, k, (16,), generator=g)
    a[torch.arange(16), cols] = 2.0
    a = a.to(torch.float8_e4m3fn)
    a_s = torch.rand(16, 3, generator=g) + 0.5
    c = K.fp8_gemm_f32(a.cuda(), a_s.cuda(), b.cuda(), b_s.cuda()).cpu()
    nb = torch.arange(n) // 128
    for i in range(16):
        kb = int(cols[i]) // 128
        want = (2.0 * b.float()[:, cols[i]]) * a_s[i, kb] * b_s[nb, kb]
        assert torch.allclose(c[i], want, rtol=3e-7, atol=0)


def test_prefill_sampled(K):
    """M=4096, 7168 -> 18432 at full size; the oracle evaluates a sample of rows/columns."""
    from dsv3fp8 import workloads
    x = workloads.activations(4096, 7168, seed=0, device="cuda")
    w8, ws = workloads.weight(18432, 7168, seed=1, device="cuda")
    a, a_s = K.act_quant(x)
    c32, c16 = _gemm_both(K, a, a_s, w8, ws)
    rows = torch.arange(5, 4096, 97, device="cuda")
    cols = torch.cat([torch.arange(0, 256), torch.arange(9000, 9300), torch.arange(18432 - 200, 18432)]).cuda()
    # the oracle needs whole 128-row scale blocks of b: evaluate per 128-aligned column block
    ref_cols = []
    for blk in torch.unique(cols // 128).tolist():
        ref_cols.append(oracle.fp8_gemm_f32(a[rows].cpu(), a_s[rows].cpu(),
                                            w8[blk * 128:(blk + 1) * 128].cpu(), ws[blk:blk + 1].cpu()))
    ref = torch.cat(ref_cols, 1)
    colidx = torch.cat([torch.arange(b * 128, (b + 1) * 128) for b in torch.unique(cols // 128).tolist()]).cuda()
    got = c32[rows][:, colidx].cpu()
    rms = ref.pow(2).mean().sqrt().item()
    assert (got - ref).abs().max().item() <= TOL * rms
    assert torch.equal(c16.view(torch.int16), c32.to(torch.bfloat16).view(torch.int16))


def _sampled_reference(a, a_s, w8, ws, rows, col_blocks):
    """oracle.fp8_gemm_f32 on the sampled rows of a and whole 128-row blocks of b (the oracle needs whole scale
    blocks); returns the reference and the column indices it covers."""
    ref = torch.cat([oracle.fp8_gemm_f32(a[rows].cpu(), a_s[rows].cpu(), w8[b * 128:(b + 1) * 128].cpu(),
                                         ws[b:b + 1].cpu()) for b in col_blocks], 1)
    cols = torch.cat([torch.arange(b * 128, (b + 1) * 128) for b in col_blocks])
    return ref, cols


def test_prefill_w2_sampled(K):
    """The second half of the prefill configuration at full size: M=4096, 18432 -> 7168 (448 tall tiles, 1.75
    rounds, 144 K blocks); the oracle evaluates a sample of rows and column blocks."""
    from dsv3fp8 import workloads
    x = workloads.activations(4096, 18432, seed=2, device="cuda")
    w8, ws = workloads.weight(7168, 18432, seed=3, device="cuda")
    a, a_s = K.act_quant(x)
    c32, c16 = _gemm_both(K, a, a_s, w8, ws)
    rows = torch.cat([torch.arange(3, 4096, 211), torch.tensor([0, 255, 256, 4095])]).cuda()
    ref, cols = _sampled_reference(a, a_s, w8, ws, rows, [0, 1, 27, 28, 55])
    got = c32[rows][:, cols.cuda()].cpu()
    rms = ref.pow(2).mean().sqrt().item()
    assert (got - ref).abs().max().item() <= TOL * rms
    assert torch.equal(c16.view(torch.int16), c32.to(torch.bfloat16).view(torch.int16))


@pytest.mark.parametrize("m,k,n", [
    (4096, 512, 32768),     # 16 x 128 tiles of 4 K blocks: 8 tiles per workgroup, every block of a tile is one of its "last two"
    (2048, 1536, 12288),    # 8 x 48 = 384 tiles of 12 blocks: half of the workgroups compute two tiles, the others one
    (1280, 4096, 16384),    # 5 x 64 = 320 tiles of 32 blocks (the longest K range that takes this route)
])
def test_several_tiles_per_workgroup(K, m, k, n):
    """Whole 256 x 256 tiles in more than one round with a short K range: the 16-bit product runs in workgroups that
    compute their tiles one after the other (the last K blocks of a tile request the first copies of the next one), the
    binary32 product of the same call one tile per workgroup; the oracle evaluates a sample, and the bf16 result
    must be the rounding of the binary32 one bit for bit."""
    from dsv3fp8 import workloads
    x = workloads.activations(m, k, seed=m % 97, device="cuda")
    w8, ws = workloads.weight(n, k, seed=n % 89, device="cuda")
    a, a_s = K.act_quant(x)
    c32, c16 = _gemm_both(K, a, a_s, w8, ws)
    rows = torch.cat([torch.arange(5, m, 97), torch.tensor([0, 255, 256, m - 1])]).cuda()
    nb = n // 128
    ref, cols = _sampled_reference(a, a_s, w8, ws, rows, [0, 1, 2, nb // 2, nb - 2, nb - 1])
    got = c32[rows][:, cols.cuda()].cpu()
    rms = ref.pow(2).mean().sqrt().item()
    assert (got - ref).abs().max().item() <= TOL * rms
    assert torch.equal(c16.view(torch.int16), c32.to(torch.bfloat16).view(torch.int16))
    # fp16 results take the same route
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        h16 = K.fp8_gemm(a, a_s, w8, ws)
    finally:
        torch.set_default_dtype(old)
    assert torch.equal(h16.view(torch.int16), c32.to(torch.float16).view(torch.int16))


def test_every_kernel_family_replays_in_a_graph(K):
    """act_quant + fp8_gemm over shapes that take every family of GEMM kernels (one- and two-row kernel with and
    without K slices, activation-streaming kernel, one group of the grouped few-row kernel, K-sliced mid-M tiles,
    two tile heights in one launch, several tiles per workgroup) captured in one HIP graph: three replays with
    fresh activations and eager work between them, each compared with the eager result bit for bit."""
    from dsv3fp8 import workloads
    shapes = [(1, 7168, 1536), (2, 1536, 24576), (8, 7168, 2112), (32, 7168, 576), (64, 512, 32768),
              (4, 16384, 7168), (130, 2048, 4096), (1030, 512, 17000), (2048, 512, 12288), (1280, 4096, 16384)]
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        weights = [workloads.weight(n, k, seed=i + 3, device="cuda") for i, (m, k, n) in enumerate(shapes)]
        xs = [workloads.activations(m, k, seed=i, device="cuda") for i, (m, k, n) in enumerate(shapes)]

        def run():
            return [K.fp8_gemm(*K.act_quant(x), w8, ws) for x, (w8, ws) in zip(xs, weights)]
        run()                                               # warm-up outside capture (attributes, workspaces)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = run()
        for rep in range(3):
            for i, x in enumerate(xs):
                x.copy_(workloads.activations(x.size(0), x.size(1), seed=100 * rep + i, device="cuda"))
            graph.replay()
            torch.cuda.synchronize()
            eager = run()                                   # eager work between the replays
            for i, (g, e) in enumerate(zip(outs, eager)):
                assert torch.equal(g, e), (rep, shapes[i])
    finally:
        torch.set_default_dtype(old)


def test_prefill_pow2_full_size_sampled(K):
    """fp8_gemm_pow2 at M=4096 on both prefill shapes: power-of-two activation scales (ue8m0) and weight block scales
    rounded up to powers of two; sampled against the oracle and held against the general kernel everywhere."""
    from dsv3fp8 import workloads
    for (k, n, blocks) in ((7168, 18432, [0, 70, 143]), (18432, 7168, [0, 31, 55])):
        x = workloads.activations(4096, k, seed=k % 13, device="cuda")
        w8, ws = workloads.weight(n, k, seed=4, device="cuda")
        ws2 = torch.pow(2.0, torch.ceil(torch.log2(ws)))            # the bytes stay, the scales move up to 2^e
        a, a_s = K.act_quant(x, 128, "ue8m0")
        old = torch.get_default_dtype()
        try:
            torch.set_default_dtype(torch.float32)
            c32 = K.fp8_gemm_pow2(a, a_s, w8, ws2)
            gen = K.fp8_gemm(a, a_s, w8, ws2)
            torch.set_default_dtype(torch.bfloat16)
            c16 = K.fp8_gemm_pow2(a, a_s, w8, ws2)
        finally:
            torch.set_default_dtype(old)
        rows = torch.arange(7, 4096, 307).cuda()
        ref, cols = _sampled_reference(a, a_s, w8, ws2, rows, blocks)
        rms = ref.pow(2).mean().sqrt().item()
        assert (c32[rows][:, cols.cuda()].cpu() - ref).abs().max().item() <= TOL * rms
        assert (c32 - gen).abs().max().item() <= 1e-4 * rms
        assert torch.equal(c16.view(torch.int16), c32.to(torch.bfloat16).view(torch.int16))


def test_asserts_match_reference(K):
    a = torch.zeros(4, 256, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    a_s = torch.ones(4, 2, device="cuda")
    b = torch.zeros(128, 256, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    b_s = torch.ones(1, 2, device="cuda")
    with pytest.raises(AssertionError):
        K.fp8_gemm(a.t(), a_s, b, b_s)
    with pytest.raises(AssertionError):
        K.fp8_gemm(a, a_s.t(), b, b_s)


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
@pytest.mark.parametrize("m", [1, 3, 8, 16])
def test_fused_linear_equals_act_quant_then_gemm(K, m, fmt):
    """dsv3_linear_fp8 (activation quantisation inside the M <= 16 weight-streaming kernel) against the two separate
    calls on every decode shape: bit for bit wherever fp8_gemm runs the same kernel -- from three rows up the one call
    is only offered there --, and up to the order of the binary32 sums at one and two rows where fp8_gemm streams the
    activations through LDS instead (the quantised bytes and scales are the same; both sides meet the oracle's bar)."""
    from dsv3fp8 import workloads, ops, _lib
    code_fmt = _lib.SCALE_FMT_UE8M0 if fmt == "ue8m0" else _lib.SCALE_FMT_NONE
    for name, (k, n) in workloads.DECODE_SHAPES.items():
        # one call up to 131072 activation elements: always at one and two rows; from three rows up only where
        # fp8_gemm takes its M <= 16 kernel (never on weights of 96 MiB and more, nor where it streams the activations)
        fused = ops.linear_fp8_fused(m, n, k)
        if m <= 2:
            assert fused == (m * k <= 131072), name
        else:
            assert not (fused and (m * k > 131072 or n * k >= 96 << 20)), name
        x = workloads.activations(m, k, seed=m + n % 7, outliers=True).cuda()
        w8, ws = workloads.weight(n, k, seed=3)
        w8, ws = w8.cuda(), ws.cuda()
        a, a_s = K.act_quant(x, 128, fmt)
        for code in (_lib.BF16, _lib.F32):
            two = torch.ops.dsv3fp8.fp8_gemm(a, a_s, w8, ws, code)
            one = torch.ops.dsv3fp8.linear_fp8(x, w8, ws, code_fmt, code)
            assert one.dtype == two.dtype
            if torch.equal(one, two):
                continue
            assert m <= 2, (name, code)                     # (another kernel behind fp8_gemm: sums in another order)
            rms = two.float().pow(2).mean().sqrt().item()
            tol = 1e-3 * rms if code == _lib.F32 else 2.0 ** -7 * two.float().abs().max().item()
            assert (one.float() - two.float()).abs().max().item() <= tol, (name, code)
    # three rows and more where fp8_gemm itself takes the M <= 16 kernel (K below 512): one call, the same bits
    x = workloads.activations(8, 256, seed=4).cuda()
    w8, ws = workloads.weight(4096, 256, seed=5)
    a, a_s = K.act_quant(x, 128, fmt)
    assert ops.linear_fp8_fused(8, 4096, 256)
    assert torch.equal(torch.ops.dsv3fp8.linear_fp8(x, w8.cuda(), ws.cuda(), code_fmt, _lib.F32),
                       torch.ops.dsv3fp8.fp8_gemm(a, a_s, w8.cuda(), ws.cuda(), _lib.F32))
    # rows above the fused kernel's range take the two calls inside the op
    x = workloads.activations(40, 512, seed=1).cuda()
    w8, ws = workloads.weight(256, 512, seed=2)
    a, a_s = K.act_quant(x, 128, fmt)
    assert not ops.linear_fp8_fused(40, 256, 512)
    assert torch.equal(torch.ops.dsv3fp8.linear_fp8(x, w8.cuda(), ws.cuda(), code_fmt, _lib.F32),
                       torch.ops.dsv3fp8.fp8_gemm(a, a_s, w8.cuda(), ws.cuda(), _lib.F32))


@pytest.mark.parametrize("m,n,k,sliced", [
    (1024, 18432, 4096, True),    # 4 x 72 tall tiles: 256 of them as a plain launch, the last 8 column tiles in 4 K slices
    (1030, 17000, 4096, False),   # ragged M and N, 5 x 67 tall tiles: the last column tiles (one of 104 columns) as
                                  # 128-row tiles behind the tall ones, in one launch
    (1280, 18432, 1024, False),   # K too short to slice: 5 x 72 tall tiles, a partly filled second round
    (2100, 9000, 640, False),     # 9 x 36 tall tiles, ragged both ways, odd number of K blocks
])
def test_partly_filled_last_round(K, m, n, k, sliced):
    """Launches of more than one round of tiles whose last round is partly filled: the planner either cuts the K
    range of the remaining column tiles into slices or runs them as short tiles behind the tall ones."""
    from dsv3fp8 import workloads, _lib
    assert (_lib.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k) > 0) == sliced
    x = workloads.activations(m, k, seed=m)
    w8, ws = workloads.weight(n, k, seed=n % 89)
    _check(K, x, w8, ws)


def _pow2_problem(m, n, k, seed):
    """Activations quantised with power-of-two scales (ue8m0) and a weight whose block scales were rounded up to
    powers of two before quantising -- the format of config_v3.1 checkpoints."""
    from dsv3fp8 import workloads
    x = workloads.activations(m, k, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16().float()
    nb, kb = -(-n // 128), k // 128
    wp = torch.zeros(nb * 128, k)
    wp[:n] = w
    amax = wp.view(nb, 128, kb, 128).abs().amax(dim=(1, 3)).clamp_min(1e-4)
    ws = torch.pow(2.0, torch.ceil(torch.log2(amax / 448.0)))
    w8 = (wp.view(nb, 128, kb, 128) / ws[:, None, :, None]).reshape(nb * 128, k)[:n].contiguous().to(torch.float8_e4m3fn)
    a, a_s = oracle.act_quant(x, 128, "ue8m0")
    assert bool(((a_s.view(torch.int32) & 0x7FFFFF) == 0).all()) and bool(((ws.view(torch.int32) & 0x7FFFFF) == 0).all())
    return a, a_s, w8, ws


@pytest.mark.parametrize("m,n,k", [
    (300, 640, 1024),      # short tiles
    (2050, 8192, 384),     # tall tiles, a 2-row edge tile, odd number of K blocks
    (1030, 17000, 512),    # two tile heights in one launch, ragged N
    (130, 4096, 2048),     # K range cut into slices (binary32 slabs)
    (16, 1536, 7168),      # few rows: the same kernels as fp8_gemm
    (2048, 12288, 512),    # 384 whole tall tiles of 4 K blocks: workgroups that compute two tiles in a row (16-bit results)
])
def test_power_of_two_scales_in_the_matrix_instruction(K, m, n, k):
    a, a_s, w8, ws = _pow2_problem(m, n, k, seed=m)
    ref = oracle.fp8_gemm_f32(a, a_s, w8, ws)
    old = torch.get_default_dtype()
    try:
        torch.set_default_dtype(torch.float32)
        c32 = K.fp8_gemm_pow2(a.cuda(), a_s.cuda(), w8.cuda(), ws.cuda())
        gen = K.fp8_gemm(a.cuda(), a_s.cuda(), w8.cuda(), ws.cuda())
        torch.set_default_dtype(torch.bfloat16)
        c16 = K.fp8_gemm_pow2(a.cuda(), a_s.cuda(), w8.cuda(), ws.cuda())
    finally:
        torch.set_default_dtype(old)
    rms = ref.pow(2).mean().sqrt().item()
    assert (c32.cpu() - ref).abs().max().item() <= TOL * rms
    assert (c32 - gen).abs().max().item() <= 1e-4 * rms                  # same products, another order of additions
    assert torch.equal(c16.cpu().view(torch.int16), c32.cpu().to(torch.bfloat16).view(torch.int16))


def test_power_of_two_scales_exact_small_integers(K):
    """Small-integer fp8 values (block sums below 2^11) and power-of-two scales whose products span seven binades
    far from 1: every partial sum fits 24 bits, so the result is independent of the summation order and the scale
    operands must reproduce 2^e exactly."""
    g = torch.Generator().manual_seed(4)
    for (m, n, k) in [(200, 384, 512), (600, 1000, 1280)]:
        a = torch.randint(-4, 5, (m, k), generator=g).float().to(torch.float8_e4m3fn)
        b = torch.randint(-4, 5, (n, k), generator=g).float().to(torch.float8_e4m3fn)
        a_s = torch.pow(2.0, torch.randint(-12, -8, (m, k // 128), generator=g).float())
        b_s = torch.pow(2.0, torch.randint(-10, -6, (-(-n // 128), k // 128), generator=g).float())
        ref = oracle.fp8_gemm_f32(a, a_s, b, b_s)
        old = torch.get_default_dtype()
        torch.set_default_dtype(torch.float32)
        try:
            c32 = K.fp8_gemm_pow2(a.cuda(), a_s.cuda(), b.cuda(), b_s.cuda())
        finally:
            torch.set_default_dtype(old)
        assert torch.equal(c32.cpu(), ref)


def test_seeded_shape_sweep(K):
    """Thirty seeded shapes across the dispatcher's regimes (few rows, mid M with and without K slicing, whole
    rounds, partly filled last rounds, ragged M and N), each against the oracle."""
    from dsv3fp8 import workloads
    g = torch.Generator().manual_seed(2024)

    def pick(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))
    shapes = []
    while len(shapes) < 30:
        m = pick(1, 64) if len(shapes) % 5 == 0 else pick(65, 2600)
        n = pick(1, 300) if len(shapes) % 7 == 0 else pick(256, 9000)
        k = 128 * pick(1, 16)
        if m * n * k <= 1.2e10:
            shapes.append((m, n, k))
    worst = 0.0
    for i, (m, n, k) in enumerate(shapes):
        x = workloads.activations(m, k, seed=100 + i)
        w8, ws = workloads.weight(n, k, seed=200 + i)
        worst = max(worst, _check(K, x, w8, ws))
    assert worst <= TOL


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_fused_linear_non_finite_activations(K, fmt):
    """The quantiser inside dsv3_linear_fp8 forms its scales as act_quant does (a NaN or an infinity in a block reaches
    the scale): rows that hold one come out as NaN in the one call and in the two calls alike, the other rows bit-equal."""
    from dsv3fp8 import workloads, ops, _lib
    code_fmt = _lib.SCALE_FMT_UE8M0 if fmt == "ue8m0" else _lib.SCALE_FMT_NONE
    k, n = 384, 576                             # (four rows run as one call where K is below 512)
    x = workloads.activations(4, k, seed=9)
    x[0, 100] = float("nan")
    x[1, 300] = float("inf")
    x[2, 383] = float("-inf"); x[2, 5] = float("nan")
    assert ops.linear_fp8_fused(4, n, k)
    w8, ws = workloads.weight(n, k, seed=3)
    xc, w8, ws = x.cuda(), w8.cuda(), ws.cuda()
    a, a_s = K.act_quant(xc, 128, fmt)
    two = torch.ops.dsv3fp8.fp8_gemm(a, a_s, w8, ws, _lib.F32)
    one = torch.ops.dsv3fp8.linear_fp8(xc, w8, ws, code_fmt, _lib.F32)
    assert bool(torch.isnan(two[:3]).all()) and bool(torch.isfinite(two[3]).all())
    assert torch.equal(torch.isnan(one), torch.isnan(two))
    assert torch.equal(one[3], two[3])


_RING_CASES = [(1, 16384, 7168), (2, 16384, 7168), (1, 32768, 2048), (2, 32768, 1000)]


def _ring_outputs():
    """fp8_gemm and the one-call linear on shapes whose M <= 16 kernel runs its ring variant (every wavefront's K range
    two ring rounds or more): the weight loads and their counted waits are written out by hand there."""
    import dsv3fp8 as K
    from dsv3fp8 import workloads, ops, _lib
    out = {}
    for m, k, n in _RING_CASES:
        x = workloads.activations(m, k, seed=m + k % 13).cuda()
        w8, ws = workloads.weight(n, k, seed=n % 17)
        w8, ws = w8.cuda(), ws.cuda()
        a, a_s = K.act_quant(x)
        out[f"gemm_{m}_{k}_{n}"] = torch.ops.dsv3fp8.fp8_gemm(a, a_s, w8, ws, _lib.F32).cpu()
        assert ops.linear_fp8_fused(m, n, k)
        out[f"linear_{m}_{k}_{n}"] = torch.ops.dsv3fp8.linear_fp8(x, w8, ws, _lib.SCALE_FMT_NONE, _lib.F32).cpu()
    return out


def test_ring_variant_equals_batch_variant(K, tmp_path):
    """The ring variant of the M <= 16 kernel (loads and waits in inline assembly, a slot refilled as soon as it has been
    multiplied) against the batch variant of the same kernel (compiler-scheduled loads; DSV3_SKINNY_NORING=1, read once
    per process, hence the second process), with and without the in-kernel quantiser: bit for bit."""
    import os, subprocess, sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    ring = _ring_outputs()
    dst = tmp_path / "batch.pt"
    code = ("import sys, torch\n"
            f"sys.path[:0] = [{str(root)!r}, {str(root / 'deepseek-v3_amd')!r}]\n"
            "from tests.test_gpu_fp8_gemm import _ring_outputs\n"
            f"torch.save(_ring_outputs(), {str(dst)!r})\n")
    env = dict(os.environ, DSV3_SKINNY_NORING="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    batch = torch.load(dst, weights_only=True)
    assert set(batch) == set(ring)
    for key, v in ring.items():
        assert torch.equal(v, batch[key]), key
        assert torch.isfinite(v).all() and v.abs().max() > 0
