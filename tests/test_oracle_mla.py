"""Pins the oracle of the absorbed-attention products with the FP8 weight wkv_b (oracle.wkv_b_absorb,
inference/model.py:481-483 and :495) and of the attention layer around them (oracle.mla, model.py:456-497).
The reference has no test for either; the pins are a scalar triple loop, one-hot inputs that must read single
dequantised weights, an exact integer case, and -- for the layer -- the identity between the absorbed form
and the textbook attention over explicitly up-projected keys and values (the reference's "naive" branch)."""
import math

import numpy as np
import torch
import torch.nn.functional as F

from oracle import oracle

FP8 = torch.float8_e4m3fn


def _wkv_b(heads, nope, v, c, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(heads * (nope + v), c, generator=g) * 0.05).bfloat16()
    return oracle.block_quant_weight(w)


def test_absorb_brute_force_tiny():
    heads, nope, v, c = 2, 32, 32, 128
    w8, s = _wkv_b(heads, nope, v, c, 0)
    wd = oracle.weight_dequant(w8, s).double()            # [heads*(nope+v), c]
    g = torch.Generator().manual_seed(1)
    xq = torch.randn(3, heads, nope, generator=g).bfloat16()
    xv = torch.randn(3, heads, c, generator=g).bfloat16()
    yq = oracle.wkv_b_absorb_f32(xq, w8, s, "q", nope, v)
    yv = oracle.wkv_b_absorb_f32(xv, w8, s, "v", nope, v)
    for m in range(3):
        for h in range(heads):
            for cc in range(0, c, 17):
                ref = sum(float(xq[m, h, d]) * float(wd[h * (nope + v) + d, cc]) for d in range(nope))
                assert abs(yq[m, h, cc].item() - ref) <= 1e-5 * (1 + abs(ref))
            for d in range(0, v, 5):
                ref = sum(float(xv[m, h, cc]) * float(wd[h * (nope + v) + nope + d, cc]) for cc in range(c))
                assert abs(yv[m, h, d].item() - ref) <= 1e-5 * (1 + abs(ref))


def test_absorb_one_hot_reads_single_weights():
    """x = e_d selects row d of the head's first nope rows (side q); x = e_c selects column c of its last v
    rows (side v).  A wrong slice, a transposed operand or a wrong head stride fails here exactly."""
    heads, nope, v, c = 3, 64, 32, 256
    w8, s = _wkv_b(heads, nope, v, c, 2)
    wd = oracle.weight_dequant(w8, s).view(heads, nope + v, c)
    for d in (0, 17, 63):
        x = torch.zeros(1, heads, nope, dtype=torch.bfloat16); x[..., d] = 1
        y = oracle.wkv_b_absorb(x, w8, s, "q", nope, v)
        assert torch.equal(y[0], wd[:, d, :])
    for cc in (0, 129, 255):
        x = torch.zeros(1, heads, c, dtype=torch.bfloat16); x[..., cc] = 1
        y = oracle.wkv_b_absorb(x, w8, s, "v", nope, v)
        assert torch.equal(y[0], wd[:, nope:, cc])


def test_absorb_exact_integer_case():
    heads, nope, v, c = 2, 64, 64, 128
    g = torch.Generator().manual_seed(3)
    wi = torch.randint(-3, 4, (heads * (nope + v), c), generator=g)
    w8 = wi.float().to(FP8)
    s = torch.ones(heads * (nope + v) // 128, c // 128)
    xq = torch.randint(-2, 3, (5, heads, nope), generator=g)
    xv = torch.randint(-2, 3, (5, heads, c), generator=g)
    w3 = wi.view(heads, nope + v, c).numpy()
    yq = np.einsum("mhd,hdc->mhc", xq.numpy(), w3[:, :nope])
    yv = np.einsum("mhc,hdc->mhd", xv.numpy(), w3[:, nope:])
    assert np.array_equal(oracle.wkv_b_absorb_f32(xq.bfloat16(), w8, s, "q", nope, v).numpy(), yq.astype(np.float32))
    assert np.array_equal(oracle.wkv_b_absorb_f32(xv.bfloat16(), w8, s, "v", nope, v).numpy(), yv.astype(np.float32))


def small_mla_params(dim, heads, q_rank, kv_rank, nope, rope, v, seed):
    """Random FP8 weights of one attention layer: name -> (weight, scale), norms -> weight."""
    g = torch.Generator().manual_seed(seed)

    def lin(out_f, in_f):
        return oracle.block_quant_weight((torch.randn(out_f, in_f, generator=g) * in_f ** -0.5).bfloat16())
    return {
        "wq_a": lin(q_rank, dim), "q_norm": (1 + 0.1 * torch.randn(q_rank, generator=g)).bfloat16(),
        "wq_b": lin(heads * (nope + rope), q_rank),
        "wkv_a": lin(kv_rank + rope, dim), "kv_norm": (1 + 0.1 * torch.randn(kv_rank, generator=g)).bfloat16(),
        "wkv_b": lin(heads * (nope + v), kv_rank), "wo": lin(dim, heads * v),
    }


def _freqs(rope, seqlen, base=10000.0):
    f = base ** (-torch.arange(0, rope, 2, dtype=torch.float32) / rope)
    ang = torch.outer(torch.arange(seqlen), f)
    return torch.polar(torch.ones_like(ang), ang)


def test_mla_absorbed_equals_textbook_attention():
    """The absorbed layer against float64 attention over explicit per-head keys and values,
    k = [wkv_b_k . kv_norm(kv), rot(k_pe)], v = wkv_b_v . kv_norm(kv), with unquantised (dequantised-weight)
    linears.  The two differ by the FP8 activation quantisation and the bf16 roundings only."""
    dim, heads, q_rank, kv_rank, nope, rope, v = 256, 4, 128, 128, 64, 32, 64
    p = small_mla_params(dim, heads, q_rank, kv_rank, nope, rope, v, 5)
    bsz, seqlen = 2, 6
    g = torch.Generator().manual_seed(6)
    x = torch.randn(bsz, seqlen, dim, generator=g).bfloat16()
    freqs = _freqs(rope, seqlen)
    mask = torch.full((seqlen, seqlen), float("-inf")).triu_(1)
    scale = (nope + rope) ** -0.5
    kv_cache = torch.zeros(bsz, 16, kv_rank, dtype=torch.bfloat16)
    pe_cache = torch.zeros(bsz, 16, rope, dtype=torch.bfloat16)
    got = oracle.mla(x, 0, freqs, mask, p, kv_cache, pe_cache, heads, nope, rope, v, kv_rank, scale).double()

    W = {k: oracle.weight_dequant(*val).double() for k, val in p.items() if isinstance(val, tuple)}
    xd = x.double()
    rms = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()

    def rot(t):   # [b, s, h, r]
        tc = torch.view_as_complex(t.reshape(*t.shape[:-1], -1, 2))
        return torch.view_as_real(tc * freqs.to(torch.complex128).view(1, seqlen, 1, -1)).flatten(3)
    q = F.linear(rms(F.linear(xd, W["wq_a"]), p["q_norm"]), W["wq_b"]).view(bsz, seqlen, heads, nope + rope)
    q = torch.cat([q[..., :nope], rot(q[..., nope:])], dim=-1)
    kva = F.linear(xd, W["wkv_a"])
    lat, k_pe = rms(kva[..., :kv_rank], p["kv_norm"]), rot(kva[..., kv_rank:].unsqueeze(2))
    kvh = F.linear(lat, W["wkv_b"]).view(bsz, seqlen, heads, nope + v)
    k = torch.cat([kvh[..., :nope], k_pe.expand(-1, -1, heads, -1)], dim=-1)
    sc = torch.einsum("bshd,bthd->bsht", q, k) * scale + mask.double().unsqueeze(1)
    o = torch.einsum("bsht,bthd->bshd", sc.softmax(-1), kvh[..., nope:])
    ref = F.linear(o.flatten(2), W["wo"])
    err = (got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()
    assert err < 0.05, err
    # the caches hold the normalised latent and the rotated shared key of the positions just written
    assert (kv_cache[:, :seqlen].double() - lat).abs().max() < 0.1 and kv_cache[:, seqlen:].abs().max() == 0
    assert (pe_cache[:, :seqlen].double() - k_pe.squeeze(2)).abs().max() < 0.1
    # the "naive" branch (per-head key / value caches, model.py:470-479, 488-490) against the same textbook result,
    # its caches against the explicit keys and values, and against the absorbed branch
    k_cache = torch.zeros(bsz, 16, heads, nope + rope, dtype=torch.bfloat16)
    v_cache = torch.zeros(bsz, 16, heads, v, dtype=torch.bfloat16)
    naive = oracle.mla(x, 0, freqs, mask, p, k_cache, v_cache, heads, nope, rope, v, kv_rank, scale,
                       attn_impl="naive").double()
    err_n = (naive - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()
    assert err_n < 0.08, err_n                   # (one more FP8 activation quantisation: the latent in front of wkv_b)
    assert (naive - got).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt() < 0.08
    assert (k_cache[:, :seqlen].double() - k).abs().max() < 0.3 and k_cache[:, seqlen:].abs().max() == 0
    assert (v_cache[:, :seqlen].double() - kvh[..., nope:]).abs().max() < 0.3 and v_cache[:, seqlen:].abs().max() == 0


def test_rotary_table_equals_the_reference_expressions_bit_for_bit():
    """precompute_freqs_cis against the reference's expressions written out literally (model.py:297-372): the same
    binary32 operations in the same order, for the extended window (YaRN) and for the plain one."""
    import math
    import sys
    from pathlib import Path
    sys.path.insert(0, str(Path(__file__).resolve().parent.parent / "deepseek-v3_amd"))
    try:
        from dsv3fp8 import model as M
    except ImportError:
        import pytest
        pytest.skip("the package needs its HIP library to import")
    for max_seq_len in (4096 * 4, 4096):
        args = M.ModelArgs(max_seq_len=max_seq_len)
        dim, base, factor = args.qk_rope_head_dim, args.rope_theta, args.rope_factor

        def correction_dim(num_rotations):
            return dim * math.log(args.original_seq_len / (num_rotations * 2 * math.pi)) / (2 * math.log(base))
        freqs = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
        if max_seq_len > args.original_seq_len:
            low = max(math.floor(correction_dim(args.beta_fast)), 0)
            high = min(math.ceil(correction_dim(args.beta_slow)), dim - 1)
            if low == high:
                high += 0.001
            ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - low) / (high - low), 0, 1)
            smooth = 1 - ramp
            freqs = freqs / factor * (1 - smooth) + freqs * smooth
        t = torch.arange(max_seq_len)
        f = torch.outer(t, freqs)
        want = torch.polar(torch.ones_like(f), f)
        got = M.precompute_freqs_cis(args)
        assert torch.equal(torch.view_as_real(got), torch.view_as_real(want))
