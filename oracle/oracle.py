"""TEST INFRASTRUCTURE ONLY.

torch-CPU restatement of the arithmetic of DeepSeek-V3's block-scaled FP8 path.
Nothing in the shipped package imports this module; only ``tests/``, the smoke
check and the bench's ``cpu_baseline`` leg do, and only as the checker.

Each function cites the reference lines it restates (paths relative to the
reference checkout).  All arithmetic is IEEE binary32 on the CPU:

* ``act_quant``      inference/kernel.py:23-35, 51-57
* ``weight_dequant`` inference/kernel.py:76-86, 104-110
* ``fp8_gemm``       inference/kernel.py:145-172, 188-196
* ``linear``         inference/model.py:131-163
* ``gate``           inference/model.py:566-598
* ``mlp`` / ``moe``  inference/model.py:532, 633, 669-693
* ``block_quant_weight`` README_WEIGHTS.md:83-92 (zero padding of ragged blocks)
* ``wkv_b_absorb``   inference/model.py:481-483, 495 (the two wkv_b products of the absorbed attention)
* ``rms_norm`` / ``rotary`` / ``mla``  inference/model.py:270-291, 375-392, 456-497

Pinning (see tests/test_oracle_*.py): the conversions and all three kernels are
checked against the independent plain-C restatement in ``dsv3_oracle.c`` and
against closed-form known answers; ``wkv_b_absorb`` against a scalar triple loop,
one-hot inputs that read single dequantised weights and exact integer cases.  "Parity unpinned": the choice among
equal scores in ``gate`` (torch.topk leaves ties unspecified; the workloads are generated without ties), and what
``act_quant`` does with a NaN or an infinity in a block -- this restatement follows torch's ``amax`` (the NaN reaches
the scale, in both scale formats), and no file of the reference says whether its Triton maximum does the same.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0
BLOCK = 128


def ue8m0_round_up(s: torch.Tensor) -> torch.Tensor:
    """s -> 2^ceil(log2 s) for positive binary32 (kernel.py:29-31).

    Defined on the bits so that it does not depend on a libm: a power of two is
    kept, any other value moves up to the next power of two.  Infinity and NaN
    pass through, as they do through exp2(ceil(log2(s))).
    """
    bits = s.contiguous().view(torch.int32)
    exp = bits >> 23
    mant = bits & 0x7FFFFF
    exp = exp + (mant != 0).to(torch.int32)
    return torch.where(torch.isfinite(s), (exp << 23).view(torch.float32), s)


def act_quant(x: torch.Tensor, block_size: int = BLOCK,
              scale_fmt: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """kernel.py:23-35: per run of ``block_size`` contiguous elements
    amax = max|x|, clamped below at 1e-4; s = amax / 448; y = e4m3(x / s)."""
    assert x.is_contiguous()
    assert x.size(-1) % block_size == 0
    xf = x.float().view(-1, block_size)
    amax = xf.abs().amax(dim=-1, keepdim=True)
    amax = torch.maximum(amax, torch.tensor(1e-4, dtype=torch.float32))
    s = amax / 448.0
    if scale_fmt == "ue8m0":
        s = ue8m0_round_up(s)
    y = (xf / s).to(FP8).view(x.shape)
    s = s.view(*x.shape[:-1], x.size(-1) // block_size)
    return y, s


def expand_block_scale(s: torch.Tensor, m: int, n: int, block_size: int = BLOCK) -> torch.Tensor:
    """[ceil(m/b), ceil(n/b)] block scales -> [m, n] per-element scales."""
    return s.repeat_interleave(block_size, 0)[:m].repeat_interleave(block_size, 1)[:, :n]


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = BLOCK,
                   out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """kernel.py:83-86: y[i,j] = out_dtype( f32(x[i,j]) * s[i//b, j//b] )."""
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    m, n = x.shape
    return (x.float() * expand_block_scale(s, m, n, block_size)).to(out_dtype)


def fp8_gemm_f32(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """kernel.py:157-166 in binary32, result left in binary32:
    c = sum_kb (a_kb @ b_kb^T) * a_s[:, kb, None] * b_s[n//128, kb][None, :]."""
    k = a.size(-1)
    m = a.numel() // k
    n = b.size(0)
    af = a.reshape(m, k).float()
    bf = b.float()
    asf = a_s.reshape(m, -1).float()
    nb = torch.arange(n) // BLOCK
    acc = torch.zeros(m, n, dtype=torch.float32)
    # a last block of fewer than 128 values is masked, i.e. zero-filled (kernel.py:145, 158-159): its scales are
    # column ceil(k / 128) - 1 of both scale tensors
    for kb in range(-(-k // BLOCK)):
        sl = slice(kb * BLOCK, min((kb + 1) * BLOCK, k))
        dot = af[:, sl] @ bf[:, sl].t()
        acc += dot * asf[:, kb, None] * b_s[nb, kb][None, :]
    return acc.view(*a.shape[:-1], n)


def fp8_gemm(a, a_s, b, b_s, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """kernel.py:167 + 193: the binary32 accumulator cast to the output dtype."""
    return fp8_gemm_f32(a, a_s, b, b_s).to(out_dtype)


def block_quant_weight(w: torch.Tensor, block_size: int = BLOCK,
                       scale_fmt: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """README_WEIGHTS.md:83-92: per 128x128 block (ragged edge blocks are
    zero-padded, which leaves their amax unchanged) scale = amax / 448 and
    w8 = e4m3(w / scale); the stored scale is the dequantisation multiplier
    (``weight_scale_inv``)."""
    m, n = w.shape
    mb, nb = -(-m // block_size), -(-n // block_size)
    wp = torch.zeros(mb * block_size, nb * block_size, dtype=torch.float32)
    wp[:m, :n] = w.float()
    blocks = wp.view(mb, block_size, nb, block_size)
    amax = blocks.abs().amax(dim=(1, 3))
    amax = torch.maximum(amax, torch.tensor(1e-4, dtype=torch.float32))
    s = amax / 448.0
    if scale_fmt == "ue8m0":                  # kernel.py:29-31 applied to the block scale
        s = ue8m0_round_up(s)
    w8 = (blocks / s[:, None, :, None]).view(mb * block_size, nb * block_size)[:m, :n].contiguous().to(FP8)
    return w8, s


def linear(x, weight, bias=None, scale=None, gemm_impl: str = "fp8",
           scale_fmt: Optional[str] = None) -> torch.Tensor:
    """model.py:153-163.  ``scale`` plays the role of ``weight.scale``."""
    if weight.element_size() > 1:
        return F.linear(x, weight, bias)
    if gemm_impl == "bf16":
        return F.linear(x, weight_dequant(weight, scale, out_dtype=x.dtype), bias)
    xq, xs = act_quant(x, BLOCK, scale_fmt)
    y = fp8_gemm(xq, xs, weight, scale, out_dtype=x.dtype)
    if bias is not None:
        y += bias
    return y


def mlp(x, w1, s1, w2, s2, w3, s3, scale_fmt=None) -> torch.Tensor:
    """model.py:532 / 633: w2( silu(w1 x) * w3 x ) with fp8 linears."""
    h = F.silu(linear(x, w1, scale=s1, scale_fmt=scale_fmt)) * linear(x, w3, scale=s3, scale_fmt=scale_fmt)
    return linear(h, w2, scale=s2, scale_fmt=scale_fmt)


def gate_route(scores, gate_bias, topk: int, n_groups: int, topk_groups: int,
               route_scale: float, score_func: str = "sigmoid"):
    """model.py:577-598: everything after the router's linear layer.  ``scores`` is its output [tokens, experts]."""
    tokens = scores.size(0)
    if score_func == "softmax":
        scores = scores.softmax(dim=-1, dtype=torch.float32)
    else:
        scores = scores.sigmoid()
    original = scores
    if gate_bias is not None:
        scores = scores + gate_bias
    if n_groups > 1:
        scores = scores.view(tokens, n_groups, -1)
        if gate_bias is None:
            group_scores = scores.amax(dim=-1)
        else:
            group_scores = scores.topk(2, dim=-1)[0].sum(dim=-1)
        idx = group_scores.topk(topk_groups, dim=-1)[1]
        mask = torch.ones(tokens, n_groups, dtype=torch.bool).scatter_(1, idx, False)
        scores = scores.masked_fill(mask.unsqueeze(-1), float("-inf")).flatten(1)
    indices = torch.topk(scores, topk, dim=-1)[1]
    weights = original.gather(1, indices)
    if score_func == "sigmoid":
        weights = weights / weights.sum(dim=-1, keepdim=True)
    weights = weights * route_scale
    return weights, indices


def gate(x, gate_weight, gate_bias, topk: int, n_groups: int, topk_groups: int,
         route_scale: float, score_func: str = "sigmoid"):
    """model.py:576-598."""
    weights, indices = gate_route(F.linear(x, gate_weight), gate_bias, topk, n_groups, topk_groups, route_scale,
                                  score_func)
    return weights.type_as(x), indices


def moe(x, weights, indices, experts, shared, scale_fmt=None) -> torch.Tensor:
    """model.py:679-693 at world_size 1.  ``experts`` is a list of
    (w1, s1, w2, s2, w3, s3); ``shared`` is one such tuple."""
    shape = x.shape
    x = x.view(-1, shape[-1])
    y = torch.zeros_like(x)
    counts = torch.bincount(indices.flatten(), minlength=len(experts)).tolist()
    for i, ex in enumerate(experts):
        if counts[i] == 0:
            continue
        idx, top = torch.where(indices == i)
        y[idx] += mlp(x[idx], *ex, scale_fmt=scale_fmt) * weights[idx, top, None]
    z = mlp(x, *shared)   # the shared expert is an MLP of Column/RowParallelLinear: no scale_fmt (model.py:233,262)
    return (y + z).view(shape)


def wkv_b_absorb_f32(x: torch.Tensor, wkv_b: torch.Tensor, scale: torch.Tensor, side: str,
                     nope_dim: int, v_dim: int) -> torch.Tensor:
    """model.py:481-483 and :495 with the result left in binary32.  The weight is dequantised to bf16 first
    (model.py:481, kernel.py:83-86) and viewed as [heads, nope+v, c] (model.py:482);
    side "q": "bshd,hdc->bshc" with wkv_b[:, :nope]; side "v": "bshc,hdc->bshd" with wkv_b[:, -v:].
    ``x`` is [..., heads, d or c]."""
    heads = x.size(-2)
    w = weight_dequant(wkv_b, scale).float().view(heads, nope_dim + v_dim, wkv_b.size(1))
    if side == "q":
        return torch.einsum("...hd,hdc->...hc", x.float(), w[:, :nope_dim])
    return torch.einsum("...hc,hdc->...hd", x.float(), w[:, -v_dim:])


def wkv_b_absorb(x, wkv_b, scale, side: str, nope_dim: int, v_dim: int) -> torch.Tensor:
    """The bf16 einsum of the reference: binary32 accumulation, one rounding to the dtype of ``x``."""
    return wkv_b_absorb_f32(x, wkv_b, scale, side, nope_dim, v_dim).to(x.dtype)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """model.py:291 (F.rms_norm): x * rsqrt(mean(x^2) + eps) * weight, evaluated in binary32."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(x.dtype)


def rotary(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    """model.py:375-392: consecutive pairs of the last dimension times e^{i theta} of the position."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    y = torch.view_as_real(xc * freqs_cis.view(1, x.size(1), 1, xc.size(-1))).flatten(3)
    return y.to(x.dtype)


def _bf16_einsum(eq: str, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.einsum(eq, a.float(), b.float()).to(a.dtype)


def mla(x, start_pos: int, freqs_cis, mask, p: dict, kv_cache, pe_cache, n_heads: int, nope_dim: int,
        rope_dim: int, v_dim: int, kv_rank: int, softmax_scale: float, scale_fmt=None,
        attn_impl: str = "absorb") -> torch.Tensor:
    """model.py:456-497 with a low-rank query (q_lora_rank > 0), at world_size 1: the "absorb" branch, or the
    "naive" one (model.py:470-479, 488-490), for which ``kv_cache`` / ``pe_cache`` are the per-head
    k_cache [b, t, h, nope + rope] / v_cache [b, t, h, v].
    ``p`` maps a layer name to (weight, scale) for the five linears and to the weight for the two norms;
    the caches are updated in place like the reference's buffers.  Every einsum is a bf16 matmul: binary32
    accumulation, one rounding."""
    bsz, seqlen, _ = x.shape
    end_pos = start_pos + seqlen
    lin = lambda name, t, fmt=None: linear(t, p[name][0], scale=p[name][1], scale_fmt=fmt)
    # wq_a and wkv_a are plain Linear layers and take scale_fmt; wq_b, wkv_b, wo are parallel layers and do not
    q = lin("wq_b", rms_norm(lin("wq_a", x, scale_fmt), p["q_norm"]))
    q = q.view(bsz, seqlen, n_heads, nope_dim + rope_dim)
    q_nope, q_pe = torch.split(q, [nope_dim, rope_dim], dim=-1)
    q_pe = rotary(q_pe, freqs_cis)
    kv, k_pe = torch.split(lin("wkv_a", x, scale_fmt), [kv_rank, rope_dim], dim=-1)
    k_pe = rotary(k_pe.unsqueeze(2), freqs_cis)
    if attn_impl == "naive":
        k_cache, v_cache = kv_cache, pe_cache
        q = torch.cat([q_nope, q_pe], dim=-1)
        kv = lin("wkv_b", rms_norm(kv, p["kv_norm"])).view(bsz, seqlen, n_heads, nope_dim + v_dim)
        k_nope, v = torch.split(kv, [nope_dim, v_dim], dim=-1)
        k_cache[:bsz, start_pos:end_pos] = torch.cat([k_nope, k_pe.expand(-1, -1, n_heads, -1)], dim=-1)
        v_cache[:bsz, start_pos:end_pos] = v
        scores = _bf16_einsum("bshd,bthd->bsht", q, k_cache[:bsz, :end_pos]) * softmax_scale
        if mask is not None:
            scores = scores + mask.unsqueeze(1)
        scores = scores.softmax(dim=-1, dtype=torch.float32).type_as(x)
        return lin("wo", _bf16_einsum("bsht,bthd->bshd", scores, v_cache[:bsz, :end_pos]).flatten(2))
    q_nope = wkv_b_absorb(q_nope, p["wkv_b"][0], p["wkv_b"][1], "q", nope_dim, v_dim)
    kv_cache[:bsz, start_pos:end_pos] = rms_norm(kv, p["kv_norm"])
    pe_cache[:bsz, start_pos:end_pos] = k_pe.squeeze(2)
    scores = (_bf16_einsum("bshc,btc->bsht", q_nope, kv_cache[:bsz, :end_pos]) +
              _bf16_einsum("bshr,btr->bsht", q_pe, pe_cache[:bsz, :end_pos])) * softmax_scale
    if mask is not None:
        scores = scores + mask.unsqueeze(1)
    scores = scores.softmax(dim=-1, dtype=torch.float32).type_as(x)
    o = _bf16_einsum("bsht,btc->bshc", scores, kv_cache[:bsz, :end_pos])
    o = wkv_b_absorb(o, p["wkv_b"][0], p["wkv_b"][1], "v", nope_dim, v_dim)
    return lin("wo", o.flatten(2))
