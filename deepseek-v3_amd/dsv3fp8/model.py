"""Host-side callers of the FP8 kernels, mirroring the part of the reference's
``inference/model.py`` that sits directly on top of them: the ``linear()``
dispatch (model.py:131-163), ``Linear`` and its column/row parallel variants
(model.py:166-267), the SwiGLU / routing modules that issue the FP8 linears
of the MoE layer (``MLP`` :500-532, ``Gate`` :535-598, ``Expert`` :601-633,
``MoE`` :636-693), and the attention layer ``MLA`` (:395-497) whose absorbed
form multiplies with the FP8 weight ``wkv_b`` directly.  Names, constructor arguments, the ``weight.scale``
convention and the module-level switches (``gemm_impl``, ``block_size``) follow
the reference so that code written against it runs unchanged.

This build runs on one GPU: ``world_size`` is fixed at 1, so the parallel
variants reduce to plain ``Linear`` and no collective is issued.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Literal, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .kernel import act_quant, fp8_gemm, fp8_gemm_pow2, weight_dequant

world_size = 1
rank = 0
block_size = 128
gemm_impl: Literal["bf16", "fp8"] = "bf16"     # the reference's default (model.py:16); set to "fp8" for the FP8 GEMM path
attn_impl: Literal["naive", "absorb"] = "absorb"   # model.py:17


@dataclass
class ModelArgs:
    """The subset of the reference's ModelArgs (model.py:19-86) that these modules read; defaults of the 671B
    configuration (inference/configs/config_671B.json)."""
    dim: int = 7168
    inter_dim: int = 18432
    moe_inter_dim: int = 2048
    n_routed_experts: int = 256
    n_shared_experts: int = 1
    n_activated_experts: int = 8
    n_expert_groups: int = 8
    n_limited_groups: int = 4
    score_func: Literal["softmax", "sigmoid"] = "sigmoid"
    route_scale: float = 2.5
    # attention (MLA) and its rotary embedding
    max_batch_size: int = 8
    max_seq_len: int = 4096 * 4
    n_heads: int = 128
    q_lora_rank: int = 1536
    kv_lora_rank: int = 512
    qk_nope_head_dim: int = 128
    qk_rope_head_dim: int = 64
    v_head_dim: int = 128
    original_seq_len: int = 4096
    rope_theta: float = 10000.0
    rope_factor: float = 40
    beta_fast: int = 32
    beta_slow: int = 1
    mscale: float = 1.


def _scales_are_powers_of_two(weight: torch.Tensor, scale: Optional[torch.Tensor] = None) -> bool:
    """Whether every block scale of an fp8 weight is a power of two (checkpoints made for ``scale_fmt = "ue8m0"``,
    inference/configs/config_v3.1.json:22, store them that way).  Looked at once per version of the scale tensor
    (one device-to-host read), never while a graph is being captured.  The verdict is keyed on the scale tensor's
    storage address and version counter; a tensor made under inference_mode has no counter, so such scales must
    not be rewritten in place after the first forward (reload them into a new module instead)."""
    scale = weight.scale if scale is None else scale
    try:
        version = (scale.data_ptr(), scale._version)
    except RuntimeError:            # a tensor made under inference_mode has no version counter: looked at once
        version = (scale.data_ptr(), -1)
    cached = getattr(weight, "_dsv3_pow2", None)
    if cached is not None and cached[0] == version:
        return cached[1]
    if torch.cuda.is_current_stream_capturing():
        return False
    flag = bool(((scale.detach().view(torch.int32) & 0x7FFFFF) == 0).all().item()) and bool((scale > 0).all().item())
    weight._dsv3_pow2 = (version, flag)
    return flag


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           scale_fmt: Optional[str] = None) -> torch.Tensor:
    """y = x @ weight.T + bias with the reference's three-way dispatch (model.py:153-163): wide weights go to
    ``F.linear``; 1-byte weights are dequantised first when ``gemm_impl == "bf16"``, otherwise the activation
    is quantised per 1x128 block and multiplied with ``fp8_gemm``.  ``weight.scale`` carries the block scales."""
    if weight.element_size() > 1:
        return F.linear(x, weight, bias)
    if gemm_impl == "bf16":
        return F.linear(x, weight_dequant(weight, weight.scale), bias)
    if (scale_fmt == "ue8m0" and x.is_cuda and block_size == 128 and x.numel() > 64 * x.size(-1)
            and _scales_are_powers_of_two(weight)):
        # activation and weight scales are all powers of two: they go into the matrix instruction's scale operands
        xq, xs = act_quant(x, block_size, scale_fmt)
        y = fp8_gemm_pow2(xq, xs, weight, weight.scale)
    elif (x.is_cuda and x.is_contiguous() and weight.is_contiguous() and block_size == 128
            and x.size(-1) % block_size == 0):
        # the same two steps behind one op, which runs them as a single launch for few rows (decode)
        fmt = ops._lib.SCALE_FMT_UE8M0 if scale_fmt == "ue8m0" else ops._lib.SCALE_FMT_NONE
        y = torch.ops.dsv3fp8.linear_fp8(x, weight, weight.scale, fmt, ops.dtype_code(torch.get_default_dtype()))
    else:
        xq, xs = act_quant(x, block_size, scale_fmt)
        y = fp8_gemm(xq, xs, weight, weight.scale)
    if bias is not None:
        y += bias
    return y


class Linear(nn.Module):
    """Linear layer whose weight may be fp8 with a block-scale tensor attached as ``weight.scale``
    (shape ``[ceil(out/128), ceil(in/128)]``, fp32), as in model.py:166-205."""
    dtype = torch.bfloat16
    scale_fmt: Optional[str] = None

    def __init__(self, in_features: int, out_features: int, bias: bool = False, dtype=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features, dtype=dtype or Linear.dtype))
        if self.weight.element_size() == 1:
            rows = -(-out_features // block_size)
            cols = -(-in_features // block_size)
            self.weight.scale = self.scale = nn.Parameter(torch.empty(rows, cols, dtype=torch.float32))
        else:
            self.register_parameter("scale", None)
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
        else:
            self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, self.bias, self.scale_fmt)


class ColumnParallelLinear(Linear):
    """Output features split over ranks (model.py:208-234); at world_size 1 the whole layer.  Like the
    reference, it does not forward ``scale_fmt`` (model.py:233)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, dtype=None):
        assert out_features % world_size == 0, f"Output features must be divisible by world size (world_size={world_size})"
        self.part_out_features = out_features // world_size
        super().__init__(in_features, self.part_out_features, bias, dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, self.bias)


class RowParallelLinear(Linear):
    """Input features split over ranks (model.py:237-267); the partial products would be all-reduced before
    the bias is added.  At world_size 1 there is nothing to reduce."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, dtype=None):
        assert in_features % world_size == 0, f"Input features must be divisible by world size (world_size={world_size})"
        self.part_in_features = in_features // world_size
        super().__init__(self.part_in_features, out_features, bias, dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = linear(x, self.weight)
        if self.bias is not None:
            y += self.bias
        return y


class RMSNorm(nn.Module):
    """x / rms(x) * weight over the last dimension (model.py:270-291)."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.dim = dim
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.rms_norm(x, (self.dim,), self.weight, self.eps)


def precompute_freqs_cis(args: ModelArgs) -> torch.Tensor:
    """Rotary phases e^{i * pos * f_j} for every position below ``max_seq_len`` as a complex64
    ``[max_seq_len, qk_rope_head_dim / 2]`` tensor (model.py:294-372).  Beyond ``original_seq_len`` the
    frequencies are stretched YaRN-style: pair j keeps its frequency where it completes more than ``beta_fast``
    turns over the original window, is divided by ``rope_factor`` where it completes fewer than ``beta_slow``,
    and is blended linearly in between.  The binary32 expressions are evaluated in the reference's order
    (1 / base^(j/dim); keep = 1 - ramp; f / factor * (1 - keep) + f * keep), so the table is the same bit for bit."""
    dim, base = args.qk_rope_head_dim, args.rope_theta
    freqs = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    if args.max_seq_len > args.original_seq_len:
        def pair_index(turns: float) -> float:     # the (fractional) pair that makes `turns` rotations in the window
            return dim * math.log(args.original_seq_len / (turns * 2 * math.pi)) / (2 * math.log(base))
        lo = max(math.floor(pair_index(args.beta_fast)), 0)
        hi = min(math.ceil(pair_index(args.beta_slow)), dim - 1)
        span = (hi - lo) if hi != lo else 0.001
        ramp = torch.clamp((torch.arange(dim // 2, dtype=torch.float32) - lo) / span, 0, 1)
        keep = 1 - ramp
        freqs = freqs / args.rope_factor * (1 - keep) + freqs * keep
    angles = torch.outer(torch.arange(args.max_seq_len), freqs)
    return torch.polar(torch.ones_like(angles), angles)


def apply_rotary_emb(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    """Rotate consecutive pairs of the last dimension of ``x`` ``[b, s, h, r]`` by the phases of positions
    ``[s, r/2]``, in binary32, and return the dtype of ``x`` (model.py:375-392)."""
    pairs = x.float().unflatten(-1, (-1, 2))
    re, im = pairs[..., 0], pairs[..., 1]
    cos = freqs_cis.real.view(1, x.size(1), 1, -1)
    sin = freqs_cis.imag.view(1, x.size(1), 1, -1)
    return torch.stack((re * cos - im * sin, re * sin + im * cos), dim=-1).flatten(-2).to(x.dtype)


class MLA(nn.Module):
    """Host of the two ``wkv_b`` products of the absorbed multi-head latent attention (model.py:395-497).

    In the reference's default cache layout (``attn_impl == "absorb"``) the compressed latent
    (``kv_cache`` [b, t, kv_lora_rank]) and the shared rotary key (``pe_cache``) are cached and the up-projection
    ``wkv_b`` is folded into the query (``q_nope @ wkv_b[:, :nope]``, before the scores) and into the output
    (``@ wkv_b[:, -v:]^T``, after the weighted sum).  With ``wkv_b`` in FP8 the reference dequantises the whole
    weight on every call (model.py:481); here the two products read the FP8 weight and its block scales in place
    (``torch.ops.dsv3fp8.wkv_b_absorb``) with the same bf16 rounding of every dequantised weight.
    ``attn_impl == "naive"`` (model.py:443-445, 470-479, 488-490) caches per-head keys and values instead
    (``k_cache`` [b, t, h, nope + rope], ``v_cache`` [b, t, h, v]): ``wkv_b`` is then an ordinary linear layer on
    the new positions' latents (an FP8 GEMM through ``linear()``), and the scores and the weighted sum are plain
    per-head einsums.
    ``MLA.fused = False`` selects the dequantise-then-einsum sequence instead.  Everything between the two products
    (scores, softmax, weighted sum) is bf16 torch arithmetic that never touches FP8 data; it is here so that the
    products can be tested in place.  Parameter names are the checkpoint's.

    ``wq_a`` and ``wkv_a`` read the same input.  With FP8 weights (and ``q_lora_rank`` a multiple of the block size,
    so that both keep their own scale blocks) ``stack_a()`` lays them out as one ``[q_lora_rank + kv_lora_rank +
    rope, dim]`` weight whose halves the two layers keep as views, and the forward pass runs one linear instead of
    two (``MLA.stacked_a = False`` keeps them apart).
    """

    fused: bool = True
    stacked_a: bool = True

    def __init__(self, args: ModelArgs):
        super().__init__()
        if attn_impl not in ("absorb", "naive"):
            raise ValueError(f"attn_impl must be 'absorb' or 'naive', not {attn_impl!r}")
        self.attn_impl = attn_impl
        nope, rope, v = args.qk_nope_head_dim, args.qk_rope_head_dim, args.v_head_dim
        self.dim, self.n_heads, self.n_local_heads = args.dim, args.n_heads, args.n_heads // world_size
        self.q_lora_rank, self.kv_lora_rank = args.q_lora_rank, args.kv_lora_rank
        self.qk_nope_head_dim, self.qk_rope_head_dim, self.v_head_dim, self.qk_head_dim = nope, rope, v, nope + rope
        # projections, by their checkpoint names: query (optionally through a low-rank pair), latent + rotary key,
        # the up-projection that gets absorbed, output
        if self.q_lora_rank:
            self.wq_a = Linear(self.dim, self.q_lora_rank)
            self.q_norm = RMSNorm(self.q_lora_rank)
            self.wq_b = ColumnParallelLinear(self.q_lora_rank, self.n_heads * self.qk_head_dim)
        else:
            self.wq = ColumnParallelLinear(self.dim, self.n_heads * self.qk_head_dim)
        self.wkv_a = Linear(self.dim, self.kv_lora_rank + rope)
        self.kv_norm = RMSNorm(self.kv_lora_rank)
        self.wkv_b = ColumnParallelLinear(self.kv_lora_rank, self.n_heads * (nope + v))
        self.wo = RowParallelLinear(self.n_heads * v, self.dim)
        # 1/sqrt(d), times the YaRN magnitude correction squared when the window is extended (model.py:438-441)
        yarn = 0.1 * args.mscale * math.log(args.rope_factor) + 1.0 if args.max_seq_len > args.original_seq_len else 1.0
        self.softmax_scale = self.qk_head_dim ** -0.5 * yarn * yarn
        if self.attn_impl == "naive":
            caches = (("k_cache", (self.n_local_heads, self.qk_head_dim)), ("v_cache", (self.n_local_heads, v)))
        else:
            caches = (("kv_cache", (self.kv_lora_rank,)), ("pe_cache", (rope,)))
        for name, width in caches:
            self.register_buffer(name, torch.zeros(args.max_batch_size, args.max_seq_len, *width), persistent=False)

    def stack_a(self) -> bool:
        """wq_a over wkv_a in one buffer (scales likewise); returns whether the layers qualify.  Idempotent; the
        layers' parameters become views, so in-place weight loading keeps working."""
        if getattr(self, "_wa", None) is not None:
            return True
        if self.q_lora_rank == 0 or self.q_lora_rank % block_size or self.wq_a.weight.element_size() != 1 \
                or self.wkv_a.weight.element_size() != 1 or self.wq_a.scale_fmt != self.wkv_a.scale_fmt:
            return False
        qa, ka = self.wq_a, self.wkv_a
        with torch.no_grad():
            w = torch.cat([qa.weight.data.view(torch.uint8), ka.weight.data.view(torch.uint8)]).view(qa.weight.dtype)
            sc = torch.cat([qa.scale.data, ka.scale.data])
            qa.weight.data, ka.weight.data = w[:qa.out_features], w[qa.out_features:]
            qa.scale.data, ka.scale.data = sc[:qa.scale.size(0)], sc[qa.scale.size(0):]
        w.scale = sc
        self._wa = w
        return True

    def _absorb(self, x: torch.Tensor, side: int, wkv_b: Optional[torch.Tensor]) -> torch.Tensor:
        """One of the two wkv_b products.  ``wkv_b`` is the [h, nope+v, c] bf16 weight for the einsum path, or
        None to read the FP8 weight in place."""
        if wkv_b is None:
            return torch.ops.dsv3fp8.wkv_b_absorb(x, self.wkv_b.weight, self.wkv_b.scale, side,
                                                  self.qk_nope_head_dim, self.v_head_dim)
        if side == ops._lib.ABSORB_Q:
            return torch.einsum("bshd,hdc->bshc", x, wkv_b[:, :self.qk_nope_head_dim])
        return torch.einsum("bshc,hdc->bshd", x, wkv_b[:, -self.v_head_dim:])

    def _project(self, x: torch.Tensor):
        """Per-head queries [b, s, h, nope + rope] and the latent + rotary-key row [b, s, kv_lora_rank + rope]."""
        if self.stacked_a and gemm_impl == "fp8" and x.is_cuda and self.stack_a():
            qa, kva = torch.split(linear(x, self._wa, None, self.wq_a.scale_fmt),
                                  [self.q_lora_rank, self.kv_lora_rank + self.qk_rope_head_dim], dim=-1)
            q = self.wq_b(self.q_norm(qa))
        else:
            q = self.wq_b(self.q_norm(self.wq_a(x))) if self.q_lora_rank else self.wq(x)
            kva = self.wkv_a(x)
        return q.unflatten(-1, (self.n_local_heads, self.qk_head_dim)), kva

    def _dequantised_wkv_b(self, x: torch.Tensor) -> Optional[torch.Tensor]:
        """[h, nope+v, c] weight for the einsum path, or None when the products read the FP8 weight in place."""
        w = self.wkv_b.weight
        if w.element_size() == 1:
            if self.fused and x.is_cuda and x.dtype == torch.bfloat16:
                return None
            w = weight_dequant(w, self.wkv_b.scale, block_size)
        return w.view(self.n_local_heads, -1, self.kv_lora_rank)

    def forward(self, x: torch.Tensor, start_pos: int, freqs_cis: torch.Tensor, mask: Optional[torch.Tensor]):
        b, s = x.size(0), x.size(1)
        t = start_pos + s
        q, kva = self._project(x)
        if self.attn_impl == "naive":
            return self._forward_naive(x, q, kva, start_pos, freqs_cis, mask)
        wkv_b = self._dequantised_wkv_b(x)
        # this step's rows of the two caches
        self.kv_cache[:b, start_pos:t] = self.kv_norm(kva[..., :self.kv_lora_rank])
        self.pe_cache[:b, start_pos:t] = apply_rotary_emb(kva[..., self.kv_lora_rank:].unsqueeze(2), freqs_cis).squeeze(2)
        latent, rope_keys = self.kv_cache[:b, :t], self.pe_cache[:b, :t]
        # scores over the latent (query folded through wkv_b) plus the rotary part; softmax in binary32
        q_latent = self._absorb(q[..., :self.qk_nope_head_dim], ops._lib.ABSORB_Q, wkv_b)
        q_rope = apply_rotary_emb(q[..., self.qk_nope_head_dim:], freqs_cis)
        scores = torch.einsum("bshc,btc->bsht", q_latent, latent) + torch.einsum("bshr,btr->bsht", q_rope, rope_keys)
        scores = scores * self.softmax_scale
        if mask is not None:
            scores = scores + mask.unsqueeze(1)
        probs = scores.softmax(dim=-1, dtype=torch.float32).type_as(x)
        out = self._absorb(torch.einsum("bsht,btc->bshc", probs, latent), ops._lib.ABSORB_V, wkv_b)
        return self.wo(out.flatten(2))


    def _forward_naive(self, x, q, kva, start_pos: int, freqs_cis, mask):
        """Per-head key / value caches (model.py:470-479, 488-490): the new positions' latents go through wkv_b as a
        linear layer, keys are [nope part | the shared rotary key], scores and weighted sum are per-head einsums."""
        b, s = x.size(0), x.size(1)
        t = start_pos + s
        nope = self.qk_nope_head_dim
        q = torch.cat([q[..., :nope], apply_rotary_emb(q[..., nope:], freqs_cis)], dim=-1)
        rope_key = apply_rotary_emb(kva[..., self.kv_lora_rank:].unsqueeze(2), freqs_cis)
        kv = self.wkv_b(self.kv_norm(kva[..., :self.kv_lora_rank])).unflatten(-1, (self.n_local_heads, nope + self.v_head_dim))
        self.k_cache[:b, start_pos:t] = torch.cat([kv[..., :nope], rope_key.expand(-1, -1, self.n_local_heads, -1)], dim=-1)
        self.v_cache[:b, start_pos:t] = kv[..., nope:]
        scores = torch.einsum("bshd,bthd->bsht", q, self.k_cache[:b, :t]) * self.softmax_scale
        if mask is not None:
            scores = scores + mask.unsqueeze(1)
        probs = scores.softmax(dim=-1, dtype=torch.float32).type_as(x)
        return self.wo(torch.einsum("bsht,bthd->bshd", probs, self.v_cache[:b, :t]).flatten(2))


class MLP(nn.Module):
    """SwiGLU feed-forward w2(silu(w1 x) * w3 x) (model.py:500-532); also the shared expert of the MoE layer."""

    def __init__(self, dim: int, inter_dim: int):
        super().__init__()
        self.w1 = ColumnParallelLinear(dim, inter_dim)
        self.w2 = RowParallelLinear(inter_dim, dim)
        self.w3 = ColumnParallelLinear(dim, inter_dim)

    stacked: bool = True

    def stack_13(self) -> bool:
        """w1 over w3 in one [2*inter, dim] FP8 buffer (scales likewise), the two layers keeping views of it, so
        that both projections of an input are one GEMM.  Returns whether the layers qualify; re-stacks if the
        layers' storage was moved since (MoE.stack_experts does that for its shared expert)."""
        w1, w3 = self.w1, self.w3
        if w1.weight.element_size() != 1 or w3.weight.element_size() != 1 or w1.out_features % block_size \
                or w1.in_features % block_size or w1.out_features != w3.out_features:
            return False
        w13 = getattr(self, "_w13", None)
        nbytes = w1.out_features * w1.in_features
        if w13 is not None and w13.data_ptr() == w1.weight.data_ptr() and w3.weight.data_ptr() == w13.data_ptr() + nbytes:
            return True
        with torch.no_grad():
            if w3.weight.data_ptr() == w1.weight.data_ptr() + nbytes and \
                    w3.scale.data_ptr() == w1.scale.data_ptr() + w1.scale.numel() * 4:
                # already adjacent (views of a stacked expert buffer): alias instead of copying
                w = torch.as_strided(w1.weight.data, (2 * w1.out_features, w1.in_features), (w1.in_features, 1))
                sc = torch.as_strided(w1.scale.data, (2 * w1.scale.size(0), w1.scale.size(1)), (w1.scale.size(1), 1))
            else:
                w = torch.cat([w1.weight.data.view(torch.uint8), w3.weight.data.view(torch.uint8)]).view(w1.weight.dtype)
                sc = torch.cat([w1.scale.data, w3.scale.data])
                w1.weight.data, w3.weight.data = w[:w1.out_features], w[w1.out_features:]
                w1.scale.data, w3.scale.data = sc[:w1.scale.size(0)], sc[w1.scale.size(0):]
        w.scale = sc
        self._w13 = w
        return True

    def forward(self, x: torch.Tensor, quantised: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
        """``quantised``: ``act_quant(x, block_size)`` (no scale format) where the caller already holds it; the
        stacked projection then starts from it instead of quantising ``x`` once more."""
        if (self.stacked and gemm_impl == "fp8" and world_size == 1 and x.is_cuda and x.dtype == torch.bfloat16
                and x.is_contiguous() and torch.get_default_dtype() == torch.bfloat16 and block_size == 128
                and self.w2.bias is None and self.w1.bias is None and self.w3.bias is None and self.stack_13()):
            # one GEMM for both projections, SwiGLU fused with the re-quantisation of w2's input: the same
            # arithmetic and roundings as the three linears and two tensor ops below
            h = linear(x, self._w13) if quantised is None else fp8_gemm(quantised[0], quantised[1], self._w13, self._w13.scale)
            gq, gs = torch.ops.dsv3fp8.swiglu_quant(h.view(-1, h.size(-1)), block_size, ops._lib.SCALE_FMT_NONE)
            y = fp8_gemm(gq, gs, self.w2.weight, self.w2.weight.scale)
            return y.view(*x.size()[:-1], y.size(-1))
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class Gate(nn.Module):
    """Router (model.py:535-598): scores from a bf16 linear, sigmoid or softmax, an additive selection bias
    (present only for dim == 7168, model.py:564), group-limited top-k, and weights taken from the unbiased
    scores, normalised for sigmoid scoring and multiplied by ``route_scale``."""

    def __init__(self, args: ModelArgs):
        super().__init__()
        self.dim = args.dim
        self.topk = args.n_activated_experts
        self.n_groups = args.n_expert_groups
        self.topk_groups = args.n_limited_groups
        self.score_func = args.score_func
        self.route_scale = args.route_scale
        self.weight = nn.Parameter(torch.empty(args.n_routed_experts, args.dim))
        self.bias = nn.Parameter(torch.empty(args.n_routed_experts, dtype=torch.float32)) if self.dim == 7168 else None

    fused: bool = True

    def _fused_ok(self, scores: torch.Tensor) -> bool:
        experts = scores.size(-1)
        return (self.fused and scores.is_cuda and scores.dtype == torch.bfloat16 and experts <= 512
                and self.topk <= min(64, experts) and self.n_groups <= 64 and experts % self.n_groups == 0
                and self.topk <= self.topk_groups * (experts // self.n_groups))

    def forward(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        scores = linear(x, self.weight)
        if self._fused_ok(scores):
            # everything after the linear layer in one launch (the tensor-op sequence below is what it computes)
            func = ops._lib.SCORE_SOFTMAX if self.score_func == "softmax" else ops._lib.SCORE_SIGMOID
            return torch.ops.dsv3fp8.gate_route(scores.contiguous(), self.bias, self.topk, self.n_groups,
                                                self.topk_groups, func, float(self.route_scale))
        scores = scores.softmax(dim=-1, dtype=torch.float32) if self.score_func == "softmax" else scores.sigmoid()
        unbiased = scores
        if self.bias is not None:
            scores = scores + self.bias
        if self.n_groups > 1:
            grouped = scores.view(x.size(0), self.n_groups, -1)
            group_scores = grouped.amax(dim=-1) if self.bias is None else grouped.topk(2, dim=-1)[0].sum(dim=-1)
            keep = group_scores.topk(self.topk_groups, dim=-1)[1]
            dropped = grouped.new_ones(x.size(0), self.n_groups, dtype=torch.bool).scatter_(1, keep, False)
            scores = grouped.masked_fill(dropped.unsqueeze(-1), float("-inf")).flatten(1)
        indices = torch.topk(scores, self.topk, dim=-1)[1]
        weights = unbiased.gather(1, indices)
        if self.score_func == "sigmoid":
            weights = weights / weights.sum(dim=-1, keepdim=True)
        weights = weights * self.route_scale
        return weights.type_as(x), indices


class Expert(nn.Module):
    """One routed expert: the same SwiGLU as MLP on plain ``Linear`` layers (model.py:601-633), which do
    forward ``Linear.scale_fmt``."""

    def __init__(self, dim: int, inter_dim: int):
        super().__init__()
        self.w1 = Linear(dim, inter_dim)
        self.w2 = Linear(inter_dim, dim)
        self.w3 = Linear(dim, inter_dim)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class MoE(nn.Module):
    """Mixture-of-experts layer (model.py:636-693): route, run every expert that received tokens on its token
    list, scatter-add the weighted outputs in expert order, add the shared expert.

    With FP8 experts and ``gemm_impl == "fp8"`` the token lists stay on the device: the routed experts run as
    two grouped GEMMs over expert-sorted rows (w1|w3 stacked, then w2) with SwiGLU and the re-quantisation fused
    between them, and one kernel adds the weighted outputs per token in the order the reference's loop does.
    ``MoE.grouped = False`` selects the reference's expert-by-expert loop (same kernels, one expert at a time).
    """

    grouped: bool = True
    fold_shared_max_tokens: int = 512
    # True: SwiGLU and the re-quantisation run in the epilogue of the w1|w3 grouped GEMM where the library has that form
    # (tile-kernel launches, bf16 intermediate): the same bits as the two calls, no [pairs, 2*inter] intermediate
    # (268 MB less at 32768 pairs) and equal or a little less time (0-1 % of the layer at 4096 tokens).
    fuse_swiglu_epilogue: bool = True

    def __init__(self, args: ModelArgs):
        super().__init__()
        self.dim = args.dim
        assert args.n_routed_experts % world_size == 0, f"Number of experts must be divisible by world size (world_size={world_size})"
        self.n_routed_experts = args.n_routed_experts
        self.n_local_experts = args.n_routed_experts // world_size
        self.n_activated_experts = args.n_activated_experts
        self.experts_start_idx = rank * self.n_local_experts
        self.experts_end_idx = self.experts_start_idx + self.n_local_experts
        self.gate = Gate(args)
        self.experts = nn.ModuleList([Expert(args.dim, args.moe_inter_dim)
                                      if self.experts_start_idx <= i < self.experts_end_idx else None
                                      for i in range(self.n_routed_experts)])
        self.shared_experts = MLP(args.dim, args.n_shared_experts * args.moe_inter_dim)
        self._stacked = None

    def stack_experts(self) -> None:
        """Move the routed experts' weights into two contiguous buffers, [E, 2*inter, dim] (w1 over w3) and
        [E, dim, inter] (w2), with their scales alongside; each expert's parameters become views of them, so
        ``load_model``-style in-place copies and the expert-by-expert path keep working on the same memory.
        A shared expert of the same shape (``n_shared_experts == 1``) is stacked behind them as entry E, so the
        grouped GEMMs can run it as one more group."""
        if self._stacked is not None:
            return
        exs = list(self.experts)
        inter, dim = exs[0].w1.out_features, self.dim
        assert inter % block_size == 0 and dim % block_size == 0
        dev, fp8 = exs[0].w1.weight.device, exs[0].w1.weight.dtype
        sh = self.shared_experts
        self._shared_stacked = (sh.w1.out_features == inter and sh.w1.weight.dtype == fp8
                                and sh.w1.weight.device == dev)
        if self._shared_stacked:
            exs.append(sh)
        n = len(exs)
        ib, db = inter // block_size, dim // block_size
        with torch.no_grad():
            w13 = torch.empty(n, 2 * inter, dim, dtype=fp8, device=dev)
            s13 = torch.empty(n, 2 * ib, db, dtype=torch.float32, device=dev)
            w2 = torch.empty(n, dim, inter, dtype=fp8, device=dev)
            s2 = torch.empty(n, db, ib, dtype=torch.float32, device=dev)
            for i, ex in enumerate(exs):
                for lin, wv, sv in ((ex.w1, w13[i, :inter], s13[i, :ib]), (ex.w3, w13[i, inter:], s13[i, ib:]),
                                    (ex.w2, w2[i], s2[i])):
                    wv.view(torch.uint8).copy_(lin.weight.data.view(torch.uint8))
                    sv.copy_(lin.scale.data)
                    lin.weight.data = wv
                    lin.scale.data = sv
        self._stacked = (w13, s13, w2, s2)

    def _grouped_ok(self, x: torch.Tensor) -> bool:
        ex = self.experts[self.experts_start_idx]
        inter = ex.w1.out_features
        pairs = x.size(0) * self.n_activated_experts
        # the grouped kernels' limits: up to 16 experts per token, 32-bit offsets into the gathered rows and into x
        fits = (0 < x.size(0) and self.n_activated_experts <= 16 and pairs * max(inter, self.dim) < 2 ** 32
                and x.size(0) * self.dim < 2 ** 32)
        return (self.grouped and fits and gemm_impl == "fp8" and world_size == 1 and x.is_cuda
                and ex.w1.weight.element_size() == 1 and x.dtype == torch.bfloat16
                and torch.get_default_dtype() == torch.bfloat16
                and ex.w1.out_features % block_size == 0 and self.dim % block_size == 0)

    def _forward_grouped(self, x: torch.Tensor, weights: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        self.stack_experts()
        w13, s13, w2, s2 = self._stacked
        # Few tokens: the shared expert rides along as group E that every token selects with weight 1 -- it has the
        # highest index, so the ordered combine adds it last, bf16(y + bf16(z * 1)) = bf16(y + z), exactly where
        # the reference adds z.  That saves its three separate GEMM + quantise launches; with many tokens the dense
        # large-M kernel runs it faster than 128-row groups do.  Its linears never take scale_fmt (model.py:233,
        # 262), so the shortcut needs the routed experts to use none either.
        fold = (self._shared_stacked and Linear.scale_fmt is None and indices.size(0) <= self.fold_shared_max_tokens
                and indices.size(1) < 16)
        if not fold:
            w13, s13, w2, s2 = (t[:self.n_routed_experts] for t in self._stacked)
        # counts per expert, expert-sorted token list, each token's rows in ascending expert order (the order in
        # which the reference's loop adds them, model.py:684-689) and the tile table -- all on the device
        _, a_rows, rows, w_sorted, tile_group, tile_row0, tile_rows = torch.ops.dsv3fp8.moe_route(
            indices.contiguous(), weights.contiguous(), self.n_routed_experts, fold)
        pairs = rows.numel()
        fmt = ops._lib.SCALE_FMT_UE8M0 if Linear.scale_fmt == "ue8m0" else ops._lib.SCALE_FMT_NONE
        code = ops.dtype_code(torch.get_default_dtype())
        xq, xs = act_quant(x, block_size, Linear.scale_fmt)           # quantised once: 1x128 blocks are per token
        # power-of-two activation scales on experts whose block scales are powers of two as well: the scales go
        # into the matrix instruction (the whole stacked buffers are looked at, once per version of their contents)
        pow2 = (Linear.scale_fmt == "ue8m0" and _scales_are_powers_of_two(self._stacked[0], self._stacked[1])
                and _scales_are_powers_of_two(self._stacked[2], self._stacked[3]))
        gemm = torch.ops.dsv3fp8.fp8_gemm_grouped_pow2 if pow2 else torch.ops.dsv3fp8.fp8_gemm_grouped
        if self.fuse_swiglu_epilogue and not pow2 and torch.get_default_dtype() == torch.bfloat16:
            gq, gs = torch.ops.dsv3fp8.fp8_gemm_grouped_swiglu(xq, xs, a_rows, w13, s13, pairs, tile_group, tile_row0,
                                                               tile_rows, fmt)
        else:
            h = gemm(xq, xs, a_rows, w13, s13, pairs, tile_group, tile_row0, tile_rows, code)
            gq, gs = torch.ops.dsv3fp8.swiglu_quant(h, block_size, fmt)
        out = gemm(gq, gs, None, w2, s2, pairs, tile_group, tile_row0, tile_rows, code)
        # (the shared expert's linears quantise x with no scale format, model.py:233: xq serves them when the routed
        # experts use none either)
        z = None if fold else self.shared_experts(x, (xq, xs) if Linear.scale_fmt is None else None).contiguous()
        return torch.ops.dsv3fp8.moe_combine(out, rows, w_sorted, z)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shape = x.size()
        x = x.view(-1, self.dim)
        weights, indices = self.gate(x)
        if self._grouped_ok(x):
            return self._forward_grouped(x, weights, indices).view(shape)
        y = torch.zeros_like(x)
        counts = torch.bincount(indices.flatten(), minlength=self.n_routed_experts).tolist()
        for i in range(self.experts_start_idx, self.experts_end_idx):
            if counts[i] == 0:
                continue
            idx, top = torch.where(indices == i)
            y[idx] += self.experts[i](x[idx]) * weights[idx, top, None]
        z = self.shared_experts(x)
        return (y + z).view(shape)
