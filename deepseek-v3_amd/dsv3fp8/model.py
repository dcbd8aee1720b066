"""Host-side callers of the FP8 kernels, mirroring the part of the reference's
``inference/model.py`` that sits directly on top of them: the ``linear()``
dispatch (model.py:131-163), ``Linear`` and its column/row parallel variants
(model.py:166-267), and the SwiGLU / routing modules that issue the FP8 linears
of the MoE layer (``MLP`` :500-532, ``Gate`` :535-598, ``Expert`` :601-633,
``MoE`` :636-693).  Names, constructor arguments, the ``weight.scale``
convention and the module-level switches (``gemm_impl``, ``block_size``) follow
the reference so that code written against it runs unchanged.

This build runs on one GPU: ``world_size`` is fixed at 1, so the parallel
variants reduce to plain ``Linear`` and no collective is issued.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Literal, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .kernel import act_quant, fp8_gemm, weight_dequant

world_size = 1
rank = 0
block_size = 128
gemm_impl: Literal["bf16", "fp8"] = "bf16"     # the reference's default (model.py:16); set to "fp8" for the FP8 GEMM path


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


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           scale_fmt: Optional[str] = None) -> torch.Tensor:
    """y = x @ weight.T + bias with the reference's three-way dispatch (model.py:153-163): wide weights go to
    ``F.linear``; 1-byte weights are dequantised first when ``gemm_impl == "bf16"``, otherwise the activation
    is quantised per 1x128 block and multiplied with ``fp8_gemm``.  ``weight.scale`` carries the block scales."""
    if weight.element_size() > 1:
        return F.linear(x, weight, bias)
    if gemm_impl == "bf16":
        return F.linear(x, weight_dequant(weight, weight.scale), bias)
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


class MLP(nn.Module):
    """SwiGLU feed-forward w2(silu(w1 x) * w3 x) (model.py:500-532); also the shared expert of the MoE layer."""

    def __init__(self, dim: int, inter_dim: int):
        super().__init__()
        self.w1 = ColumnParallelLinear(dim, inter_dim)
        self.w2 = RowParallelLinear(inter_dim, dim)
        self.w3 = ColumnParallelLinear(dim, inter_dim)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
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

    def forward(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        scores = linear(x, self.weight)
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
        ``load_model``-style in-place copies and the expert-by-expert path keep working on the same memory."""
        if self._stacked is not None:
            return
        exs = list(self.experts)
        inter, dim = exs[0].w1.out_features, self.dim
        assert inter % block_size == 0 and dim % block_size == 0
        dev, fp8 = exs[0].w1.weight.device, exs[0].w1.weight.dtype
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
        return (self.grouped and gemm_impl == "fp8" and world_size == 1 and x.is_cuda
                and ex.w1.weight.element_size() == 1 and x.dtype == torch.bfloat16
                and torch.get_default_dtype() == torch.bfloat16
                and ex.w1.out_features % block_size == 0 and self.dim % block_size == 0)

    def _forward_grouped(self, x: torch.Tensor, weights: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        self.stack_experts()
        w13, s13, w2, s2 = self._stacked
        tokens, topk = indices.shape
        pairs = tokens * topk
        # counts per expert, expert-sorted token list, each token's rows in ascending expert order (the order in
        # which the reference's loop adds them, model.py:684-689) and the tile table -- all on the device
        _, a_rows, rows, w_sorted, tile_group, tile_row0, tile_rows = torch.ops.dsv3fp8.moe_route(
            indices.contiguous(), weights.contiguous(), self.n_routed_experts)
        fmt = ops._lib.SCALE_FMT_UE8M0 if Linear.scale_fmt == "ue8m0" else ops._lib.SCALE_FMT_NONE
        code = ops.dtype_code(torch.get_default_dtype())
        xq, xs = act_quant(x, block_size, Linear.scale_fmt)           # quantised once: 1x128 blocks are per token
        h = torch.ops.dsv3fp8.fp8_gemm_grouped(xq, xs, a_rows, w13, s13, pairs, tile_group, tile_row0, tile_rows, code)
        gq, gs = torch.ops.dsv3fp8.swiglu_quant(h, block_size, fmt)
        out = torch.ops.dsv3fp8.fp8_gemm_grouped(gq, gs, None, w2, s2, pairs, tile_group, tile_row0, tile_rows, code)
        z = self.shared_experts(x)
        return torch.ops.dsv3fp8.moe_combine(out, rows, w_sorted, z.contiguous())

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
