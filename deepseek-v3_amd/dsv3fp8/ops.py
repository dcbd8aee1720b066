"""PyTorch-ROCm custom ops over the C ABI.

``torch.ops.dsv3fp8.{act_quant, weight_dequant, weight_quant, fp8_gemm}`` and the grouped
mixture-of-experts ops ``{gate_route, group_tiles, moe_route, fp8_gemm_grouped, swiglu_quant, moe_combine}`` and the
attention op ``wkv_b_absorb`` take and return torch tensors; the device implementations hand raw device pointers and the
current HIP stream of the tensors' device to libdsv3fp8.so.  Only a device
("CUDA" dispatch key, which is HIP on ROCm) implementation and a shape-only Meta
implementation are registered: calling an op on CPU tensors raises.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.float32: _lib.F32}
_CODE_DTYPE = {v: k for k, v in _DTYPE_CODE.items()}
FP8 = torch.float8_e4m3fn

_libdef = torch.library.Library("dsv3fp8", "DEF")
_libdef.define("act_quant(Tensor x, int block_size, int scale_fmt) -> (Tensor, Tensor)")
_libdef.define("weight_dequant(Tensor x, Tensor s, int block_size, int out_dtype) -> Tensor")
_libdef.define("weight_quant(Tensor w, int block_size, int scale_fmt) -> (Tensor, Tensor)")
_libdef.define("fp8_gemm(Tensor a, Tensor a_s, Tensor b, Tensor b_s, int out_dtype) -> Tensor")
_libdef.define("fp8_gemm_pow2(Tensor a, Tensor a_s, Tensor b, Tensor b_s, int out_dtype) -> Tensor")
_libdef.define("linear_fp8(Tensor x, Tensor b, Tensor b_s, int scale_fmt, int out_dtype) -> Tensor")
_libdef.define("group_tiles(Tensor counts, int max_tiles) -> (Tensor, Tensor, Tensor)")
_libdef.define("moe_route(Tensor indices, Tensor weights, int experts, bool shared_group) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)")
_libdef.define("fp8_gemm_grouped(Tensor a, Tensor a_s, Tensor? a_rows, Tensor b, Tensor b_s, int rows, "
               "Tensor tile_group, Tensor tile_row0, Tensor tile_rows, int out_dtype) -> Tensor")
_libdef.define("fp8_gemm_grouped_swiglu(Tensor a, Tensor a_s, Tensor? a_rows, Tensor b, Tensor b_s, int rows, "
               "Tensor tile_group, Tensor tile_row0, Tensor tile_rows, int scale_fmt) -> (Tensor, Tensor)")
_libdef.define("fp8_gemm_grouped_pow2(Tensor a, Tensor a_s, Tensor? a_rows, Tensor b, Tensor b_s, int rows, "
               "Tensor tile_group, Tensor tile_row0, Tensor tile_rows, int out_dtype) -> Tensor")
_libdef.define("swiglu_quant(Tensor h, int block_size, int scale_fmt) -> (Tensor, Tensor)")
_libdef.define("moe_combine(Tensor expert_out, Tensor rows, Tensor weights, Tensor? shared) -> Tensor")
_libdef.define("gate_route(Tensor logits, Tensor? bias, int topk, int n_groups, int topk_groups, int score_func, "
               "float route_scale) -> (Tensor, Tensor)")
_libdef.define("wkv_b_absorb(Tensor x, Tensor wkv_b, Tensor scale, int side, int nope_dim, int v_dim) -> Tensor")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"dsv3fp8: unsupported dtype {dtype} (bf16, fp16 and fp32 are implemented)") from None


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


# split-K scratch, one buffer per (device, stream): calls on one stream are ordered, so they can share it
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _workspace(t: torch.Tensor, nbytes: int, stream: int) -> torch.Tensor:
    # Under stream capture the scratch comes from the graph's own memory pool and lives as long as the graph: the
    # cached buffer below is replaced when a larger one is needed, which would leave a graph that had captured it
    # replaying into freed memory.
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=t.device)
    key = (t.device.index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 22), dtype=torch.uint8, device=t.device)
        _workspaces[key] = ws
    return ws


def _act_quant_dev(x: torch.Tensor, block_size: int, scale_fmt: int):
    y = torch.empty_like(x, dtype=FP8)
    s = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32)
    with torch.cuda.device(x.device):
        rc = _lib.lib.dsv3_act_quant(x.data_ptr(), dtype_code(x.dtype), y.data_ptr(), s.data_ptr(),
                                     x.numel(), x.size(-1), block_size, scale_fmt, _stream(x))
    _lib.check(rc, "dsv3_act_quant")
    return y, s


def _act_quant_meta(x, block_size, scale_fmt):
    return (torch.empty_like(x, dtype=FP8),
            x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32))


def _weight_dequant_dev(x: torch.Tensor, s: torch.Tensor, block_size: int, out_dtype: int):
    y = torch.empty_like(x, dtype=_CODE_DTYPE[out_dtype])
    m, n = x.size()
    with torch.cuda.device(x.device):
        rc = _lib.lib.dsv3_weight_dequant(x.data_ptr(), s.data_ptr(), y.data_ptr(), out_dtype,
                                          m, n, block_size, _stream(x))
    _lib.check(rc, "dsv3_weight_dequant")
    return y


def _weight_dequant_meta(x, s, block_size, out_dtype):
    return torch.empty_like(x, dtype=_CODE_DTYPE[out_dtype])


def _weight_quant_dev(w: torch.Tensor, block_size: int, scale_fmt: int):
    m, n = w.size()
    y = torch.empty_like(w, dtype=FP8)
    s = w.new_empty(-(-m // block_size), -(-n // block_size), dtype=torch.float32)
    with torch.cuda.device(w.device):
        rc = _lib.lib.dsv3_weight_quant(w.data_ptr(), dtype_code(w.dtype), y.data_ptr(), s.data_ptr(), m, n,
                                        block_size, scale_fmt, _stream(w))
    _lib.check(rc, "dsv3_weight_quant")
    return y, s


def _weight_quant_meta(w, block_size, scale_fmt):
    m, n = w.size()
    return torch.empty_like(w, dtype=FP8), w.new_empty(-(-m // block_size), -(-n // block_size), dtype=torch.float32)


def _fp8_gemm_dev(a, a_s, b, b_s, out_dtype: int, entry: str = "dsv3_fp8_gemm"):
    k = a.size(-1)
    m = a.numel() // k if k else 0
    n = b.size(0)
    c = a.new_empty(*a.size()[:-1], n, dtype=_CODE_DTYPE[out_dtype])
    with torch.cuda.device(a.device):
        stream = _stream(a)
        need = _lib.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k)
        ws = _workspace(a, need, stream) if need else None
        rc = getattr(_lib.lib, entry)(a.data_ptr(), a_s.data_ptr(), b.data_ptr(), b_s.data_ptr(),
                                      c.data_ptr(), out_dtype, m, n, k,
                                      ws.data_ptr() if ws is not None else None,
                                      ws.numel() if ws is not None else 0, stream)
    _lib.check(rc, entry)
    return c


def _fp8_gemm_pow2_dev(a, a_s, b, b_s, out_dtype: int):
    return _fp8_gemm_dev(a, a_s, b, b_s, out_dtype, "dsv3_fp8_gemm_pow2")


def _fp8_gemm_meta(a, a_s, b, b_s, out_dtype):
    return a.new_empty(*a.size()[:-1], b.size(0), dtype=_CODE_DTYPE[out_dtype])


def linear_fp8_fused(m: int, n: int, k: int) -> bool:
    """Whether act_quant + fp8_gemm of an [m, k] x [n, k] linear run as one launch (dsv3_linear_fp8)."""
    return bool(_lib.lib.dsv3_linear_fp8_fused(m, n, k))


def _linear_fp8_dev(x, b, b_s, scale_fmt: int, out_dtype: int):
    """act_quant(x, 128, scale_fmt) followed by fp8_gemm, fused where the library implements it, else two calls."""
    k = x.size(-1)
    m = x.numel() // k if k else 0
    n = b.size(0)
    if not (x.dtype == torch.bfloat16 and linear_fp8_fused(m, n, k)):
        a, a_s = _act_quant_dev(x, 128, scale_fmt)
        return _fp8_gemm_dev(a, a_s, b, b_s, out_dtype)
    c = x.new_empty(*x.size()[:-1], n, dtype=_CODE_DTYPE[out_dtype])
    with torch.cuda.device(x.device):
        stream = _stream(x)
        need = _lib.lib.dsv3_fp8_gemm_workspace_bytes(m, n, k)
        ws = _workspace(x, need, stream) if need else None
        rc = _lib.lib.dsv3_linear_fp8(x.data_ptr(), _lib.BF16, b.data_ptr(), b_s.data_ptr(), c.data_ptr(), out_dtype,
                                      m, n, k, 128, scale_fmt, ws.data_ptr() if ws is not None else None,
                                      ws.numel() if ws is not None else 0, stream)
    _lib.check(rc, "dsv3_linear_fp8")
    return c


def _linear_fp8_meta(x, b, b_s, scale_fmt, out_dtype):
    return x.new_empty(*x.size()[:-1], b.size(0), dtype=_CODE_DTYPE[out_dtype])


def grouped_tile_rows() -> int:
    return int(_lib.lib.dsv3_fp8_gemm_grouped_tile_rows())


def _group_tiles_dev(counts: torch.Tensor, max_tiles: int):
    assert counts.dtype == torch.int32 and counts.is_contiguous() and counts.dim() == 1
    out = torch.empty(3, max(max_tiles, 1), dtype=torch.int32, device=counts.device)
    with torch.cuda.device(counts.device):
        rc = _lib.lib.dsv3_group_tiles(counts.data_ptr(), counts.numel(), max_tiles,
                                       out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(), _stream(counts))
    _lib.check(rc, "dsv3_group_tiles")
    return out[0, :max_tiles], out[1, :max_tiles], out[2, :max_tiles]


def _group_tiles_meta(counts, max_tiles):
    return tuple(counts.new_empty(max_tiles, dtype=torch.int32) for _ in range(3))


def _moe_route_dev(indices: torch.Tensor, weights: torch.Tensor, experts: int, shared_group: bool):
    """-> counts [groups], a_rows [tokens*cols], rows [tokens, cols], w_sorted [tokens, cols], tile_group,
    tile_row0, tile_rows, with groups = experts (+1) and cols = topk (+1 with shared_group); see dsv3_moe_route
    in include/dsv3_fp8.h."""
    assert indices.dtype == torch.int64 and indices.dim() == 2 and indices.is_contiguous()
    assert weights.shape == indices.shape and weights.is_contiguous() and weights.element_size() == 2
    tokens, topk = indices.shape
    groups, cols = experts + int(shared_group), topk + int(shared_group)
    pairs = tokens * cols
    max_tiles = pairs // grouped_tile_rows() + groups
    dev = indices.device
    ints = torch.empty(3 * groups + pairs + pairs + 3 * max_tiles, dtype=torch.int32, device=dev)
    scratch, a_rows, rows, tiles = ints.split([3 * groups, pairs, pairs, 3 * max_tiles])
    tiles = tiles.view(3, max_tiles)
    w_sorted = weights.new_empty(tokens, cols)
    with torch.cuda.device(dev):
        rc = _lib.lib.dsv3_moe_route(indices.data_ptr(), weights.data_ptr(), dtype_code(weights.dtype), tokens, topk,
                                     experts, int(shared_group), max_tiles, scratch.data_ptr(), a_rows.data_ptr(),
                                     rows.data_ptr(), w_sorted.data_ptr(), tiles[0].data_ptr(), tiles[1].data_ptr(),
                                     tiles[2].data_ptr(), _stream(indices))
    _lib.check(rc, "dsv3_moe_route")
    return scratch[:groups], a_rows, rows.view(tokens, cols), w_sorted, tiles[0], tiles[1], tiles[2]


def _moe_route_meta(indices, weights, experts, shared_group):
    tokens, topk = indices.shape
    groups, cols = experts + int(shared_group), topk + int(shared_group)
    pairs = tokens * cols
    max_tiles = pairs // grouped_tile_rows() + groups
    i32 = lambda *shape: indices.new_empty(*shape, dtype=torch.int32)
    return (i32(groups), i32(pairs), i32(tokens, cols), weights.new_empty(tokens, cols), i32(max_tiles), i32(max_tiles),
            i32(max_tiles))


def _fp8_gemm_grouped_dev(a, a_s, a_rows, b, b_s, rows: int, tile_group, tile_row0, tile_rows, out_dtype: int,
                          entry: str = "dsv3_fp8_gemm_grouped"):
    # a: [A, k] fp8; b: [groups, n, k] fp8; b_s: [groups, ceil(n/128), k/128]; result [rows, n]
    assert a.dim() == 2 and b.dim() == 3 and b_s.dim() == 3 and a.is_contiguous() and b.is_contiguous()
    assert a_s.is_contiguous() and b_s.is_contiguous() and b.size(0) == b_s.size(0)
    for t in (tile_group, tile_row0, tile_rows):
        assert t.dtype == torch.int32 and t.is_contiguous() and t.numel() == tile_group.numel()
    if a_rows is not None:
        assert a_rows.dtype == torch.int32 and a_rows.is_contiguous() and a_rows.numel() == rows
    k, n = a.size(1), b.size(1)
    assert b.size(2) == k
    c = a.new_empty(rows, n, dtype=_CODE_DTYPE[out_dtype])
    with torch.cuda.device(a.device):
        rc = getattr(_lib.lib, entry)(
            a.data_ptr(), a_s.data_ptr(), a_rows.data_ptr() if a_rows is not None else None, a.size(0),
            b.data_ptr(), b_s.data_ptr(), b.stride(0), b_s.stride(0),
            c.data_ptr(), out_dtype, rows, n, k,
            tile_group.data_ptr(), tile_row0.data_ptr(), tile_rows.data_ptr(), tile_group.numel(), _stream(a))
    _lib.check(rc, entry)
    return c


def _fp8_gemm_grouped_pow2_dev(a, a_s, a_rows, b, b_s, rows: int, tile_group, tile_row0, tile_rows, out_dtype: int):
    return _fp8_gemm_grouped_dev(a, a_s, a_rows, b, b_s, rows, tile_group, tile_row0, tile_rows, out_dtype,
                                 "dsv3_fp8_gemm_grouped_pow2")


def _fp8_gemm_grouped_meta(a, a_s, a_rows, b, b_s, rows, tile_group, tile_row0, tile_rows, out_dtype):
    return a.new_empty(rows, b.size(1), dtype=_CODE_DTYPE[out_dtype])


def grouped_swiglu_fused(rows: int, a_num_rows: int, inter: int, k: int) -> bool:
    """Whether the first grouped GEMM of a SwiGLU block can carry the activation and the re-quantisation in its
    epilogue (dsv3_fp8_gemm_grouped_swiglu) for a launch of this size."""
    return bool(_lib.lib.dsv3_fp8_gemm_grouped_swiglu_fused(rows, a_num_rows, inter, k))


def _fp8_gemm_grouped_swiglu_dev(a, a_s, a_rows, b, b_s, rows: int, tile_group, tile_row0, tile_rows, scale_fmt: int):
    """fp8_gemm_grouped over b = [w1 ; w3] per group followed by swiglu_quant, fused where the library implements it
    (the same bits either way); returns (y [rows, inter] e4m3, s [rows, inter / 128])."""
    k, inter = a.size(1), b.size(1) // 2
    if not grouped_swiglu_fused(rows, a.size(0), inter, k):
        h = _fp8_gemm_grouped_dev(a, a_s, a_rows, b, b_s, rows, tile_group, tile_row0, tile_rows, _lib.BF16)
        return _swiglu_quant_dev(h, 128, scale_fmt)
    assert a.dim() == 2 and b.dim() == 3 and b_s.dim() == 3 and a.is_contiguous() and b.is_contiguous()
    assert a_s.is_contiguous() and b_s.is_contiguous() and b.size(0) == b_s.size(0) and b.size(2) == k
    for t in (tile_group, tile_row0, tile_rows):
        assert t.dtype == torch.int32 and t.is_contiguous() and t.numel() == tile_group.numel()
    if a_rows is not None:
        assert a_rows.dtype == torch.int32 and a_rows.is_contiguous() and a_rows.numel() == rows
    y = a.new_empty(rows, inter, dtype=FP8)
    s = a.new_empty(rows, inter // 128, dtype=torch.float32)
    with torch.cuda.device(a.device):
        rc = _lib.lib.dsv3_fp8_gemm_grouped_swiglu(
            a.data_ptr(), a_s.data_ptr(), a_rows.data_ptr() if a_rows is not None else None, a.size(0),
            b.data_ptr(), b_s.data_ptr(), b.stride(0), b_s.stride(0), y.data_ptr(), s.data_ptr(), rows, inter, k,
            tile_group.data_ptr(), tile_row0.data_ptr(), tile_rows.data_ptr(), tile_group.numel(), 128, scale_fmt,
            _stream(a))
    _lib.check(rc, "dsv3_fp8_gemm_grouped_swiglu")
    return y, s


def _fp8_gemm_grouped_swiglu_meta(a, a_s, a_rows, b, b_s, rows, tile_group, tile_row0, tile_rows, scale_fmt):
    inter = b.size(1) // 2
    return a.new_empty(rows, inter, dtype=FP8), a.new_empty(rows, inter // 128, dtype=torch.float32)


def _swiglu_quant_dev(h: torch.Tensor, block_size: int, scale_fmt: int):
    assert h.dim() == 2 and h.is_contiguous() and h.size(1) % 2 == 0
    rows, inter = h.size(0), h.size(1) // 2
    y = h.new_empty(rows, inter, dtype=FP8)
    s = h.new_empty(rows, inter // block_size, dtype=torch.float32)
    with torch.cuda.device(h.device):
        rc = _lib.lib.dsv3_swiglu_quant(h.data_ptr(), dtype_code(h.dtype), y.data_ptr(), s.data_ptr(),
                                        rows, inter, block_size, scale_fmt, _stream(h))
    _lib.check(rc, "dsv3_swiglu_quant")
    return y, s


def _swiglu_quant_meta(h, block_size, scale_fmt):
    rows, inter = h.size(0), h.size(1) // 2
    return h.new_empty(rows, inter, dtype=FP8), h.new_empty(rows, inter // block_size, dtype=torch.float32)


def _moe_combine_dev(expert_out, rows, weights, shared):
    assert expert_out.dim() == 2 and expert_out.is_contiguous() and rows.dtype == torch.int32
    assert rows.is_contiguous() and weights.is_contiguous() and rows.shape == weights.shape
    assert weights.dtype == expert_out.dtype and (shared is None or (shared.is_contiguous() and shared.dtype == expert_out.dtype))
    tokens, topk = rows.shape
    y = expert_out.new_empty(tokens, expert_out.size(1))
    with torch.cuda.device(expert_out.device):
        rc = _lib.lib.dsv3_moe_combine(expert_out.data_ptr(), dtype_code(expert_out.dtype), rows.data_ptr(),
                                       weights.data_ptr(), shared.data_ptr() if shared is not None else None,
                                       y.data_ptr(), tokens, topk, expert_out.size(1), _stream(expert_out))
    _lib.check(rc, "dsv3_moe_combine")
    return y


def _moe_combine_meta(expert_out, rows, weights, shared):
    return expert_out.new_empty(rows.size(0), expert_out.size(1))


def _gate_route_dev(logits, bias, topk: int, n_groups: int, topk_groups: int, score_func: int, route_scale: float):
    assert logits.dim() == 2 and logits.is_contiguous() and logits.dtype == torch.bfloat16
    assert bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == logits.size(1))
    tokens, experts = logits.shape
    weights = logits.new_empty(tokens, topk)
    indices = torch.empty(tokens, topk, dtype=torch.int64, device=logits.device)
    with torch.cuda.device(logits.device):
        rc = _lib.lib.dsv3_gate_route(logits.data_ptr(), _lib.BF16, bias.data_ptr() if bias is not None else None,
                                      weights.data_ptr(), indices.data_ptr(), tokens, experts, topk, n_groups,
                                      topk_groups, score_func, route_scale, _stream(logits))
    _lib.check(rc, "dsv3_gate_route")
    return weights, indices


def _gate_route_meta(logits, bias, topk, n_groups, topk_groups, score_func, route_scale):
    return logits.new_empty(logits.size(0), topk), logits.new_empty(logits.size(0), topk, dtype=torch.int64)


def _absorb_out_dim(wkv_b, side: int, v_dim: int) -> int:
    return wkv_b.size(1) if side == _lib.ABSORB_Q else v_dim


def _wkv_b_absorb_dev(x, wkv_b, scale, side: int, nope_dim: int, v_dim: int):
    # x: [..., heads, in] bf16, innermost dimension contiguous, leading dimensions collapsible into one token axis
    # (the q_nope slice of q is such a view); wkv_b: [heads*(nope_dim+v_dim), kv_rank] fp8 with its block scales
    assert x.dim() >= 2 and x.stride(-1) == 1 and x.dtype == torch.bfloat16
    assert wkv_b.dim() == 2 and wkv_b.is_contiguous() and scale.is_contiguous() and wkv_b.element_size() == 1
    heads = x.size(-2)
    assert wkv_b.size(0) == heads * (nope_dim + v_dim), "wkv_b rows must be heads * (nope_dim + v_dim)"
    assert x.size(-1) == (nope_dim if side == _lib.ABSORB_Q else wkv_b.size(1))
    xt = x.view(-1, heads, x.size(-1))
    y = x.new_empty(*x.size()[:-1], _absorb_out_dim(wkv_b, side, v_dim))
    with torch.cuda.device(x.device):
        rc = _lib.lib.dsv3_wkv_b_absorb(xt.data_ptr(), xt.stride(0), xt.stride(1), wkv_b.data_ptr(), scale.data_ptr(),
                                        y.data_ptr(), _lib.BF16, side, xt.size(0), heads, nope_dim, v_dim,
                                        wkv_b.size(1), 128, _stream(x))
    _lib.check(rc, "dsv3_wkv_b_absorb")
    return y


def _wkv_b_absorb_meta(x, wkv_b, scale, side, nope_dim, v_dim):
    return x.new_empty(*x.size()[:-1], _absorb_out_dim(wkv_b, side, v_dim))


_libimpl = torch.library.Library("dsv3fp8", "IMPL")
for _name, _dev, _meta in (("wkv_b_absorb", _wkv_b_absorb_dev, _wkv_b_absorb_meta),
                           ("linear_fp8", _linear_fp8_dev, _linear_fp8_meta),
                           ("gate_route", _gate_route_dev, _gate_route_meta),
                           ("group_tiles", _group_tiles_dev, _group_tiles_meta),
                           ("moe_route", _moe_route_dev, _moe_route_meta),
                           ("fp8_gemm_grouped", _fp8_gemm_grouped_dev, _fp8_gemm_grouped_meta),
                           ("fp8_gemm_grouped_pow2", _fp8_gemm_grouped_pow2_dev, _fp8_gemm_grouped_meta),
                           ("fp8_gemm_grouped_swiglu", _fp8_gemm_grouped_swiglu_dev, _fp8_gemm_grouped_swiglu_meta),
                           ("swiglu_quant", _swiglu_quant_dev, _swiglu_quant_meta),
                           ("moe_combine", _moe_combine_dev, _moe_combine_meta)):
    _libimpl.impl(_name, _dev, "CUDA")
    _libimpl.impl(_name, _meta, "Meta")
_libimpl.impl("act_quant", _act_quant_dev, "CUDA")
_libimpl.impl("weight_dequant", _weight_dequant_dev, "CUDA")
_libimpl.impl("weight_quant", _weight_quant_dev, "CUDA")
_libimpl.impl("fp8_gemm", _fp8_gemm_dev, "CUDA")
_libimpl.impl("fp8_gemm_pow2", _fp8_gemm_pow2_dev, "CUDA")
_libimpl.impl("act_quant", _act_quant_meta, "Meta")
_libimpl.impl("weight_dequant", _weight_dequant_meta, "Meta")
_libimpl.impl("weight_quant", _weight_quant_meta, "Meta")
_libimpl.impl("fp8_gemm", _fp8_gemm_meta, "Meta")
_libimpl.impl("fp8_gemm_pow2", _fp8_gemm_meta, "Meta")
