"""Host-side contract of libdsv3fp8.so: it loads without a GPU, exports every symbol
include/dsv3_fp8.h declares, and validates arguments before touching HIP."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "dsv3_fp8.h"


@pytest.fixture(scope="module")
def L():
    from dsv3fp8 import _lib
    return _lib


def test_exports_every_declared_symbol(L):
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    declared = set(re.findall(r"\b(dsv3_[a-z0-9_]+)\s*\(", text))
    assert declared == set(L.EXPORTS), (declared, set(L.EXPORTS))
    for name in declared:
        assert hasattr(L.lib, name)
    assert L.lib.dsv3_version() >= 100


def test_status_strings(L):
    seen = {L.status_string(c) for c in range(8)}
    assert len(seen) == 8 and "ok" in seen
    assert L.status_string(12345) == "unknown status"


A16 = 0x1000  # a fake, 16-byte aligned, non-null address: validation must reject before dereferencing


def test_act_quant_validation(L):
    f = L.lib.dsv3_act_quant
    assert f(None, L.BF16, A16, A16, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, None, A16, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, A16, None, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, A16, A16, 100, 100, 128, 0, None) == 2        # last dim % block (kernel.py:52)
    assert f(A16, L.BF16, A16, A16, -128, 128, 128, 0, None) == 2
    assert f(A16, L.BF16, A16, A16, 384, 256, 128, 0, None) == 2        # numel not a multiple of last dim
    assert f(A16, L.BF16, A16, A16, 128, 128, 100, 0, None) == 2        # any block size, but it must divide the last dim
    assert f(A16, L.BF16, A16, A16, 128, 128, 0, 0, None) == 3
    assert f(A16, L.BF16, A16, A16, 128, 128, -128, 0, None) == 3
    assert f(A16 + 2, L.BF16, A16, A16, 128, 128, 128, 0, None) == 4
    assert f(A16, 9, A16, A16, 128, 128, 128, 0, None) == 5
    assert f(A16, L.BF16, A16, A16, 128, 128, 128, 7, None) == 5
    assert f(None, L.BF16, None, None, 0, 128, 128, 0, None) == 0       # empty input: nothing to do


def test_weight_dequant_validation(L):
    f = L.lib.dsv3_weight_dequant
    assert f(None, A16, A16, L.BF16, 128, 128, 128, None) == 1
    assert f(A16, None, A16, L.BF16, 128, 128, 128, None) == 1
    assert f(A16, A16, None, L.BF16, 128, 128, 128, None) == 1
    assert f(A16, A16, A16, L.BF16, -1, 128, 128, None) == 2
    assert f(A16, A16, A16, L.BF16, 128, 128, 0, None) == 3
    assert f(A16, A16, A16, 5, 128, 128, 128, None) == 5
    assert f(A16, A16, A16 + 1, L.BF16, 128, 128, 128, None) == 4
    assert f(None, None, None, L.BF16, 0, 128, 128, None) == 0


def test_weight_quant_validation(L):
    f = L.lib.dsv3_weight_quant
    assert f(None, L.BF16, A16, A16, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, None, A16, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, A16, None, 128, 128, 128, 0, None) == 1
    assert f(A16, L.BF16, A16, A16, 128, -1, 128, 0, None) == 2
    assert f(A16, L.BF16, A16, A16, 128, 128, 64, 0, None) == 3         # only 128 x 128 blocks exist on disk
    assert f(A16, L.BF16, A16, A16, 128, 128, 128, 5, None) == 5        # unknown scale format
    assert f(A16, 7, A16, A16, 128, 128, 128, 0, None) == 5
    assert f(A16 + 1, L.BF16, A16, A16, 128, 128, 128, 0, None) == 4
    assert f(A16, L.BF16, A16, A16 + 2, 128, 128, 128, 0, None) == 4
    assert f(None, L.BF16, None, None, 0, 128, 128, 0, None) == 0


@pytest.mark.parametrize("entry", ["dsv3_fp8_gemm", "dsv3_fp8_gemm_pow2"])
def test_fp8_gemm_validation(L, entry):
    f = getattr(L.lib, entry)
    ws = L.lib.dsv3_fp8_gemm_workspace_bytes
    assert f(None, A16, A16, A16, A16, L.BF16, 4, 128, 128, None, 0, None) == 1
    assert f(A16, A16, A16, A16, None, L.BF16, 4, 128, 128, None, 0, None) == 1
    assert f(A16, A16, A16, A16, A16, L.BF16, 70000, 128, 100, None, 0, None) == 2    # K % 128 != 0 is served by a fallback whose grid takes m <= 65535
    assert f(A16, A16, A16, A16, A16, L.BF16, -4, 128, 128, None, 0, None) == 2
    assert f(A16 + 8, A16, A16, A16, A16, L.BF16, 4, 128, 128, None, 0, None) == 4
    assert f(A16, A16, A16, A16, A16, 3, 4, 128, 128, None, 0, None) == 5
    assert f(None, None, None, None, None, L.BF16, 0, 128, 128, None, 0, None) == 0
    need = ws(8, 1536, 7168)
    assert need > 0 and ws(4096, 18432, 7168) == 0 and ws(0, 1, 128) == 0 and ws(8, 8, 100) == 0
    assert f(A16, A16, A16, A16, A16, L.BF16, 8, 1536, 7168, None, 0, None) == 6
    assert f(A16, A16, A16, A16, A16, L.BF16, 8, 1536, 7168, A16, need - 1, None) == 6
    assert f(A16, A16, A16, A16, A16, L.BF16, 8, 1536, 7168, A16 + 16, need, None) == 6


def test_fp8_gemm_static_reports_argument_errors_before_the_size_limit(L):
    """The entry point that allocates nothing checks its arguments like dsv3_fp8_gemm and only then the size of its
    scratch array: a malformed call on a large shape reports what is wrong with it, not DSV3_ERR_TOO_LARGE."""
    f = L.lib.dsv3_fp8_gemm_static
    big = (9, 129280, 7168)                                               # 84 MiB of partial sums: beyond the array
    assert L.lib.dsv3_fp8_gemm_workspace_bytes(*big) > L.lib.dsv3_fp8_gemm_static_max_bytes()
    assert f(A16, A16, A16, A16, A16, L.BF16, *big, None) == 8            # well-formed: refused for its size
    assert f(A16, A16, A16, A16, A16, 3, *big, None) == 5                 # bad dtype code
    assert f(None, A16, A16, A16, A16, L.BF16, *big, None) == 1
    assert f(A16 + 8, A16, A16, A16, A16, L.BF16, *big, None) == 4
    assert f(A16, A16, A16, A16, A16, L.BF16, 70000, 129280, 7168 + 64, None) == 2   # K % 128 != 0 with more rows than its fallback takes
    assert f(A16, A16, A16, A16, A16, L.BF16, -9, 129280, 7168, None) == 2
    assert f(None, None, None, None, None, L.BF16, 0, 129280, 7168, None) == 0   # nothing to do


def test_ops_shape_inference_and_no_cpu_fallback():
    import dsv3fp8  # noqa: F401  (registers the ops)
    x = torch.empty(2, 3, 256, device="meta", dtype=torch.bfloat16)
    y, s = torch.ops.dsv3fp8.act_quant(x, 128, 0)
    assert y.shape == (2, 3, 256) and y.dtype == torch.float8_e4m3fn and s.shape == (2, 3, 2) and s.dtype == torch.float32
    w = torch.empty(576, 256, device="meta", dtype=torch.float8_e4m3fn)
    ws = torch.empty(5, 2, device="meta")
    assert torch.ops.dsv3fp8.weight_dequant(w, ws, 128, 0).dtype == torch.bfloat16
    c = torch.ops.dsv3fp8.fp8_gemm(y, s, w, ws, 0)
    assert c.shape == (2, 3, 576) and c.dtype == torch.bfloat16
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.dsv3fp8.act_quant(torch.zeros(1, 128, dtype=torch.bfloat16), 128, 0)   # CPU tensors: no kernel


def test_python_wrappers_keep_the_reference_asserts():
    import dsv3fp8
    x = torch.empty(4, 100, device="meta", dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="divisible by block_size"):
        dsv3fp8.act_quant(x)
    with pytest.raises(AssertionError, match="contiguous"):
        dsv3fp8.act_quant(torch.empty(256, 4, device="meta", dtype=torch.bfloat16).t())
    with pytest.raises(AssertionError, match="2 dimensions"):
        dsv3fp8.weight_dequant(torch.empty(2, 4, 4, device="meta", dtype=torch.float8_e4m3fn), torch.empty(1, 1, device="meta"))


def test_grouped_validation(L):
    f = L.lib.dsv3_fp8_gemm_grouped
    assert L.lib.dsv3_fp8_gemm_grouped_tile_rows() > 0
    ok = dict(a=A16, a_s=A16, a_rows=None, an=64, b=A16, b_s=A16, bst=128 * 128, sst=1, c=A16, cd=L.BF16,
              m=64, n=128, k=128, tg=A16, t0=A16, tr=A16, nt=2, st=None)

    def call(**kw):
        v = {**ok, **kw}
        return f(*[v[key] for key in ("a", "a_s", "a_rows", "an", "b", "b_s", "bst", "sst", "c", "cd", "m", "n", "k",
                                      "tg", "t0", "tr", "nt", "st")])
    assert call(a=None) == 1 and call(tg=None) == 1 and call(c=None) == 1
    assert call(k=100) == 2 and call(k=0) == 2 and call(m=-1) == 2 and call(nt=-1) == 2
    assert call(an=1 << 30, k=128 * 64) == 2                 # byte offsets of a beyond 32 bits
    assert call(a=A16 + 4) == 4 and call(bst=100) == 4
    assert call(cd=7) == 5
    assert call(m=0, a=None, tg=None) == 0 and call(nt=0) == 0


def test_grouped_swiglu_validation(L):
    f, fused = L.lib.dsv3_fp8_gemm_grouped_swiglu, L.lib.dsv3_fp8_gemm_grouped_swiglu_fused
    assert fused(4096, 4096, 2048, 7168) and fused(321, 100, 128, 128)
    assert not fused(320, 4096, 2048, 7168)          # few rows in all: the weight-streaming kernel, two calls
    assert not fused(4096, 4096, 2000, 7168) and not fused(4096, 4096, 2048, 7100) and not fused(0, 0, 128, 128)
    ok = dict(a=A16, a_s=A16, a_rows=None, an=4096, b=A16, b_s=A16, bst=256 * 128, sst=2, y=A16, s=A16,
              m=4096, inter=128, k=128, tg=A16, t0=A16, tr=A16, nt=40, blk=128, fmt=0, st=None)

    def call(**kw):
        v = {**ok, **kw}
        return f(*[v[key] for key in ("a", "a_s", "a_rows", "an", "b", "b_s", "bst", "sst", "y", "s", "m", "inter", "k",
                                      "tg", "t0", "tr", "nt", "blk", "fmt", "st")])
    assert call(a=None) == 1 and call(y=None) == 1 and call(s=None) == 1 and call(tr=None) == 1
    assert call(k=100) == 2 and call(inter=100) == 2 and call(m=-1) == 2
    assert call(m=100) == 2                          # below the tile kernel's range: ask ..._fused first
    assert call(blk=64) == 3 and call(fmt=5) == 5
    assert call(a=A16 + 8) == 4 and call(y=A16 + 2) == 4 and call(bst=100) == 4
    assert call(m=0) == 0 and call(nt=0) == 0


def test_group_tiles_validation(L):
    f = L.lib.dsv3_group_tiles
    assert f(None, 4, 8, A16, A16, A16, None) == 1
    assert f(A16, 4, 8, None, A16, A16, None) == 1
    assert f(A16, -1, 8, A16, A16, A16, None) == 2
    assert f(A16, 4, 0, None, None, None, None) == 0


def test_swiglu_quant_validation(L):
    f = L.lib.dsv3_swiglu_quant
    assert f(None, L.BF16, A16, A16, 4, 128, 128, 0, None) == 1
    assert f(A16, L.F32, A16, A16, 4, 128, 128, 0, None) == 5          # bf16 only
    assert f(A16, L.BF16, A16, A16, 4, 128, 64, 0, None) == 3
    assert f(A16, L.BF16, A16, A16, 4, 100, 128, 0, None) == 2
    assert f(A16, L.BF16, A16, A16, 4, 128, 128, 9, None) == 5
    assert f(A16 + 2, L.BF16, A16, A16, 4, 128, 128, 0, None) == 4
    assert f(None, L.BF16, None, None, 0, 128, 128, 0, None) == 0


def test_moe_combine_validation(L):
    f = L.lib.dsv3_moe_combine
    assert f(None, L.BF16, A16, A16, None, A16, 4, 2, 128, None) == 1
    assert f(A16, L.BF16, A16, A16, None, None, 4, 2, 128, None) == 1
    assert f(A16, L.F16, A16, A16, None, A16, 4, 2, 128, None) == 5
    assert f(A16, L.BF16, A16, A16, None, A16, 4, 2, 100, None) == 2
    assert f(A16 + 2, L.BF16, A16, A16, None, A16, 4, 2, 128, None) == 4
    assert f(None, L.BF16, None, None, None, None, 0, 2, 128, None) == 0


def test_moe_route_validation(L):
    f = L.lib.dsv3_moe_route
    #     idx  w    dtype   tok topk exp shared max_tiles scratch a_rows rows w_sorted tile tables    stream
    ok = [A16, A16, L.BF16, 4,  2,   8,  0,     12,       A16,    A16,   A16, A16,     A16, A16, A16, None]

    def call(i=None, v=None):
        a = list(ok)
        if i is not None:
            a[i] = v
        return f(*a)
    assert call(0, None) == 1 and call(8, None) == 1 and call(12, None) == 1
    assert call(2, L.F32) == 5
    assert call(4, 0) == 2 and call(4, 17) == 2 and call(5, 0) == 2 and call(3, -1) == 2
    assert call(0, A16 + 4) == 4


def test_wkv_b_absorb_validation(L):
    f = L.lib.dsv3_wkv_b_absorb
    #     x    ts        hs   w    ws   y    dtype   side tokens heads nope v   kv_rank block stream
    ok = [A16, 128 * 192, 192, A16, A16, A16, L.BF16, 0,   4,     128,  128, 128, 512,   128,  None]

    def call(i=None, v=None):
        a = list(ok)
        if i is not None:
            a[i] = v
        return f(*a)
    assert call(0, None) == 1 and call(3, None) == 1 and call(4, None) == 1 and call(5, None) == 1
    assert call(6, L.F32) == 5
    assert call(13, 64) == 3
    assert call(7, 2) == 2                         # neither side
    assert call(10, 32) == 2 and call(10, 96) == 2  # side Q implements nope_dim 64 and 128
    assert call(12, 500) == 2 and call(11, 100) == 2
    assert call(2, 100) == 2 and call(1, 12) == 2   # head stride shorter than the row / strides not multiples of 8
    assert call(0, A16 + 8) == 4 and call(5, A16 + 2) == 4
    assert call(8, -1) == 2 and call(9, 70000) == 2
    assert call(8, 0) == 0                           # nothing to do: no launch, no dereference
    v = list(ok); v[7] = 1; v[12] = 384
    assert f(*v) == 2                               # side V implements kv_rank 128, 256, 512


def test_gate_route_validation(L):
    f = L.lib.dsv3_gate_route
    #     logits dtype   bias  w    idx  tokens experts topk groups topk_groups func scale stream
    ok = [A16,   L.BF16, None, A16, A16, 4,     256,    8,   8,     4,          1,   2.5,  None]

    def call(i=None, v=None):
        a = list(ok)
        if i is not None:
            a[i] = v
        return f(*a)
    assert call(0, None) == 1 and call(3, None) == 1 and call(4, None) == 1
    assert call(1, L.F32) == 5 and call(10, 2) == 5
    assert call(6, 513) == 2 and call(7, 0) == 2 and call(7, 65) == 2 and call(5, -1) == 2
    assert call(8, 7) == 2                          # experts not divisible by the number of groups
    assert call(9, 9) == 2 and call(9, 0) == 2
    a = list(ok); a[8], a[9], a[7] = 64, 1, 8       # one group of 4 experts cannot supply 8
    assert f(*a) == 2
    assert call(0, A16 + 1) == 4 and call(4, A16 + 4) == 4
    assert call(5, 0) == 0


def test_linear_fp8_validation(L):
    f, fused = L.lib.dsv3_linear_fp8, L.lib.dsv3_linear_fp8_fused
    assert fused(1, 1536, 7168) and fused(2, 7168, 16384) and not fused(16, 7168, 16384) and not fused(17, 1536, 7168)
    # 3+ rows: two calls wherever fp8_gemm takes the activation-streaming kernel (K of 512 and more); one and two rows
    # are always one call
    assert fused(8, 4096, 256) and not fused(8, 24576, 1536) and not fused(8, 7168, 16384)
    assert fused(1, 24576, 1536) and fused(2, 576, 7168) and fused(1, 32768, 512)
    assert not fused(4096, 1536, 7168)
    assert not fused(4, 1536, 7000) and not fused(0, 8, 128)
    #     x    dtype   b    b_s  c    cdtype  m  n     k     block fmt ws    ws_bytes stream
    ok = [A16, L.BF16, A16, A16, A16, L.BF16, 2, 1536, 7168, 128,  0,  A16 * 16, 1 << 30, None]

    def call(i=None, v=None):
        a = list(ok)
        if i is not None:
            a[i] = v
        return f(*a)
    assert call(0, None) == 1 and call(2, None) == 1 and call(3, None) == 1 and call(4, None) == 1
    assert call(1, L.F32) == 5 and call(5, 7) == 5 and call(10, 3) == 5
    assert call(9, 64) == 3
    assert call(8, 7000) == 2 and call(6, 64) == 2          # K not a multiple of 128; too many rows for the fused kernel
    assert call(0, A16 + 2) == 4
    assert call(11, None) == 6 and call(12, 16) == 6         # the split-K workspace is required and checked
    assert call(6, 0) == 0
