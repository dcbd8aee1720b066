#!/usr/bin/env python3
"""Benchmark of the block-scaled FP8 path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A step is one pass of the hot path -- the FP8 branch of ``linear()``
(reference: inference/model.py:159-160): ``act_quant`` then ``fp8_gemm`` -- over
one batch of M = 4096 synthetic tokens through the dense-MLP w1 projection
(7168 -> 18432), inputs resident in HBM.  ``value`` is 2*M*N*K / step time.
Before the W warm-up steps the same step runs untimed for ``settle_ms`` so that
the measurement starts from the clocks the GPU holds under sustained load.

The JSON line also carries
  roofline      the dominant kernel (fp8_gemm) timed alone with HIP events on the
                launch stream: achieved TFLOP/s vs the dense fp8 MFMA peak;
  cpu_baseline  the torch-CPU oracle timed on this host on a bounded row sample;
  extras        the other configurations: act_quant / weight_dequant bandwidth,
                the w2 prefill shape and the decode sweep (GB/s over algorithmic bytes,
                weights rotated through > 512 MB so the Infinity Cache cannot hold them).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "deepseek-v3_amd"))
sys.path.insert(0, str(ROOT))

import torch  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
FP8_MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 (no sparsity)
SETTLE_S = 0.15                # untimed run of the step before the warm-up steps (see settle())
METRIC = "fp8_gemm TFLOP/s & %fp8 MFMA peak @M=4096; decode-GEMM HBM GB/s @M=1-64"


class Probes:
    """libdsv3probe.so: kernels of known traffic / arithmetic (read stream, copy, fp8 MFMA loop, empty launch) that
    give the ceilings this GPU sustains.  Measurement infrastructure only."""

    def __init__(self):
        import ctypes as C
        path = ROOT / "bench" / "probes" / "libdsv3probe.so"
        if not path.exists():                                  # built by __graft_entry__.build(); only if nothing is there
            import importlib.util
            spec = importlib.util.spec_from_file_location("dsv3_probe_build", path.parent / "build.py")
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            mod.build_probes(verbose=False)
        L = self.lib = C.CDLL(str(path))
        L.dsv3_probe_read_stream.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_void_p]
        L.dsv3_probe_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.dsv3_probe_mfma.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.dsv3_probe_mix.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.dsv3_probe_mfma_flops.restype = C.c_double
        L.dsv3_probe_mfma_flops.argtypes = [C.c_int]
        L.dsv3_probe_null.argtypes = [C.c_void_p]
        self.sink = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")
        self.pool = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device="cuda")      # 1 GiB of random bytes

    @staticmethod
    def _st():
        return torch.cuda.current_stream().cuda_stream

    def read(self, offset: int, nbytes: int):
        rc = self.lib.dsv3_probe_read_stream(self.pool.data_ptr() + offset, nbytes, self.sink.data_ptr(), 0, self._st())
        assert rc == 0

    def read_stream_us(self, nbytes: int) -> float:
        """Microseconds per launch of a plain read stream over `nbytes` contiguous bytes, rotating through the pool
        like the decode sweep rotates its weights (HIP graph, back-to-back launches)."""
        nbytes = nbytes // 4096 * 4096
        copies = max(2, min(160, (1 << 30) // nbytes, -(-640_000_000 // nbytes)))
        launches = [(lambda i=i: self.read(i * nbytes, nbytes)) for i in range(copies)]
        if len(launches) < 40:
            launches = launches * (-(-40 // len(launches)))
        return time_graph(launches)

    def mix_gbps(self, dst, rd: int, wr: int) -> float:
        """GB/s (bytes read + written) of a stream that reads rd and writes wr bytes per unit, over ~1 GiB."""
        import ctypes as C
        n_read = self.pool.numel() if rd >= wr else self.pool.numel() // 2
        done = C.c_size_t(0)
        call = lambda: self.lib.dsv3_probe_mix(self.pool.data_ptr(), dst.data_ptr(), n_read, rd, wr, C.byref(done), self._st())
        assert call() == 0
        us = time_graph([call] * 4)
        return (done.value + done.value * wr // rd) / us / 1e3

    def mix_same_size_us(self, rd: int, wr: int, bytes_read: int, copies: int) -> float:
        """Microseconds per launch of the rd : wr stream over `bytes_read` input bytes, sources and destinations
        rotating like the measured kernel's (so neither side is served by the Infinity Cache)."""
        copies = max(1, min(copies, self.pool.numel() // bytes_read))
        bytes_written = bytes_read * wr // rd
        dst = torch.empty(copies * bytes_written, dtype=torch.uint8, device="cuda")
        calls = [(lambda i=i: self.lib.dsv3_probe_mix(self.pool.data_ptr() + i * bytes_read, dst.data_ptr() + i * bytes_written,
                                                      bytes_read, rd, wr, None, self._st())) for i in range(copies)]
        assert calls[0]() == 0
        us = time_graph(calls * 2)
        del dst
        return us

    def mfma_tflops(self, mode: int, iters: int = 4000) -> float:
        us = time_graph([lambda: self.lib.dsv3_probe_mfma(iters, mode, self.pool.data_ptr(), self.sink.data_ptr(), self._st())] * 10)
        return self.lib.dsv3_probe_mfma_flops(iters) / us / 1e6

    def ceilings(self) -> dict:
        n = self.pool.numel()
        dst = torch.empty_like(self.pool)
        rd = time_graph([lambda: self.read(0, n)] * 4)
        cp = time_graph([lambda: self.lib.dsv3_probe_copy(self.pool.data_ptr(), dst.data_ptr(), n, 0, self._st())] * 4)
        r2w1 = self.mix_gbps(dst, 2, 1)
        r1w2 = self.mix_gbps(dst, 1, 2)
        del dst
        nl = time_graph([lambda: self.lib.dsv3_probe_null(self._st())] * 100)
        return {"hbm_read_stream_GBps": round(n / rd / 1e3, 1), "hbm_copy_GBps": round(2 * n / cp / 1e3, 1),
                "hbm_read2_write1_GBps": round(r2w1, 1), "hbm_read1_write2_GBps": round(r1w2, 1),
                "fp8_mfma_loop_TFLOPs": round(self.mfma_tflops(0), 1),
                "fp8_mfma_loop_changing_operands_TFLOPs": round(self.mfma_tflops(1), 1),
                "fp8_mfma_loop_with_fold_TFLOPs": round(self.mfma_tflops(2), 1),
                "fp8_mfma_loop_with_fold_no_shared_operand_TFLOPs": round(self.mfma_tflops(8), 1),
                "fp8_mfma_loop_with_fold_and_operand_traffic_TFLOPs": round(self.mfma_tflops(3), 1),
                "fp8_mfma_loop_with_operand_traffic_no_fold_TFLOPs": round(self.mfma_tflops(4), 1),
                "fp8_mfma_32x32x64_loop_changing_operands_TFLOPs": round(self.mfma_tflops(5), 1),
                "fp8_mfma_32x32x64_loop_with_fold_TFLOPs": round(self.mfma_tflops(6), 1),
                "fp8_mfma_32x32x64_loop_with_fold_and_operand_traffic_TFLOPs": round(self.mfma_tflops(7), 1),
                "empty_launch_us": round(nl, 2),
                "note": "measured on this GPU in this run: 1 GiB read stream; 1 GiB copy (bytes read + written); streams "
                        "that read two bytes per byte written (the mix of act_quant and weight_quant) and one per two "
                        "written (weight_dequant); registers-only v_mfma_f32_16x16x128_f8f6f4 loops, 8 wavefronts per "
                        "CU: one operand pair for all instructions, 4 x 4 fragments of random bytes accumulated in the "
                        "matrix core (what power-of-two scales allow), and the same with every product folded into "
                        "its accumulator by four FMAs (what binary32 block scales need) -- the chip is power limited, "
                        "so the rate falls as operands toggle and as vector work is added (no_shared_operand: an issue "
                        "order in which consecutive instructions share neither operand, where the others share one); "
                        "the fold loop inside the data movement "
                        "of a 256 x 256 x 128 GEMM step and nothing else (per 16 products a wavefront copies 4 KiB from "
                        "L2 into LDS and reads six 2 KiB fragments from LDS into the operand registers; no barrier, the "
                        "copied bytes are not consumed): what the chip sustains for the GEMM's instruction mix and "
                        "traffic when every overlap is perfect, and the same without the fold (the ceiling of "
                        "power-of-two scales); the three loops again on v_mfma_f32_32x32x64_f8f6f4, two chained "
                        "instructions per 128-wide scale block (half the operand-register reads per flop, 16 fold FMAs "
                        "per 32 x 32 x 128 product); empty kernel in a graph"}


class NoProbes:
    """Stand-in when libdsv3probe.so cannot be built or loaded: no ceilings, no streams beside the kernels; everything
    the library itself does is still measured."""

    def __init__(self, why: str):
        self.why = why

    def ceilings(self):
        return None

    def read_stream_us(self, nbytes: int):
        return None

    def mix_same_size_us(self, rd: int, wr: int, bytes_read: int, copies: int):
        return None


def _ratio(a, b, digits: int = 3):
    return None if a is None or b is None else round(a / b, digits)


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_loop(fn, steps: int, warmup: int) -> float:
    """Average milliseconds per call over exactly `steps` calls (events on the launch stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = _events(2)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def settle(fn, seconds: float) -> None:
    """Runs fn back to back for `seconds` of wall time, untimed.  A GPU that comes out of idle takes some tens of
    milliseconds of sustained load to reach the clocks it then holds (the same launch measures 600 us a few
    milliseconds into a run and 475 us from 30 ms on); the warm-up steps that follow start from that state."""
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


GRAPH_SETTLE_S = 0.03


def time_graph(launches, replays: int = 5) -> float:
    """Microseconds per launch (median over the replays) with the launches captured in one HIP graph, so that
    back-to-back kernels are not separated by host launch latency.  `launches` is a list of
    zero-argument callables (typically the same op over rotating buffers).  Before the timed replays the graph is
    replayed untimed for GRAPH_SETTLE_S of wall time: like the headline step (settle()), a short kernel measured
    right after the set-up work of its cell runs 5 % slower than a few tens of milliseconds later (16384 -> 7168
    at one row: 23.2 us as the first measurement of a process, 21.5-21.9 us from the second on)."""
    for fn in launches[: min(3, len(launches))]:
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for fn in launches:
            fn()
    g.replay()
    torch.cuda.synchronize()
    t_end = time.perf_counter() + GRAPH_SETTLE_S
    while time.perf_counter() < t_end:
        g.replay()
        torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        e0, e1 = _events(2)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    return sorted(times)[len(times) // 2] * 1e3 / len(launches)          # median replay


def measured_traffic():
    """HBM bytes per launch of the dominant kernel on this workload, from the committed rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE summary (profiles/fp8_gemm_prefill_traffic.json); None when it has not been taken."""
    f = ROOT / "profiles" / "fp8_gemm_prefill_traffic.json"
    if not f.exists():
        return None
    try:
        return json.loads(f.read_text())["hbm_bytes_per_launch"]
    except (ValueError, KeyError):
        return None


def decode_bytes(m, n, k):
    return n * k + 4 * (-(-n // 128)) * (k // 128) + m * k + 4 * m * (k // 128) + 2 * m * n


def _bw(nbytes: float, us: float, copy_gbps: float, mix_us: float) -> dict:
    """mix_us: a plain stream of the same size and read : write ratio as this kernel, measured the same way."""
    gbs = nbytes / us / 1e3
    return {"us": round(us, 2), "GBps": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 3),
            "frac_of_measured_copy": _ratio(gbs, copy_gbps),
            "plain_stream_same_size_and_mix_us": None if mix_us is None else round(mix_us, 2),
            "frac_of_that_stream": _ratio(mix_us, us)}


def run_extras(K, W, probes, ceil):
    out = {}
    copy_c, read_c = (ceil["hbm_copy_GBps"], ceil["hbm_read_stream_GBps"]) if ceil else (None, None)
    x = W.activations(4096, 7168, 0, "cuda", outliers=True)
    xs = [x.clone() for _ in range(12)]                       # 12 x 58.7 MB > Infinity Cache
    us = time_graph([(lambda t=t: K.act_quant(t)) for t in xs] * 2)
    out["act_quant_4096x7168"] = _bw(88.998e6, us, copy_c, probes.mix_same_size_us(2, 1, 4096 * 7168 * 2, 12))
    del xs
    w8, s = W.random_fp8_weight(18432, 7168, 2, "cuda")
    ws_ = [w8.clone() for _ in range(5)]
    us = time_graph([(lambda t=t: K.weight_dequant(t, s)) for t in ws_] * 2)
    out["weight_dequant_18432x7168"] = _bw(396.394e6, us, copy_c, probes.mix_same_size_us(1, 2, 18432 * 7168, 6))
    del ws_, w8
    wb = [(torch.randn(18432, 7168, device="cuda") * 0.02).bfloat16() for _ in range(4)]   # 4 x 264 MB
    us = time_graph([(lambda t=t: K.weight_quant(t)) for t in wb] * 2)
    out["weight_quant_18432x7168"] = _bw(396.394e6, us, copy_c, probes.mix_same_size_us(2, 1, 18432 * 7168 * 2, 4))
    del wb
    k, n = W.PREFILL_SHAPES["w2"]
    a, a_s = K.act_quant(W.activations(4096, k, 0, "cuda"))
    wq, wsc = W.weight(n, k, 1, "cuda")
    settle(lambda: K.fp8_gemm(a, a_s, wq, wsc), 0.05)
    ms = time_loop(lambda: K.fp8_gemm(a, a_s, wq, wsc), 20, 3)
    tf = 2 * 4096 * n * k / ms / 1e9
    out["fp8_gemm_M4096_w2_18432to7168"] = {"us": round(ms * 1e3, 1), "TFLOPs": round(tf, 1),
                                           "mfma_frac": round(tf / FP8_MFMA_PEAK_TFLOPS, 3)}
    # the same shape with power-of-two scales (scale_fmt "ue8m0" activations, block scales rounded up to 2^e):
    # the scales ride in the matrix instruction's scale operands
    a2, a2_s = K.act_quant(W.activations(4096, k, 0, "cuda"), 128, "ue8m0")
    wsc2 = torch.pow(2.0, torch.ceil(torch.log2(wsc)))
    settle(lambda: K.fp8_gemm_pow2(a2, a2_s, wq, wsc2), 0.05)
    ms = time_loop(lambda: K.fp8_gemm_pow2(a2, a2_s, wq, wsc2), 20, 3)
    tf = 2 * 4096 * n * k / ms / 1e9
    out["fp8_gemm_pow2_M4096_w2_18432to7168"] = {"us": round(ms * 1e3, 1), "TFLOPs": round(tf, 1),
                                                "mfma_frac": round(tf / FP8_MFMA_PEAK_TFLOPS, 3)}
    del a, a_s, wq, wsc, a2, a2_s, wsc2
    dec = {}
    for name, (k, n) in W.DECODE_SWEEP.items():
        wq, wsc = W.weight(n, k, 1, "cuda")
        copies = max(2, min(160, -(-640_000_000 // (n * k))))
        wqs = [wq.clone() for _ in range(copies)]
        floor_us = probes.read_stream_us(n * k)               # a plain read stream over as many bytes as the weight
        for m in W.DECODE_M:
            a, a_s = K.act_quant(W.activations(m, k, m, "cuda"))
            launches = [(lambda t=t: K.fp8_gemm(a, a_s, t, wsc)) for t in wqs]
            if len(launches) < 40:
                launches = launches * (-(-40 // len(launches)))
            us = time_graph(launches)
            gbs = decode_bytes(m, n, k) / us / 1e3
            dec[f"{name}_{k}to{n}_M{m}"] = {"us": round(us, 2), "GBps": round(gbs, 1),
                                            "hbm_frac": round(gbs / HBM_PEAK_GBS, 3),
                                            "frac_of_measured_read": _ratio(gbs, read_c),
                                            "read_stream_same_bytes_us": None if floor_us is None else round(floor_us, 2),
                                            "read_stream_same_bytes_over_gemm_time": _ratio(floor_us, us)}
        del wqs
    out["decode"] = dec
    # linear() at decode sizes: act_quant + fp8_gemm as two launches against the fused single launch
    lin = {}
    for name, (k, n) in W.DECODE_SHAPES.items():
        wq, wsc = W.weight(n, k, 1, "cuda")
        copies = max(2, min(160, -(-640_000_000 // (n * k))))
        wqs = [wq.clone() for _ in range(copies)]
        xa = W.activations(1, k, 1, "cuda")

        def two(t):
            q, qs = K.act_quant(xa)
            return K.fp8_gemm(q, qs, t, wsc)
        l2 = [(lambda t=t: two(t)) for t in wqs]
        l1 = [(lambda t=t: torch.ops.dsv3fp8.linear_fp8(xa, t, wsc, 0, 0)) for t in wqs]
        if len(l1) < 40:
            l1, l2 = l1 * (-(-40 // len(l1))), l2 * (-(-40 // len(l2)))
        lin[f"{name}_M1"] = {"two_launch_us": round(time_graph(l2), 2), "fused_us": round(time_graph(l1), 2)}
        del wqs
    out["linear_decode"] = lin
    out["moe_layer_T4096"] = run_moe(K, W)
    out["moe_layer_T4096_balanced"] = run_moe(K, W, bias_std=0.0, expert_loop=False)
    out["wkv_b_absorb"] = run_absorb(K, W)
    return out


def decode_trace(K, W, launches_per_cell: int = 60):
    """For `rocprofv3 --kernel-trace`: every cell of the decode sweep as plain launches (no graph) over rotating
    weight copies, cell after cell in a fixed order, with a device synchronisation between cells.  Prints one JSON
    line naming the cells in launch order and the launches per cell, so that the kernel rows of the trace (sorted by
    start time) can be cut into cells: a launch is one GEMM kernel, followed by the kernel that adds its K slices
    when the plan has any."""
    order = []
    for name, (k, n) in W.DECODE_SWEEP.items():
        wq, wsc = W.weight(n, k, 1, "cuda")
        copies = max(2, min(160, -(-640_000_000 // (n * k))))
        wqs = [wq.clone() for _ in range(copies)]
        for m in W.DECODE_M:
            a, a_s = K.act_quant(W.activations(m, k, m, "cuda"))
            torch.cuda.synchronize()
            for i in range(launches_per_cell):
                K.fp8_gemm(a, a_s, wqs[i % copies], wsc)
            torch.cuda.synchronize()
            order.append({"cell": f"{name}_{k}to{n}_M{m}", "bytes": decode_bytes(m, n, k)})
        del wqs
    print(json.dumps({"decode_trace": {"launches_per_cell": launches_per_cell, "cells": order}}), flush=True)


def grouped_rows_sweep(K, W, rows_per_group=(16, 64, 96, 128, 160, 192, 256), launches: int = 6):
    """For `rocprofv3 --kernel-trace` / `--pmc GRBM_GUI_ACTIVE`: the grouped GEMM at the MoE layer's w1|w3 shape
    (256 groups, 7168 -> 4096, one weight of 29 MB per group, all streamed from HBM) with the SAME number of rows
    in every group, one row count after the other, as plain launches.  Every group is one tile slot, so a compute
    unit runs 16 tiles of 56 K blocks per launch and the time per K block is launch time / (16 * 56).  Prints one
    JSON line with the launch order and HIP-event times so that the trace's rows can be cut into row counts."""
    groups, n, k = 256, 4096, 7168
    w8, sc = W.weight(n, k, 40, "cuda")
    w = w8.unsqueeze(0).repeat(groups, 1, 1)                   # distinct storage per group: 7.5 GB
    s = sc.unsqueeze(0).repeat(groups, 1, 1).contiguous()
    from dsv3fp8 import ops as _ops
    g = torch.ops.dsv3fp8.fp8_gemm_grouped
    code = _ops.dtype_code(torch.bfloat16)
    out = []
    for r in rows_per_group:
        m = groups * r
        a, a_s = K.act_quant(W.activations(m, k, r, "cuda"))
        counts = torch.full((groups,), r, dtype=torch.int32, device="cuda")
        tg, t0, tr = torch.ops.dsv3fp8.group_tiles(counts, groups + 8)
        fn = lambda: g(a, a_s, None, w, s, m, tg, t0, tr, code)
        ms = time_loop(fn, launches - 2, 2)
        out.append({"rows_per_group": r, "launches": launches, "us": round(ms * 1e3, 1),
                    "us_per_k_block": round(ms * 1e3 / (16 * (k // 128)), 3),
                    "weight_GBps": round(groups * n * k / ms / 1e6, 1)})
        del a, a_s
    print(json.dumps({"grouped_rows_sweep": {"shape": "256 groups x (rows, 7168) -> 4096", "cells": out}}), flush=True)


def decode_roofline(dec: dict, ceil: dict) -> dict:
    """The metric's second half in one block: the decode sweep (M = 1, 8, 32, 64 over the MLA projections) as HBM
    fractions of its algorithmic bytes, against the 8 TB/s peak and against this GPU's measured read stream."""
    import math
    geomean = lambda xs: math.exp(sum(math.log(x) for x in xs) / len(xs))
    fr = [v["hbm_frac"] for v in dec.values()]
    worst = min(dec, key=lambda k_: dec[k_]["hbm_frac"])
    best = max(dec, key=lambda k_: dec[k_]["hbm_frac"])
    geo = geomean(fr)
    five = [v["hbm_frac"] for k_, v in dec.items() if "stacked" not in k_]      # the five projections of the layer alone
    res = {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s", "cells": len(fr),
           "kernels": ["fp8_gemm_skinny_kernel (one and two rows on weights of 64 and more 16-row strips; up to 16 rows "
                       "where the next kernel has no plan)",
                       "fp8_gemm_stream_kernel (1 .. 64 rows wherever its planner has a plan; up to 32 rows on weights "
                       ">= 96 MiB of 8192 and more rows)",
                       "large-M kernel, K sliced (33 .. 64 rows on weights >= 96 MiB of 8192 and more rows)",
                       "splitk_reduce_kernel (second launch of a K-sliced plan)"],
           "bytes": "N*K + 4*ceil(N/128)*(K/128) + M*K + 4*M*K/128 + 2*M*N per launch",
           "frac_min": min(fr), "frac_min_cell": worst, "frac_max": max(fr), "frac_max_cell": best,
           "frac_geomean": round(geo, 3),
           "frac_geomean_five_projections": round(geomean(five), 3)}
    if ceil:
        res["frac_geomean_of_measured_read"] = round(geo * HBM_PEAK_GBS / ceil["hbm_read_stream_GBps"], 3)
        res["measured_read_stream_GBps"] = ceil["hbm_read_stream_GBps"]
        # launch time of a plain read stream over exactly the weight's bytes, divided by the GEMM's launch time
        # (both in the same kind of graph over rotating buffers): what is left once the floor of a launch this
        # short is taken out
        ratios = {k_: v["read_stream_same_bytes_over_gemm_time"] for k_, v in dec.items()}
        res["read_stream_same_bytes_over_gemm_time_geomean"] = round(geomean(list(ratios.values())), 3)
        res["read_stream_same_bytes_over_gemm_time_M1"] = {k_: r for k_, r in ratios.items() if k_.endswith("_M1")}
    return res


def run_absorb(K, W, token_counts=(1, 16, 64, 128, 4096)):
    """The two wkv_b products of the absorbed attention on the fp8 weight (128 heads, 128 + 128 rows each, rank
    512), per token count: microseconds of the fused kernels (rotating weight copies, HIP graph) beside the
    reference's sequence on the same device -- weight_dequant of the whole weight, then two bf16 einsums."""
    heads, nope, v, c = 128, 128, 128, 512
    copies = 24                                                # 24 x 16.8 MB > Infinity Cache
    w8, sc = W.random_fp8_weight(heads * (nope + v), c, 7, "cuda")
    w8s = [w8.clone() for _ in range(copies)]
    wd = K.weight_dequant(w8, sc).view(heads, nope + v, c)
    op = torch.ops.dsv3fp8.wkv_b_absorb
    res = {}
    for tokens in token_counts:
        g = torch.Generator(device="cuda").manual_seed(tokens)
        q = torch.randn(tokens, heads, nope + 64, generator=g, device="cuda").bfloat16()[..., :nope]
        o = torch.randn(tokens, heads, c, generator=g, device="cuda").bfloat16()
        n = copies if tokens < 1024 else 6
        us_q = time_graph([(lambda t=t: op(q, t, sc, 0, nope, v)) for t in w8s[:n]])
        us_v = time_graph([(lambda t=t: op(o, t, sc, 1, nope, v)) for t in w8s[:n]])
        us_d = time_graph([(lambda t=t: K.weight_dequant(t, sc)) for t in w8s[:n]])
        us_e = time_graph([lambda: torch.einsum("mhd,hdc->mhc", q, wd[:, :nope]),
                           lambda: torch.einsum("mhc,hdc->mhd", o, wd[:, nope:])] * 3) * 2
        wbytes = heads * 128 * c
        res[f"T{tokens}"] = {"q_us": round(us_q, 2), "v_us": round(us_v, 2),
                             "q_GBps": round((wbytes + tokens * heads * (nope + c) * 2) / us_q / 1e3, 1),
                             "v_GBps": round((wbytes + tokens * heads * (c + v) * 2) / us_v / 1e3, 1),
                             "dequant_then_einsums_us": round(us_d + us_e, 2)}
    return res


def run_moe(K, W, tokens: int = 4096, bias_std: float = 0.1, expert_loop: bool = True):
    """The MoE-layer configuration: one MoE layer (256 routed + 1 shared SwiGLU experts, 7168 -> 2048 -> 7168, fp8
    block-scaled weights generated on the device), T tokens, sigmoid gate with bias over random logits'
    weights, 8 groups / top-4 groups / top-8 experts, route_scale 2.5.  Timed twice: the grouped path
    (device-side token lists, two grouped GEMMs, fused SwiGLU + re-quantisation, ordered combine) and the
    reference's host-driven pass over the experts' token lists (model.py:679-693) on the same kernels.

    The logits have a standard deviation of 1.7, so the best sigmoid scores of a token lie within 0.04 of 1 and a
    bias drawn with bias_std = 0.1 decides most of the selection: the load is skewed (a third of the experts get no
    token, the busiest about 1100 of the 32768 rows).  bias_std = 0 gives the balanced load a trained router aims
    for (97 .. 161 rows per expert), in which every expert's weights are streamed.  The result names the load."""
    from dsv3fp8 import model as Mdl
    old = Mdl.gemm_impl, Mdl.Linear.dtype, Mdl.MoE.grouped
    Mdl.gemm_impl, Mdl.Linear.dtype = "fp8", torch.float8_e4m3fn
    try:
        args = Mdl.ModelArgs()
        with torch.device("cuda"):
            moe = Mdl.MoE(args)
        g = torch.Generator(device="cuda").manual_seed(5)
        with torch.no_grad():
            moe.gate.weight.copy_(torch.randn(args.n_routed_experts, args.dim, generator=g, device="cuda") * 0.02)
            moe.gate.bias.copy_(torch.randn(args.n_routed_experts, generator=g, device="cuda") * bias_std)
            protos = [W.weight(args.moe_inter_dim, args.dim, 40, "cuda"), W.weight(args.dim, args.moe_inter_dim, 41, "cuda")]
            for ex in list(moe.experts) + [moe.shared_experts]:
                for lin, (w8, sc) in ((ex.w1, protos[0]), (ex.w3, protos[0]), (ex.w2, protos[1])):
                    lin.weight.copy_(w8)          # distinct storage per expert: 11.3 GB of weights are streamed
                    lin.scale.copy_(sc)
        moe.stack_experts()
        x = W.activations(tokens, args.dim, 6, "cuda")
        flops = 2.0 * 3 * args.dim * args.moe_inter_dim * (tokens * args.n_activated_experts + tokens)
        res = {}
        with torch.inference_mode():
            counts = torch.bincount(moe.gate(x)[1].reshape(-1), minlength=args.n_routed_experts)
            hit = int((counts > 0).sum())
            res["load"] = {"bias_std": bias_std, "experts_with_tokens": hit,
                           "rows_per_expert_min_mean_max": [int(counts.min()), float(counts.float().mean()), int(counts.max())]}
            wbytes = (hit + 1) * 3 * args.dim * args.moe_inter_dim      # weights of the experts that get a token
            for key, grouped, steps in (("grouped", True, 10), ("expert_loop", False, 2))[:2 if expert_loop else 1]:
                Mdl.MoE.grouped = grouped
                ms = time_loop(lambda: moe(x), steps, 2 if grouped else 1)
                res[key] = {"ms": round(ms, 3), "TFLOPs": round(flops / ms / 1e9, 1),
                            "weight_stream_GBps": round(wbytes / ms / 1e6, 1),
                            "mfma_frac": round(flops / ms / 1e9 / FP8_MFMA_PEAK_TFLOPS, 4),
                            "hbm_frac": round(wbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
            Mdl.MoE.grouped = True
            res["grouped_stages_us"] = moe_stages(moe, x, Mdl)
            if expert_loop:                  # decode sizes on the same layer, one captured forward each
                Mdl.MoE.grouped = True
                dec = {}
                for t in (1, 8, 32):
                    xd = W.activations(t, args.dim, 60 + t, "cuda")
                    hit_d = int(moe.gate(xd)[1].unique().numel())
                    us = time_graph([lambda: moe(xd)], replays=20)
                    wb = (hit_d + 1) * 3 * args.dim * args.moe_inter_dim
                    dec[f"T{t}"] = {"us": round(us, 1), "experts_with_tokens": hit_d,
                                    "weight_stream_GBps": round(wb / us / 1e3, 1)}
                res["decode_graph"] = dec
        res["note"] = ("grouped: MoE.forward as shipped (no host sync); expert_loop: the reference's per-expert "
                       "loop, 3 act_quant + 3 fp8_gemm per expert")
        return res
    finally:
        Mdl.gemm_impl, Mdl.Linear.dtype, Mdl.MoE.grouped = old


def moe_stages(moe, x, Mdl):
    """Microseconds of each launch group of MoE._forward_grouped on fixed inputs, timed one stage at a time (same
    ops, same arguments, same order as the layer issues them)."""
    ops, bs = Mdl.ops, Mdl.block_size
    w13, s13, w2, s2 = (t[:moe.n_routed_experts] for t in moe._stacked)
    code = ops.dtype_code(torch.get_default_dtype())
    st = {}

    def t(name, fn, steps=10):
        st[name] = round(time_loop(fn, steps, 2) * 1e3, 1)
        return fn()
    weights, indices = t("gate", lambda: moe.gate(x))
    route = t("moe_route", lambda: torch.ops.dsv3fp8.moe_route(indices.contiguous(), weights.contiguous(),
                                                                 moe.n_routed_experts, False))
    _, a_rows, rows, w_sorted, tile_group, tile_row0, tile_rows = route
    pairs = rows.numel()
    xq, xs = t("act_quant", lambda: Mdl.act_quant(x, bs, None))
    g = torch.ops.dsv3fp8.fp8_gemm_grouped
    h = t("grouped_w1w3", lambda: g(xq, xs, a_rows, w13, s13, pairs, tile_group, tile_row0, tile_rows, code))
    gq, gs = t("swiglu_quant", lambda: torch.ops.dsv3fp8.swiglu_quant(h, bs, 0))
    out = t("grouped_w2", lambda: g(gq, gs, None, w2, s2, pairs, tile_group, tile_row0, tile_rows, code))
    z = t("shared_expert", lambda: moe.shared_experts(x, (xq, xs)).contiguous())
    t("moe_combine", lambda: torch.ops.dsv3fp8.moe_combine(out, rows, w_sorted, z))
    # the first GEMM with the activation and the re-quantisation in its epilogue, which is what MoE.forward runs
    # (MoE.fuse_swiglu_epilogue) in place of grouped_w1w3 + swiglu_quant
    st["w1w3_with_swiglu_epilogue"] = round(time_loop(lambda: torch.ops.dsv3fp8.fp8_gemm_grouped_swiglu(
        xq, xs, a_rows, w13, s13, pairs, tile_group, tile_row0, tile_rows, 0), 10, 2) * 1e3, 1)
    # the launches of one forward: the fused first GEMM counts, the two-call form beside it does not
    st["sum"] = round(sum(v for k, v in st.items() if k not in ("grouped_w1w3", "swiglu_quant")), 1)
    return st


CPU_THREADS_CAP = 16      # a one-GPU box gives a job 16 host cores, whatever os.cpu_count() shows there


def _host() -> dict:
    model = "unknown"
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                model = ln.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"os_cpu_count": os.cpu_count(), "torch_num_threads": torch.get_num_threads(), "cpu_model": model,
            "threads_cap": CPU_THREADS_CAP}


def _cpu_time(fn, budget_s: float, max_passes: int = 8):
    """Seconds per pass of fn on the host: one untimed pass, then whole passes until budget_s has gone by."""
    fn()
    passes, t0 = 0, time.perf_counter()
    while True:
        fn()
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or passes >= max_passes:
            return dt / passes, passes


def cpu_baseline(W, rows: int = 1024):
    """The torch-CPU oracle (a port of the reference arithmetic) on the first `rows` tokens of
    the same workload, on the host's threads (at most CPU_THREADS_CAP)."""
    from oracle import oracle
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, CPU_THREADS_CAP)))
    x = W.activations(rows, 7168, 0, "cpu")
    w8, ws = W.weight(18432, 7168, 1, "cpu")
    oracle.linear(x[:64], w8, scale=ws)                      # warm-up
    passes, t0 = 0, time.perf_counter()
    while True:                                              # whole passes over the sample until >= 10 s of CPU work
        oracle.linear(x, w8, scale=ws)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= 10.0 or passes >= 8:
            break
    return {"value": round(2 * rows * passes * 18432 * 7168 / dt / 1e12, 4), "unit": "TFLOP/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.linear() (act_quant + fp8_gemm, fp32 torch-CPU), {passes} passes over {rows} of 4096 rows, "
                      f"K=7168 -> N=18432, {dt:.2f} s", "host": _host()}


def cpu_baselines_other_configs(W) -> dict:
    """The oracle timed on the host for the configurations beside the headline one (the headline's figure is
    `cpu_baseline`): config 1 whole, config 2 whole (act_quant, weight_dequant), config 3 all cells (fp8_gemm at 1, 8,
    32, 64 rows over the five projections), config 5 on 16 routed experts and 256 tokens (every token still selects 8
    experts in 4 of 8 groups; flops 1/16 of the full layer's, stated beside the figure).  About 40 s in all."""
    from oracle import oracle
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, CPU_THREADS_CAP)))
    out = {"host": _host()}
    x, w8, ws = W.cfg1_cpu_plumbing()
    sec, n = _cpu_time(lambda: oracle.linear(x, w8, scale=ws), 1.0)
    out["cfg1_linear_16x7168_to_1536"] = {"ms": round(sec * 1e3, 2), "GFLOPs": round(2 * 16 * 1536 * 7168 / sec / 1e9, 1), "passes": n}
    xa = W.activations(4096, 7168, 0, "cpu", outliers=True)
    sec, n = _cpu_time(lambda: oracle.act_quant(xa), 2.0, 4)
    out["cfg2_act_quant_4096x7168"] = {"ms": round(sec * 1e3, 1), "GBps": round(88.998e6 / sec / 1e9, 2), "passes": n}
    del xa
    wq, wsc = W.random_fp8_weight(18432, 7168, 2, "cpu")
    sec, n = _cpu_time(lambda: oracle.weight_dequant(wq, wsc), 3.0, 3)
    out["cfg2_weight_dequant_18432x7168"] = {"ms": round(sec * 1e3, 1), "GBps": round(396.394e6 / sec / 1e9, 2), "passes": n}
    del wq, wsc
    dec = {}
    for name, (k, nn) in W.DECODE_SHAPES.items():
        w8, ws = W.weight(nn, k, 1, "cpu")
        for m in W.DECODE_M:
            a, a_s = oracle.act_quant(W.activations(m, k, m, "cpu"))
            sec, n = _cpu_time(lambda: oracle.fp8_gemm(a, a_s, w8, ws), 0.6, 2)
            dec[f"{name}_{k}to{nn}_M{m}"] = {"ms": round(sec * 1e3, 1), "GBps": round(decode_bytes(m, nn, k) / sec / 1e9, 2)}
        del w8, ws
    out["cfg3_decode_fp8_gemm"] = dec
    # config 5, reduced: 16 routed experts (2 per group), 256 tokens, the same router rule and expert shapes
    experts_n, tokens, dim, inter = 16, 256, 7168, 2048
    g = torch.Generator().manual_seed(5)
    protos = [W.weight(inter, dim, 40, "cpu"), W.weight(dim, inter, 41, "cpu")]
    ex = (protos[0][0], protos[0][1], protos[1][0], protos[1][1], protos[0][0], protos[0][1])
    xm = W.activations(tokens, dim, 6, "cpu")
    scores = (torch.randn(tokens, experts_n, generator=g) * 1.7).bfloat16()
    wts, idx = oracle.gate_route(scores, torch.randn(experts_n, generator=g) * 0.1, 8, 8, 4, 2.5)
    wts = wts.type_as(xm)
    sec, n = _cpu_time(lambda: oracle.moe(xm, wts, idx, [ex] * experts_n, ex), 4.0, 2)
    flops = 2.0 * 3 * dim * inter * (tokens * 8 + tokens)
    out["cfg5_moe_16_experts_256_tokens"] = {
        "ms": round(sec * 1e3, 1), "TFLOPs": round(flops / sec / 1e12, 4), "passes": n,
        "scaling": "1/16 of the full layer's tokens and routed experts (flops 1/16); at this rate the full layer "
                   f"(3.247e12 flop) would take {3.247e12 / (flops / sec):.1f} s"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only-absorb", type=int, default=0, metavar="TOKENS",
                    help="profiling aid: run only the wkv_b_absorb leg at this token count and print its JSON")
    ap.add_argument("--decode-trace", action="store_true",
                    help="profiling aid: run only the decode sweep as plain launches (see decode_trace) and print "
                         "the cell order")
    ap.add_argument("--grouped-rows-sweep", action="store_true",
                    help="profiling aid: run only the grouped GEMM with equal row counts per group (see "
                         "grouped_rows_sweep)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device copy (a kernel of known HBM traffic) so that rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings of the same run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path is built and measured on ONE GPU (one GPU's share of the work at its real "
                 "shape); --gpus must be 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback.")

    import dsv3fp8 as K                      # fails loudly if libdsv3fp8.so has not been built
    from dsv3fp8 import workloads as W
    torch.set_default_dtype(torch.bfloat16)  # as the reference's caller does (generate.py:109)
    torch.cuda.set_device(0)
    if args.decode_trace:
        decode_trace(K, W)
        return
    if args.grouped_rows_sweep:
        grouped_rows_sweep(K, W)
        return
    if args.only_absorb:
        if args.copy_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
            torch.empty_like(src).copy_(src)
            torch.cuda.synchronize()
        print(json.dumps({"wkv_b_absorb": run_absorb(K, W, (args.only_absorb,))}), flush=True)
        return

    M = W.PREFILL_M
    k, n = W.PREFILL_SHAPES["w1"]
    x = W.activations(M, k, 0, "cuda")
    w8, ws = W.weight(n, k, 1, "cuda")
    flops = 2.0 * M * n * k

    def step():
        a, a_s = K.act_quant(x, 128, None)
        return K.fp8_gemm(a, a_s, w8, ws)

    settle(step, SETTLE_S)
    ms = time_loop(step, args.steps, args.warmup)
    value = flops / ms / 1e9                                 # TFLOP/s

    a, a_s = K.act_quant(x)
    gemm_ms = time_loop(lambda: K.fp8_gemm(a, a_s, w8, ws), args.steps, args.warmup)
    achieved = flops / gemm_ms / 1e9

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    try:
        probes = Probes()
    except Exception as e:                   # the probes are measurement aids: without them the line has no ceilings
        print(f"bench.py: ceiling probes unavailable ({type(e).__name__}: {e})", file=sys.stderr, flush=True)
        probes = NoProbes(f"{type(e).__name__}: {e}")
    ceil = probes.ceilings()
    c = ceil or {}
    line = {
        "metric": METRIC, "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_ms": int(SETTLE_S * 1e3), "graph_settle_ms": int(GRAPH_SETTLE_S * 1e3), "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 (f32 accumulate)", "data": "synthetic",
        "config": {"workload": "cfg4 prefill linear(): act_quant + fp8_gemm, M=4096 tokens, dense MLP w1 "
                               "K=7168 -> N=18432, bf16 act ~N(0,1), fp8 weights block-quantised from ~N(0,0.02), "
                               "bf16 out", "M": M, "N": n, "K": k, "block": 128},
        "roofline": {"kernel": "fp8_gemm_two_heights_kernel", "bound": "mfma", "achieved": round(achieved, 2),
                     "peak": FP8_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / FP8_MFMA_PEAK_TFLOPS, 4), "traffic": measured_traffic(),
                     "launch_us": round(gemm_ms * 1e3, 2), "flops_per_launch": flops,
                     "frac_of_measured_mfma_loop": _ratio(achieved, c.get("fp8_mfma_loop_TFLOPs"), 4),
                     "frac_of_measured_mfma_loop_with_fold": _ratio(achieved, c.get("fp8_mfma_loop_with_fold_TFLOPs"), 4),
                     "frac_of_measured_mfma_loop_with_fold_and_operand_traffic":
                         _ratio(achieved, c.get("fp8_mfma_loop_with_fold_and_operand_traffic_TFLOPs"), 4)},
        "ceilings": ceil,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(W)
    if not args.no_extras:
        line["extras"] = run_extras(K, W, probes, ceil)
        line["roofline_decode"] = decode_roofline(line["extras"]["decode"], ceil)
        if not args.no_cpu:
            line["extras"]["cpu_oracle_other_configs"] = cpu_baselines_other_configs(W)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
