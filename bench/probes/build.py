"""Builds libdsv3probe.so, the benchmark's ceiling probes (read stream, copy, read/write mixes, fp8 MFMA loops, empty
launch) for gfx950, beside its source.  Measurement infrastructure of bench.py; the product library never loads it.

    python bench/probes/build.py
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
SRC = HERE / "probes.hip"
LIB_PATH = HERE / "libdsv3probe.so"

# -packed-fp32-ops off: the compiler must not form v_pk_{add,mul,fma}_f32 from scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-fno-fast-math", "-ffp-contract=off",
]


def build_probes(verbose: bool = True) -> Path:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: cannot build libdsv3probe.so")
    tmp = LIB_PATH.with_suffix(".so.tmp")
    r = subprocess.run([hipcc, *HIPCC_FLAGS, "-shared", str(SRC), "-o", str(tmp)], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {SRC.name}:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[build] linked {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_probes()
    sys.exit(0)
