"""Compile the HIP sources in ``csrc/`` into ``libajq.so`` next to this file.

Cross-compiles for gfx950 with hipcc; needs no GPU.  Run as
``python -m ajllm_amd.build`` or call :func:`build_library`.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
SOURCE = PACKAGE_DIR / "csrc" / "ajq.hip"
LIBRARY = PACKAGE_DIR / "libajq.so"
# measurement probes for bench.py (include/ajq_bench.h); the operator library does not depend on it
BENCH_SOURCE = PACKAGE_DIR / "csrc" / "ajq_bench.hip"
BENCH_LIBRARY = PACKAGE_DIR / "libajq_bench.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # kernel arguments arrive in SGPRs with the wave instead of by a scalar load
    # at its start (the short GEMV kernels issue their first loads that much sooner)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def build_library(verbose: bool = False, source: Path = SOURCE, library: Path = LIBRARY) -> Path:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = library.with_suffix(".so.tmp%d" % os.getpid())
    cmd = [hipcc, *HIPCC_FLAGS, str(source), "-o", str(tmp)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    stderr = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{stderr}")
    if stderr.strip() and verbose:
        print(stderr, file=sys.stderr)
    os.replace(tmp, library)
    return library


def build_bench_library(verbose: bool = False) -> Path:
    return build_library(verbose, BENCH_SOURCE, BENCH_LIBRARY)


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_bench_library(verbose=True))
