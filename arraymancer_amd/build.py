"""Builds libam_hip.so (the gfx950 HIP library behind the C ABI of include/am_hip.h) in-tree.

    python -m arraymancer_amd.build        # compile every translation unit and link

hipcc cross-compiles for gfx950 without a GPU. Objects go to arraymancer_amd/csrc/_obj/, the
library to arraymancer_amd/libam_hip.so.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "_obj")
LIB_PATH = os.path.join(PKG_DIR, "libam_hip.so")

SOURCES = [
    "runtime.hip", "diag.hip",
    "elementwise_f32.hip", "elementwise_f64.hip", "elementwise_i32.hip", "elementwise_i64.hip",
    "gemm_f32.hip", "gemm_f64.hip", "gemm_i32.hip", "gemm_i64.hip", "gemv.hip", "im2col.hip", "reduce.hip", "loss.hip", "gru.hip", "optim.hip",
]

# -ffp-contract=off: every float operation of an epilogue / map body is rounded on its own, so
# results are comparable bit for bit with the CPU statement of the same expression (the matrix
# products themselves are MFMA builtins and are not affected).
# -packed-fp32-ops off: no packed-FP32 VALU forms are generated.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
] + os.environ.get("AM_HIP_EXTRA_FLAGS", "").split()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr[-4000:]}")
    return obj


def build(jobs: int | None = None, verbose: bool = False) -> str:
    """Compiles every source (always, also when a built library exists) and links. Returns the
    path of the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB_PATH} from {len(objs)} objects")
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
