"""Builds ``libtpq_gfx950.so`` (the C-ABI kernel library) in-tree with hipcc.

Usage: ``python -m tensorplay_amd.build`` or ``tensorplay_amd.build.build_library()``.
hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libtpq_gfx950.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["tpq_core.hip", "quantize_rowwise.hip", "int4_mm.hip", "int4_flight.hip", "int8_gemm.hip", "ternary_mm.hip", "int8pack_mm.hip", "affine_quant.hip", "lowbit_mm.hip", "rms_norm.hip", "probe.hip"]

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32.
# -ffp-contract=off: fused multiply-adds only where the source asks for one,
# so fp32 epilogues round exactly like the scalar CPU code they are checked against.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-warning-option",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the kernel library cannot be built")
    return exe


def build_library(verbose: bool = False, jobs: int = 5, tuning: bool = False) -> str:
    """tuning=True compiles the sweep knobs in (-DTPQ_TUNING: TPQ_* environment variables pick kernels and workgroup
    shapes); the library that ships is built without it and never reads the environment."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    cc = hipcc()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        cmd = [cc, *HIPCC_FLAGS, *(["-DTPQ_TUNING"] if tuning else []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        proc = subprocess.run(cmd, capture_output=True, text=True)
        noise = "packed-fp32-ops' is not a recognized feature"
        err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    link = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv, tuning="--tuning" in sys.argv))
