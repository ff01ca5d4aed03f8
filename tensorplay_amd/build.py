"""Builds the gfx950 libraries in-tree with hipcc (which cross-compiles without a GPU present).

``libtpq_gfx950.so``        the C-ABI kernel library: the operators of include/tpq.h and nothing else.
``libtpq_gfx950_hooks.so``  the same sources with -DTPQ_TEST_HOOKS: exports tpq_set_kernel_override as well, with which the
                            tests pin a route so that a kernel is checked on every shape it can take.  Only tests load it.
``libtpq_probe.so``         the pure-read measurement probe (csrc/probe.hip).  Only bench.py loads it.

Usage: ``python -m tensorplay_amd.build`` (all three) or ``tensorplay_amd.build.build_library()``.
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
HOOKS_LIB_PATH = os.path.join(HERE, "libtpq_gfx950_hooks.so")
PROBE_LIB_PATH = os.path.join(HERE, "libtpq_probe.so")
QUANT_STAMPS_LIB_PATH = os.path.join(HERE, "libtpq_quant_stamps.so")  # the row quantizer with clock readings per phase (quant_stamps.py)

SOURCES = ["tpq_core.hip", "quantize_rowwise.hip", "int4_mm.hip", "int4_flight.hip", "int8_gemm.hip", "ternary_mm.hip", "int8pack_mm.hip", "affine_quant.hip", "lowbit_mm.hip", "rms_norm.hip", "dense_mm.hip", "packed_linear.hip"]
# the sources that read a pinned route: the only ones compiled a second time for the test-hook library
HOOK_SOURCES = ["tpq_core.hip", "int4_mm.hip", "int8_gemm.hip", "lowbit_mm.hip"]

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


def _compile(cc: str, src: str, obj: str, extra: list, verbose: bool) -> str:
    cmd = [cc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
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


def _link(cc: str, objs: list, path: str) -> str:
    tmp = path + ".tmp"
    proc = subprocess.run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, path)
    return path


def build_library(verbose: bool = False, jobs: int = 6, tuning: bool = False, hooks: bool = True, probe: bool = True) -> str:
    """Compiles every source and links the kernel library; with hooks / probe also the test-hook library and the
    measurement probe.  tuning=True compiles the sweep knobs in (-DTPQ_TUNING: TPQ_* environment variables pick kernels
    and workgroup shapes); the library that ships is built without it and never reads the environment."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    cc = hipcc()
    tune = ["-DTPQ_TUNING"] if tuning else []
    work = [(src, os.path.join(obj_dir, src.replace(".hip", ".o")), tune) for src in SOURCES]
    if hooks:
        work += [(src, os.path.join(obj_dir, src.replace(".hip", ".hooks.o")), tune + ["-DTPQ_TEST_HOOKS"]) for src in HOOK_SOURCES]
    if probe:
        work.append(("probe.hip", os.path.join(obj_dir, "probe.o"), []))
        work.append(("quantize_rowwise.hip", os.path.join(obj_dir, "quantize_rowwise.stamps.o"), ["-DTPQ_QUANT_STAMPS"]))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda w: _compile(cc, w[0], w[1], w[2], verbose), work))
    plain = [os.path.join(obj_dir, src.replace(".hip", ".o")) for src in SOURCES]
    _link(cc, plain, LIB_PATH)
    if hooks:
        hooked = [os.path.join(obj_dir, src.replace(".hip", ".hooks.o" if src in HOOK_SOURCES else ".o")) for src in SOURCES]
        _link(cc, hooked, HOOKS_LIB_PATH)
    if probe:
        _link(cc, [os.path.join(obj_dir, "probe.o")], PROBE_LIB_PATH)
        _link(cc, [os.path.join(obj_dir, "quantize_rowwise.stamps.o"), os.path.join(obj_dir, "tpq_core.o")], QUANT_STAMPS_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv, tuning="--tuning" in sys.argv))
