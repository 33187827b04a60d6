"""Builds liblce_gfx950.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950.

The library is seven objects: ``csrc/lce_abi.hip`` (the C ABI and the kernels that do not depend on the GEMM element
type) and ``csrc/lce_dtype.hip`` compiled once per (element type, direction).  They are compiled side by side
(``LCE_BUILD_JOBS`` processes, default: the host's cores, at most one per object) and linked into one shared library.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(OUT_DIR, "obj")
OUT = os.path.join(OUT_DIR, "liblce_gfx950.so")

# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32 from scalar code
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-cuda-compat",  # non-template kernels in the shared headers are `inline`: one weak host stub per object
]

# (object name, source, defines); element types by their LCE_DTYPE_* numbers: 0 bf16, 1 fp32, 2 fp16.  The backward objects
# take longest, so they come first.
OBJECTS = [
    ("bwd_bf16", "lce_dtype.hip", ["-DLCE_TU_DTYPE=0", "-DLCE_TU_PART=1"]),
    ("bwd_f16", "lce_dtype.hip", ["-DLCE_TU_DTYPE=2", "-DLCE_TU_PART=1"]),
    ("bwd_f32", "lce_dtype.hip", ["-DLCE_TU_DTYPE=1", "-DLCE_TU_PART=1"]),
    ("fwd_bf16", "lce_dtype.hip", ["-DLCE_TU_DTYPE=0", "-DLCE_TU_PART=0"]),
    ("fwd_f16", "lce_dtype.hip", ["-DLCE_TU_DTYPE=2", "-DLCE_TU_PART=0"]),
    ("fwd_f32", "lce_dtype.hip", ["-DLCE_TU_DTYPE=1", "-DLCE_TU_PART=0"]),
    ("abi", "lce_abi.hip", []),
]


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 target feature and says so: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({' '.join(cmd[-3:])}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra: list[str] | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    jobs = int(os.environ.get("LCE_BUILD_JOBS", "0")) or min(len(OBJECTS), os.cpu_count() or 1)
    objs = [os.path.join(OBJ_DIR, name + ".o") for name, _, _ in OBJECTS]
    cmds = [
        [hipcc, *FLAGS, *(extra or []), *defs, "-c", os.path.join(CSRC, src), "-o", obj]
        for (_, src, defs), obj in zip(OBJECTS, objs)
    ]
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for fut in [pool.submit(_run, cmd, verbose) for cmd in cmds]:
            fut.result()
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT], verbose)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
