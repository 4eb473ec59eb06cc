"""Builds libfsgs_hip.so (hand-written HIP for gfx950) in-tree with hipcc. No torch headers are involved.

Every source is compiled to its own object (in parallel) and the objects are linked into one shared library.
`build()` recompiles everything; `build(incremental=True)` (or `python -m fast_sp_gs_amd.build -i`) recompiles only
sources that are newer than their object, or older than a header.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = PKG_DIR / "build"
LIB_PATH = PKG_DIR / "libfsgs_hip.so"
SOURCES = ["api.hip", "preprocess.hip", "binning.hip", "blend_fwd.hip", "blend_bwd.hip", "blend_topk.hip", "fast_preprocess.hip",
           "fast_blend.hip", "point_ops.hip", "lbs_bwd.hip", "ssim.hip", "epilogue.hip", "simple_knn.hip", "compaction.hip", "gs3d_preprocess.hip", "gs3d_blend.hip", "mlp.hip"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed-FP32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Build-time choices of the kernels (-DFSGS_BWD_ROWS=1, -DFSGS_FWD_BATCH=..., ...) can be handed in through the
# environment; they select among variants that compute the same results.
HIPCC_FLAGS += os.environ.get("FSGS_HIPCC_DEFINES", "").split()
NOISE = "packed-fp32-ops"


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _run(cmd) -> str:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if NOISE not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{log}")
    return log


def build(verbose: bool = False, incremental: bool = False, jobs: int = 0) -> Path:
    """Compile every HIP source into one shared object."""
    OBJ_DIR.mkdir(exist_ok=True)
    hipcc = hipcc_path()
    headers_mtime = max(p.stat().st_mtime for p in list(CSRC.glob("*.hpp")) + list((PKG_DIR.parent / "include").glob("*.h")))
    todo = []
    for s in SOURCES:
        src, obj = CSRC / s, OBJ_DIR / (s + ".o")
        if incremental and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, headers_mtime):
            continue
        todo.append((src, obj))
    jobs = jobs or min(len(todo) or 1, int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        logs = list(pool.map(lambda so: _run([hipcc, *HIPCC_FLAGS, "-c", str(so[0]), "-o", str(so[1])]), todo))
    logs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[str(OBJ_DIR / (s + ".o")) for s in SOURCES],
                      "-o", str(LIB_PATH)]))
    if verbose:
        text = "\n".join(l for l in logs if l.strip())
        if text:
            print(text)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, incremental="-i" in sys.argv[1:]))
