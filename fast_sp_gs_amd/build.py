"""Builds libfsgs_hip.so (hand-written HIP for gfx950) in-tree with hipcc. No torch headers are involved."""
from __future__ import annotations

import os
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libfsgs_hip.so"
SOURCES = ["api.hip", "preprocess.hip", "binning.hip", "blend_fwd.hip", "blend_bwd.hip", "blend_topk.hip", "fast_preprocess.hip",
           "fast_blend.hip", "point_ops.hip", "lbs_bwd.hip", "ssim.hip", "epilogue.hip", "simple_knn.hip", "compaction.hip", "gs3d_preprocess.hip", "gs3d_blend.hip", "mlp.hip"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # packed-FP32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def build(verbose: bool = False) -> Path:
    """Compile every HIP source into one shared object; always recompiles."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, *[str(CSRC / s) for s in SOURCES], "-o", str(LIB_PATH)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
