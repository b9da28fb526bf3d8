"""Builds libmnb_mi355x.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m onnxruntime_amd.build [--force]
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libmnb_mi355x.so"
OBJ_DIR = PKG / "build"

SOURCES = ["mnb_api.hip", "mnb_pack.hip", "mnb_gemv.hip", "mnb_skinny.hip", "mnb_gemm_mfma.hip", "mnb_gemm256.hip"]

# -packed-fp32-ops is switched off on purpose: scalar fp32 code must not be fused into v_pk_*_f32.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=on",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the MI355X library cannot be built")
    return exe


def _compile(src: str, extra=()) -> Path:
    OBJ_DIR.mkdir(exist_ok=True)
    obj = OBJ_DIR / (src + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(msgs))
    if msgs:
        print("\n".join(msgs), file=sys.stderr)
    return obj


def build(force: bool = True, jobs: int = 4) -> Path:
    """Compiles every HIP source and links the shared library. Always recompiles when force is set."""
    srcs = [CSRC / s for s in SOURCES]
    hdrs = list(CSRC.glob("*.h")) + list(CSRC.glob("*.cuh")) + [PKG.parent / "include" / "mnb_mi355x.h"]
    if not force and LIB.exists():
        newest = max(p.stat().st_mtime for p in srcs + hdrs)
        if LIB.stat().st_mtime >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
