"""Builds, in-tree and with hipcc:
  libmnb_mi355x.so            HIP kernels + C ABI for gfx950
  libmnb_probe.so             read-bandwidth and matrix-core-rate probes that only bench.py loads (csrc/mnb_probe.h)
  libonnxruntime_mi355x_ep.so the ONNX Runtime plugin execution provider above that C ABI (needs the ONNX Runtime
                              C API headers: directory given by ORT_INCLUDE_DIR, or an onnxruntime checkout at
                              ORT_SOURCE_DIR / /root/reference)

Usage: python -m onnxruntime_amd.build
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

# (the decode kernel's four translation units come first: they compile longest)
SKINNY_UNITS = ["mnb_skinny_w4.hip", "mnb_skinny_w4zp.hip", "mnb_skinny_w8.hip", "mnb_skinny_w2.hip"]
SOURCES = [*SKINNY_UNITS, "mnb_api.hip", "mnb_pack.hip", "mnb_quant.hip", "mnb_gemv.hip", "mnb_skinny.hip", "mnb_mid.hip", "mnb_gemm256.hip", "mnb_gemm_i8.hip", "mnb_gemm32.hip", "mnb_rows16_f32.hip", "mnb_fused.hip", "mnb_variant.hip"]
PROBE_LIB = PKG / "libmnb_probe.so"
PROBE_SOURCES = ["mnb_probe.hip"]

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


# Per-source flags.  The decode and streaming kernels take what their first loads need as leading scalar arguments; the compiler is
# asked to have those preloaded into SGPRs at wavefront start (firmware without the feature runs the compatibility
# prologue the compiler emits in front of the kernel, which loads them the usual way).
_PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=14"]
EXTRA_FLAGS = {**{u: _PRELOAD for u in SKINNY_UNITS}, "mnb_gemv.hip": _PRELOAD, "mnb_mid.hip": _PRELOAD}


def _compile(src: str, extra=()) -> Path:
    OBJ_DIR.mkdir(exist_ok=True)
    obj = OBJ_DIR / (src + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), *extra, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(msgs))
    if msgs:
        print("\n".join(msgs), file=sys.stderr)
    return obj


def build(force: bool = True, jobs: int = 6) -> Path:
    """Compiles every HIP source and links the shared library. Always recompiles when force is set."""
    srcs = [CSRC / s for s in SOURCES]
    hdrs = list(CSRC.glob("*.h")) + [PKG.parent / "include" / "mnb_mi355x.h"]
    if not force and LIB.exists():
        newest = max(p.stat().st_mtime for p in srcs + hdrs)
        if LIB.stat().st_mtime >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES + PROBE_SOURCES))
    n = len(SOURCES)
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs[:n])])
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(PROBE_LIB),
                           *map(str, objs[n:])])
    return LIB


EP_LIB = PKG / "libonnxruntime_mi355x_ep.so"
EP_SOURCES = ["ep_lib_entry.cc", "ep_factory.cc", "ep.cc", "ep_kernels.cc", "ep_fused_kernels.cc", "ep_compile.cc", "ep_profiler.cc",
              "ep_device_runtime.cc"]


def ort_include_dir() -> Path | None:
    """Directory that holds onnxruntime_c_api.h, or None when no ONNX Runtime headers are installed."""
    cands = []
    if os.environ.get("ORT_INCLUDE_DIR"):
        cands.append(Path(os.environ["ORT_INCLUDE_DIR"]))
    src = Path(os.environ.get("ORT_SOURCE_DIR", "/root/reference"))
    cands.append(src / "include" / "onnxruntime" / "core" / "session")
    for c in cands:
        if (c / "onnxruntime_c_api.h").exists() and (c / "onnxruntime_ep_c_api.h").exists():
            return c
    return None


def _compile_ep(src: str, inc: Path) -> Path:
    out_dir = OBJ_DIR / "ep"
    out_dir.mkdir(parents=True, exist_ok=True)
    obj = out_dir / (src + ".o")
    cmd = [hipcc(), "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
           "-I", str(inc), "-I", str(PKG.parent / "include"), "-c", str(CSRC / "ep" / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on ep/{src}:\n{r.stderr}")
    if r.stderr.strip():
        print(r.stderr, file=sys.stderr)
    return obj


def build_ep(jobs: int = 4) -> Path | None:
    """Compiles the plugin EP against the ONNX Runtime headers found by ort_include_dir(). Returns None (and keeps a
    previously built library) when no headers are available."""
    inc = ort_include_dir()
    if inc is None:
        print("onnxruntime_amd.build: ONNX Runtime headers not found, plugin EP not rebuilt", file=sys.stderr)
        return EP_LIB if EP_LIB.exists() else None
    if not LIB.exists():
        build()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile_ep(s, inc), EP_SOURCES))
    cmd = [hipcc(), "-shared", "-fPIC", "-o", str(EP_LIB), *map(str, objs), "-L", str(PKG), "-lmnb_mi355x",
           "-Wl,-rpath,$ORIGIN", "-Wl,--no-undefined"]
    subprocess.check_call(cmd)
    return EP_LIB


if __name__ == "__main__":
    print(build(force=True))
    print(build_ep())
