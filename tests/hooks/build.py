"""Builds tests/hooks/libmnb_test_hooks.so: the product library with the tile GEMM recompiled under -DMNB_TEST_HOOKS.

The hook build adds one exported function, MnbTestSetSplitHooks(spin_limit, drop_odd_lower), through which a test
bounds the tile GEMM's cross-workgroup wait and leaves the lower parts of odd-numbered tiles uncomputed: the give-up
path of that wait then runs from the host's choice of arguments, with every kernel still ending normally.  Every other
object is the product's own (onnxruntime_amd/build/*.o), so the product library must have been built first.
Usage: python -m tests.hooks.build
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB = HERE / "libmnb_test_hooks.so"
HOOKED = "mnb_gemm256.hip"


def build() -> Path:
    sys.path.insert(0, str(HERE.parent.parent))
    from onnxruntime_amd import build as B
    objs = []
    for src in B.SOURCES:
        obj = B.OBJ_DIR / (src + ".o")
        if src == HOOKED:
            obj = B.OBJ_DIR / (src + ".hooks.o")
            cmd = [B.hipcc(), *B.HIPCC_FLAGS, *B.EXTRA_FLAGS.get(src, []), "-DMNB_TEST_HOOKS", "-c", str(B.CSRC / src),
                   "-o", str(obj)]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"hipcc failed on {src} (test hooks):\n{r.stderr}")
        elif not obj.exists():
            raise RuntimeError(f"{obj} is missing: build the product library first (python -m onnxruntime_amd.build)")
        objs.append(str(obj))
    subprocess.check_call([B.hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs])
    return LIB


if __name__ == "__main__":
    print(build())
