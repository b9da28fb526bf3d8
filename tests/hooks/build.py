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


def _product():
    sys.path.insert(0, str(HERE.parent.parent))
    from onnxruntime_amd import build as B
    return B


def compile_hooked() -> Path:
    """The one object that differs from the product's (needs no product object, so it can run beside that build)."""
    B = _product()
    B.OBJ_DIR.mkdir(exist_ok=True)
    obj = B.OBJ_DIR / (HOOKED + ".hooks.o")
    cmd = [B.hipcc(), *B.HIPCC_FLAGS, *B.EXTRA_FLAGS.get(HOOKED, []), "-DMNB_TEST_HOOKS", "-c", str(B.CSRC / HOOKED),
           "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {HOOKED} (test hooks):\n{r.stderr}")
    return obj


def link(hooked: Path) -> Path:
    B = _product()
    objs = []
    for src in B.SOURCES:
        obj = hooked if src == HOOKED else B.OBJ_DIR / (src + ".o")
        if not obj.exists():
            raise RuntimeError(f"{obj} is missing: build the product library first (python -m onnxruntime_amd.build)")
        objs.append(str(obj))
    subprocess.check_call([B.hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs])
    return LIB


def build() -> Path:
    return link(compile_hooked())


if __name__ == "__main__":
    print(build())
