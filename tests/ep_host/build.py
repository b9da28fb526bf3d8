"""Builds the ONNX Runtime host test double (libort_host_shim.so) that the plugin-EP tests load.

It needs the same ONNX Runtime C API headers as the plugin itself; without them a previously built library is kept.
Usage: python -m tests.ep_host.build
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB = HERE / "libort_host_shim.so"


def build() -> Path | None:
    sys.path.insert(0, str(HERE.parent.parent))
    from onnxruntime_amd.build import ort_include_dir

    inc = ort_include_dir()
    if inc is None:
        print("tests.ep_host.build: ONNX Runtime headers not found, host shim not rebuilt", file=sys.stderr)
        return LIB if LIB.exists() else None
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fPIC", "-shared", "-Wall", "-I", str(inc), "-o", str(LIB),
           str(HERE / "ort_host_shim.cc"), "-ldl"]
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build())
