"""Builds a calibration library: see the package docstring."""
from __future__ import annotations

import argparse
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

from onnxruntime_amd import build as B

HERE = Path(__file__).resolve().parent
OBJ_DIR = HERE / "build"


def lib_path(tag: str = "") -> Path:
    return HERE / (f"libmnb_calibration_{tag}.so" if tag else "libmnb_calibration.so")


def build(tag: str = "", defines=(), only=(), jobs: int = 6, force: bool = False) -> Path:
    OBJ_DIR.mkdir(exist_ok=True)

    def compile_one(src: str) -> str:
        # (mnb_skinny.hip names the decode kernel as a whole: its kernels live in the units of build.SKINNY_UNITS)
        named = not only or src in only or (src in B.SKINNY_UNITS and "mnb_skinny.hip" in only)
        extra = [f"-D{d}" for d in defines] if named else []
        obj = OBJ_DIR / f"{src}.{tag if extra else 'hooks'}.o"
        if not force and not extra and obj.exists() and obj.stat().st_mtime >= max(
                p.stat().st_mtime for p in [B.CSRC / src, *B.CSRC.glob("*.h"), B.PKG.parent / "include" / "mnb_mi355x.h"]):
            return str(obj)
        cmd = [B.hipcc(), *B.HIPCC_FLAGS, *B.EXTRA_FLAGS.get(src, []), "-DMNB_TUNING_HOOKS", *extra, "-c",
               str(B.CSRC / src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
        return str(obj)

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, B.SOURCES))
    out = lib_path(tag)
    subprocess.check_call([B.hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *objs])
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--tag", default="")
    ap.add_argument("-D", dest="defines", action="append", default=[])
    ap.add_argument("--only", default="", help="comma-separated sources the -D switches apply to (default: all)")
    a = ap.parse_args()
    if a.defines and not a.tag:
        ap.error("--tag is required with -D (the plain calibration library has hooks only)")
    print(build(a.tag, a.defines, [s for s in a.only.split(",") if s]))
