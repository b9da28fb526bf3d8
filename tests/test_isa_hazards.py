"""The generated code of the matrix-core kernels never reads an MFMA result before it is there (see
isa_hazard_scan.py).  Compiles the sources to assembly with the flags of the build; no GPU needed."""
import shutil
import subprocess
import tempfile
from pathlib import Path

import pytest

from isa_hazard_scan import scan

CSRC = Path(__file__).resolve().parents[1] / "onnxruntime_amd" / "csrc"
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


SOURCES = ["mnb_skinny_w4.hip", "mnb_skinny_w4zp.hip", "mnb_skinny_w8.hip", "mnb_skinny_w2.hip", "mnb_mid.hip",
           "mnb_gemm256.hip", "mnb_rows16_f32.hip"]


@pytest.fixture(scope="module")
def assembly():
    """Every source compiled to assembly once, side by side (the decode kernel's four units take a minute or two
    each)."""
    from concurrent.futures import ThreadPoolExecutor
    from onnxruntime_amd.build import HIPCC_FLAGS
    with tempfile.TemporaryDirectory() as tmp:
        def compile_one(source):
            out = Path(tmp) / (source + ".s")
            subprocess.run([HIPCC, *HIPCC_FLAGS, "-S", "--cuda-device-only", str(CSRC / source), "-o", str(out)],
                           check=True, capture_output=True, timeout=900)
            return source, scan(out.read_text())
        with ThreadPoolExecutor(max_workers=7) as ex:
            yield dict(ex.map(compile_one, SOURCES))


@pytest.mark.skipif(not Path(HIPCC).exists(), reason="hipcc not available")
@pytest.mark.parametrize("source", SOURCES)
def test_no_early_read_of_mfma_results(assembly, source):
    findings = assembly[source]
    assert not findings, "\n".join(f"{f}: {w} wait states: {a} -> {b}" for f, w, a, b in findings[:10])


def test_scanner_flags_a_short_distance_and_accepts_nops():
    bad = """_Zk:
\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
\ts_cbranch_scc1 .LBB0_2
\tv_mov_b32_e32 v9, v8
.LBB0_2:
\tv_accvgpr_read_b32 v10, a3
\ts_endpgm
"""
    assert scan(bad) and all(w <= 2 for _, w, _, _ in scan(bad))  # one finding per path to the read
    good = bad.replace("\ts_cbranch_scc1 .LBB0_2\n", "\ts_nop 7\n\ts_cbranch_scc1 .LBB0_2\n")
    assert scan(good) == []
    chained = """_Zk:
\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
\ts_nop 7
\tv_accvgpr_read_b32 v10, a3
\ts_endpgm
"""
    assert scan(chained) == []
