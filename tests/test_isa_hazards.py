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


@pytest.mark.skipif(not Path(HIPCC).exists(), reason="hipcc not available")
@pytest.mark.parametrize("source", ["mnb_skinny.hip", "mnb_mid.hip", "mnb_gemm256.hip", "mnb_rows16_f32.hip"])
def test_no_early_read_of_mfma_results(source):
    from onnxruntime_amd.build import HIPCC_FLAGS
    with tempfile.TemporaryDirectory() as tmp:
        out = Path(tmp) / (source + ".s")
        subprocess.run([HIPCC, *HIPCC_FLAGS, "-S", "--cuda-device-only", str(CSRC / source), "-o", str(out)],
                       check=True, capture_output=True, timeout=600)
        findings = scan(out.read_text())
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
