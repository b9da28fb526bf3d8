"""Loader of the committed golden vectors (the reference's own JS op-test table for MatMulNBits)."""
import json
from pathlib import Path

import numpy as np

_PATH = Path(__file__).resolve().parent / "golden" / "js_matmulnbits_cases.json"
_DT = {"float32": np.float32, "uint8": np.uint8, "float16": np.float16}


def _tensor(t):
    if t["type"] == "uint8":  # the JS harness stores into a Uint8Array: values wrap modulo 256
        return (np.array(t["data"], dtype=np.int64) & 0xFF).astype(np.uint8).reshape(t["dims"])
    return np.array(t["data"], dtype=_DT[t["type"]]).reshape(t["dims"])


def load_js_cases():
    """Yields dicts: name, N, K, bits, block_size, A, B, scales, zero_points (or None), Y."""
    doc = json.loads(_PATH.read_text())
    out = []
    for c in doc["cases"]:
        t = [_tensor(i) for i in c["inputs"]]
        y = c["outputs"][0]
        out.append({
            "name": c["name"],
            "N": c["attrs"]["N"], "K": c["attrs"]["K"], "bits": c["attrs"]["bits"],
            "block_size": c["attrs"]["block_size"],
            "A": t[0], "B": t[1], "scales": t[2], "zero_points": t[3] if len(t) > 3 else None,
            "Y": np.array(y["data"], dtype=_DT[y["type"]]).reshape(y["dims"]),
        })
    return out
