#!/usr/bin/env python3
"""Convert the reference's own MatMulNBits op-test data into a compact fixture.

Source (read as data, in the build container only):
  /root/reference/js/web/test/data/ops/matmulnbits.jsonc
That file is the test-vector table of the reference's JavaScript op tests: for
each case it lists the operator attributes, the input tensors (A, B, scales and
optionally zero_points) and the expected output tensor.  All 23 cases are 4-bit,
fp32, with integer-valued data, so the expected outputs are exact.

Output: tests/golden/js_matmulnbits_cases.json (committed; inputs + expected
outputs only, no code).
"""
import json
import re
import sys
from pathlib import Path

SRC = Path("/root/reference/js/web/test/data/ops/matmulnbits.jsonc")
DST = Path(__file__).with_name("js_matmulnbits_cases.json")


def strip_comments(text: str) -> str:
    return re.sub(r"^\s*//.*$", "", text, flags=re.M)


def main() -> int:
    groups = json.loads(strip_comments(SRC.read_text()))
    out = []
    for g in groups:
        assert g["operator"] == "MatMulNBits"
        attrs = {a["name"]: a["data"] for a in g["attributes"]}
        for c in g["cases"]:
            out.append({
                "name": c["name"],
                "attrs": attrs,
                "inputs": [{"dims": t["dims"], "type": t["type"], "data": t["data"]} for t in c["inputs"]],
                "outputs": [{"dims": t["dims"], "type": t["type"], "data": t["data"]} for t in c["outputs"]],
            })
    DST.write_text(json.dumps({"source": "js/web/test/data/ops/matmulnbits.jsonc", "cases": out},
                              separators=(",", ":")) + "\n")
    print(f"wrote {DST} with {len(out)} cases")
    return 0


if __name__ == "__main__":
    sys.exit(main())
