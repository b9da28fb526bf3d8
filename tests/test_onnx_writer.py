"""The .onnx writer against a model file the reference's own tests hold
(onnxruntime/test/testdata/transform/runtime_optimization/matmulnbits_add.onnx, 357 bytes, copied as a data fixture):
rebuilding that model from its content must give the same bytes."""
from pathlib import Path

import numpy as np

from onnxruntime_amd import onnx_writer as ow

FIXTURE = Path(__file__).parent / "golden" / "matmulnbits_add.onnx"


def test_rebuilds_the_reference_fixture_byte_for_byte():
    want = FIXTURE.read_bytes()
    ref = ow.read_model(want)
    b_q4 = ref["initializers"]["B_Q4"]
    assert b_q4.shape == (3, 1, 16) and b_q4.dtype == np.uint8
    nodes = [
        ow.node("MatMulNBits", ["A", "B_Q4", "B_scales"], ["matmul_out"], name="matmul_Q4", domain="com.microsoft",
                int_attrs=[("K", 2), ("N", 3), ("bits", 4), ("block_size", 32)]),
        ow.node("Add", ["matmul_out", "bias"], ["C"], name="add"),
    ]
    inits = [ow.tensor("B_Q4", b_q4), ow.tensor("B_scales", np.array([-0.125, -0.125, -0.125], np.float32))]
    g = ow.graph("MatMul_Add", nodes, inits,
                 [ow.value_info("A", ow.FLOAT, ["M", 2]), ow.value_info("bias", ow.FLOAT, [3])],
                 [ow.value_info("C", ow.FLOAT, ["M", 3])])
    got = ow.model(g, [("", 21), ("com.microsoft", 1)], ir_version=10)
    assert got == want


def test_matmul_nbits_model_round_trip():
    rng = np.random.default_rng(0)
    N, K, bits, bs = 5, 70, 4, 32
    kb = (K + bs - 1) // bs
    B = rng.integers(0, 256, size=(N, kb, bs * bits // 8), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.1, size=(N, kb)).astype(np.float16)
    zp = rng.integers(0, 256, size=(N, (kb * bits + 7) // 8), dtype=np.uint8)
    bias = rng.standard_normal(N).astype(np.float16)
    data = ow.matmul_nbits_model(B, scales, zp, K, N, bits, bs, bias=bias, prefix="fc1")
    m = ow.read_model(data)
    assert m["opsets"] == [("", 21), ("com.microsoft", 1)]
    (nd,) = m["nodes"]
    assert nd["op_type"] == "MatMulNBits" and nd["domain"] == "com.microsoft"
    assert nd["inputs"] == ["A", "fc1_Q4", "fc1_scales", "fc1_zero_points", "", "fc1_bias"]   # g_idx omitted
    assert nd["attrs"] == {"K": K, "N": N, "bits": bits, "block_size": bs}
    assert np.array_equal(m["initializers"]["fc1_Q4"], B)
    assert np.array_equal(m["initializers"]["fc1_scales"].view(np.uint16), scales.view(np.uint16))
    assert np.array_equal(m["initializers"]["fc1_zero_points"], zp)
    assert np.array_equal(m["initializers"]["fc1_bias"].view(np.uint16), bias.view(np.uint16))
    # symmetric, no bias: three inputs only
    m2 = ow.read_model(ow.matmul_nbits_model(B, scales, None, K, N, bits, bs))
    assert m2["nodes"][0]["inputs"] == ["A", "W_Q4", "W_scales"]
