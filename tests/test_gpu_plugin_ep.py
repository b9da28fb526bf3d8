"""MatMulNBits through the plugin execution provider: the ONNX Runtime host test double drives the plugin library
through the plugin-EP C ABI (factory, capability, allocator, data transfer, PrePack, Memcpy kernels, Compute) and the
output is compared with the oracle and the reference's own vectors."""
import numpy as np
import pytest

from ep_host import host
from golden_cases import load_js_cases
from gpu_util import check_against_oracle
from onnxruntime_amd.synthetic import make_case

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not host.available(), reason="plugin EP or host shim not built")]

JS = load_js_cases()


def _run(c, A=None, **kw):
    return host.run_matmul_nbits(c.N, c.K, c.bits, c.block_size, c.A if A is None else A, c.B, c.scales,
                                 c.zero_points, None, c.bias, **kw)


@pytest.mark.parametrize("case", JS[::3], ids=[f"{i}" for i in range(0, len(JS), 3)])
def test_reference_vectors_through_plugin(case):
    c = case
    y, trace = host.run_matmul_nbits(c["N"], c["K"], c["bits"], c["block_size"], c["A"], c["B"], c["scales"],
                                     c["zero_points"])
    assert "claimed=1" in trace
    assert np.array_equal(y, c["Y"]), c["name"]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits,bs,zp,bias", [(4, 32, True, True), (4, 128, False, False), (8, 64, True, False),
                                             (8, 16, False, True)])
@pytest.mark.parametrize("M", [1, 7, 200])
def test_prepacked_route(oracle, dtype, bits, bs, zp, bias, M):
    c = make_case(M, 320, 512, bits, bs, dtype, has_zp=zp, has_bias=bias, seed=M + bits + bs)
    y, trace = _run(c)
    want = "prepacked=1,2,3," if zp else "prepacked=1,2,"
    assert want in trace, trace          # B, scales (and zero points) were taken over by PrePack
    check_against_oracle(oracle, c, y)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_unpacked_route_matches_prepacked(oracle, dtype):
    """Scales fed per run (not constant): no PrePack, Compute packs into stream-ordered scratch. Same bits out."""
    c = make_case(5, 200, 384, 4, 32, dtype, has_zp=True, has_bias=True, seed=3)
    y_packed, _ = _run(c)
    y_unpacked, trace = _run(c, constant=("B",), repeat=3)
    assert "prepacked= " in trace, trace
    assert np.array_equal(y_packed.view(np.uint8), y_unpacked.view(np.uint8))
    check_against_oracle(oracle, c, y_unpacked)


def test_batched_activations_and_empty_output(oracle):
    c = make_case(6, 96, 128, 4, 32, np.float16, has_zp=False, seed=11)
    A3 = c.A.reshape(2, 3, c.K)
    y, _ = _run(c, A=A3)
    assert y.shape == (2, 3, c.N)
    check_against_oracle(oracle, c, y.reshape(6, c.N))
    y0, _ = _run(c, A=np.zeros((0, c.K), np.float16))
    assert y0.shape == (0, c.N)


def test_nodes_left_to_the_cpu_provider():
    c = make_case(2, 64, 128, 4, 32, np.float32, has_zp=True, seed=5)
    g = (np.arange(c.K) // 32).astype(np.int32)

    def not_claimed(**kw):
        args = dict(zero_points=c.zero_points, g_idx=None, bits=4, B=c.B, scales=c.scales)
        args.update(kw)
        with pytest.raises(host.EpHostError) as e:
            host.run_matmul_nbits(c.N, c.K, args["bits"], 32, c.A, args["B"], args["scales"], args["zero_points"],
                                  args["g_idx"], None, constant=args.get("constant", ("B", "scales", "zero_points",
                                                                                      "g_idx")))
        assert e.value.code == host.NOT_CLAIMED

    # a group index, typed zero points: transformed when the weights are packed, so every operand must be constant
    not_claimed(g_idx=g, constant=("B", "scales", "zero_points"))
    not_claimed(g_idx=g, constant=("B", "zero_points", "g_idx"))
    not_claimed(zero_points=np.full((c.N, 4), 7.5, np.float32), constant=("B", "scales"))
    # the reference's own limits: 8-bit weights with either, zero points of another float type
    c8 = make_case(2, 64, 128, 8, 32, np.float32, seed=5)
    not_claimed(bits=8, B=c8.B, scales=c8.scales, zero_points=None, g_idx=g)
    not_claimed(bits=8, B=c8.B, scales=c8.scales, zero_points=np.full((c.N, 4), 100.5, np.float32))
    not_claimed(zero_points=np.full((c.N, 4), 7.5, np.float16))


def test_weights_prepacked_for_another_provider_are_not_claimed(oracle):
    """weight_prepacked = 1 / 2 marks B as being in a CUDA fpA_intB layout (contrib_defs.cc:3800-3805): this provider
    would repack it as if it were canonical, so it leaves the node alone; 0 (or the attribute absent) is claimed."""
    c = make_case(2, 64, 128, 4, 32, np.float16, has_zp=True, seed=8)
    names = ["A", "B", "scales", "zero_points", "g_idx", "bias"]
    types = ["T1", "T2", "T1", "T3", "T4", "T1"]
    schema = ["K", "N", "bits", "block_size", "accuracy_level", "weight_prepacked"]

    def run(prepacked):
        attrs = {"K": c.K, "N": c.N, "bits": 4, "block_size": 32, "accuracy_level": 0}
        if prepacked is not None:
            attrs["weight_prepacked"] = prepacked
        return host.run_node("MatMulNBits", attrs, schema, names, types,
                             [c.A, c.B, c.scales, c.zero_points, None, None], ("B", "scales", "zero_points"),
                             [(c.M, c.N)])

    for prepacked in (1, 2):
        with pytest.raises(host.EpHostError) as e:
            run(prepacked)
        assert e.value.code == host.NOT_CLAIMED
    for prepacked in (None, 0):
        (y,), trace = run(prepacked)
        assert "claimed=1" in trace
        check_against_oracle(oracle, c, y)


def test_shape_errors_carry_the_reference_messages():
    c = make_case(2, 64, 128, 4, 32, np.float32, has_zp=True, seed=6)
    INVALID_ARGUMENT = 2
    with pytest.raises(host.EpHostError) as e:   # constant scales of the wrong size: caught in PrePack
        host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales.reshape(-1)[:-1], c.zero_points)
    assert e.value.code == INVALID_ARGUMENT and "scales" in e.value.message
    with pytest.raises(host.EpHostError) as e:   # run-time scales of the wrong size: caught in Compute
        host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales.reshape(-1)[:-1], c.zero_points, constant=("B",))
    assert e.value.code == INVALID_ARGUMENT and "scales" in e.value.message
    with pytest.raises(host.EpHostError) as e:   # A whose inner dimension is not K
        host.run_matmul_nbits(c.N, c.K, 4, 32, c.A[:, :-1], c.B, c.scales, c.zero_points)
    assert e.value.code == INVALID_ARGUMENT and "dimension mismatch" in e.value.message


def test_accuracy_level_4_takes_int8_activations_only_with_the_sessions_consent(oracle):
    """accuracy_level = 4 permits int8 activations.  Without the session configuration entry the node is computed at
    full accuracy; with "ep.mi355x.int8_activations" = "1" it is computed with the reference's int8-activation
    arithmetic (bit for bit the oracle's restatement); configurations without an int8 route keep full accuracy."""
    M, N, K, bits, bs = 40, 192, 512, 4, 64
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, has_bias=True, seed=21)
    want8 = oracle.C.matmul_int8(c.A, c.B, c.scales, c.zero_points, c.bias, N, K, bs)
    want0 = oracle.C.matmul(c.A, c.B, c.scales, c.zero_points, c.bias, N, K, bits, bs)
    y, _ = host.run_matmul_nbits(N, K, bits, bs, c.A, c.B, c.scales, c.zero_points, bias=c.bias, accuracy_level=4)
    check_against_oracle(oracle, c, y)
    assert not np.array_equal(y, want8)
    with host.session_config(ep__mi355x__int8_activations=1):
        y8, trace = host.run_matmul_nbits(N, K, bits, bs, c.A, c.B, c.scales, c.zero_points, bias=c.bias,
                                          accuracy_level=4)
        assert np.array_equal(y8, want8)
        assert not np.array_equal(y8, want0)
        # the entry does nothing for nodes that do not carry accuracy_level 4 ...
        y0, _ = host.run_matmul_nbits(N, K, bits, bs, c.A, c.B, c.scales, c.zero_points, bias=c.bias, accuracy_level=0)
        assert np.array_equal(y0, y)
        # ... and nothing for configurations without an int8 route (8-bit weights)
        c8 = make_case(M, N, K, 8, bs, np.float16, has_zp=True, seed=22)
        y88, _ = host.run_matmul_nbits(N, K, 8, bs, c8.A, c8.B, c8.scales, c8.zero_points, accuracy_level=4)
        check_against_oracle(oracle, c8, y88)
    y_after, _ = host.run_matmul_nbits(N, K, bits, bs, c.A, c.B, c.scales, c.zero_points, bias=c.bias, accuracy_level=4)
    assert np.array_equal(y_after, y)


def test_per_call_scratch_comes_from_the_sessions_allocator(oracle):
    """Compute takes its workspace through KernelContext_GetScratchBuffer and hands it back through the allocator of
    KernelContext_GetAllocator (onnxruntime_c_api.h:5269, :4929); when the host declines -- an error status, a NULL
    buffer, a buffer the kernels cannot use -- the stream-ordered pool serves the call: same bits either way."""
    # M = 100, K = 320 (not a whole number of the streaming kernel's chunks): a staged copy of A, hence a workspace
    c = make_case(100, 320, 320, 4, 32, np.float16, has_zp=True, has_bias=True, seed=21)
    y0, _ = _run(c, repeat=3)
    st = host.last_run_stats()
    assert st["scratch_requests"] == 3 and st["scratch_served"] == 3 and st["scratch_bytes_max"] > 0, st
    assert st["scratch_freed"] == 3 and st["allocator_requests"] == st["allocators_released"] == 3, st
    check_against_oracle(oracle, c, y0)
    for mode in (1, 2, 3):
        with host.scratch_mode(mode):
            y, _ = _run(c, repeat=2)
        st = host.last_run_stats()
        assert st["scratch_requests"] == 2 and st["allocator_requests"] == st["allocators_released"] == 2, (mode, st)
        assert st["scratch_served"] == (2 if mode == 3 else 0), (mode, st)
        assert np.array_equal(y.view(np.uint8), y0.view(np.uint8)), mode
    # the unpacked route packs into scratch as well
    y_unpacked, trace = _run(c, constant=("B",), repeat=2)
    st = host.last_run_stats()
    assert "prepacked= " in trace and st["scratch_served"] == 2 and st["scratch_freed"] == 2, (trace, st)
    assert np.array_equal(y_unpacked.view(np.uint8), y0.view(np.uint8))
    # a decode call needs no workspace: no request at all
    d = make_case(1, 512, 1024, 4, 128, np.float16, seed=22)
    _run(d)
    assert host.last_run_stats()["scratch_requests"] == 0


def test_timing_mode_reports_one_compute_call():
    c = make_case(1, 1024, 1024, 4, 128, np.float16, seed=23)
    host.time_next_run(5, 50)
    _, trace = _run(c)
    st = host.last_run_stats()
    assert st["timed_computes"] == 50 and "ep_allocs_while_timed=0" in trace, (st, trace)  # the arena serves the outputs
    assert 0 < st["host_us_per_compute"] <= st["wall_us_per_compute"] < 1e4, st
    assert st["device_us_per_compute"] > 0, st
