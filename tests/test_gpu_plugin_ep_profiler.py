"""OrtEp::CreateProfiler: the host test double drives the plugin's profiler the way ONNX Runtime's session profiling
does (onnxruntime/core/session/plugin_ep/ep_event_profiling.cc: StartProfiling with ORT's clock offset, StartEvent /
StopEvent around every node execution, EndProfiling) and reads back the KERNEL events the plugin reports."""
import numpy as np
import pytest

from ep_host import host
from onnxruntime_amd.synthetic import make_case

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not host.available(), reason="plugin EP or host shim not built")]

KERNEL = 2            # OrtProfilingEventCategory_KERNEL
OFFSET_US = 5000      # the double tells the plugin that ORT's profiling began 5 ms before StartProfiling


def test_one_kernel_event_per_node_execution():
    c = make_case(4, 512, 1024, 4, 32, np.float16, has_zp=True, has_bias=True, seed=1)
    with host.profiled() as prof:
        y, _ = host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales, c.zero_points, None, c.bias, repeat=3)
    assert len(prof.events) == 3
    stamps = []
    for i, e in enumerate(prof.events):
        assert e["category"] == KERNEL and e["name"] == "mnb_skinny_kernel"
        assert e["op_name"] == "MatMulNBits" and e["shape"] == "4 x 512 x 1024"
        assert int(e["ort_event_correlation_id"]) == 1700000000000000 + i   # the ORT event it ran under
        assert 0 <= e["duration_us"] < 10000
        assert e["timestamp_us"] >= OFFSET_US                               # on ORT's timeline, not the device's
        stamps.append(e["timestamp_us"])
    assert stamps == sorted(stamps) and stamps[-1] < OFFSET_US + 5_000_000
    # profiling changes nothing in the result
    y2, _ = host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales, c.zero_points, None, c.bias)
    assert np.array_equal(y.view(np.uint16), y2.view(np.uint16))


def test_kernel_names_follow_the_route():
    c = make_case(300, 512, 1024, 4, 32, np.float16, seed=2)
    with host.profiled() as prof:
        host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales)
    assert [e["name"] for e in prof.events] == ["mnb_mid_kernel"]
    c = make_case(2, 64, 128, 4, 32, np.float32, seed=3)
    with host.profiled() as prof:
        host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales, constant=("B",))        # unpacked route
    assert [e["name"] for e in prof.events] == ["pack + MatMulNBits"]
    c = make_case(2, 64, 128, 4, 32, np.float16, has_bias=True, seed=4)
    with host.profiled() as prof:
        host.run_matmul_nbits_add(c.N, c.K, 4, 32, c.A, c.B, c.scales, c.bias)            # compiled pair
    assert [e["op_name"] for e in prof.events] == ["MatMulNBits+Add"]


def test_unprofiled_runs_report_nothing():
    c = make_case(1, 64, 128, 4, 32, np.float16, seed=5)
    with host.profiled() as prof:
        pass
    assert prof.events == []
    host.run_matmul_nbits(c.N, c.K, 4, 32, c.A, c.B, c.scales)
