#!/usr/bin/env python3
"""Benchmark of the MI355X MatMulNBits hot path.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--sweep]

Prints ONE JSON line on stdout.  Headline workload (BASELINE.json configs[1]): the decode GEMV
M=1, K=4096, N=14336, int4, block_size 128, symmetric, fp16.  One *step* is one decode pass of that projection
through the 32 decoder layers of Llama-3-8B: 32 launches, each on its own packed weight matrix (32 x 30 MB is
four times the 256 MB Infinity Cache, so every launch streams its weights from HBM).  `value` is algorithmic GB/s
of the whole step, inputs resident in HBM.  The same line carries the prefill GEMM (configs[3], M=2048) as
`prefill`, the roofline of the dominant kernel and the CPU baseline (the oracle, timed on this host).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# HBM bytes per launch are NOT measured by this program: they come from separate rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of this same command, scaled by what the same counters read for a plain copy of known size
# (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000), and are copied here from the summary named in TRAFFIC_SOURCE (KiB per
# dispatch as printed there).  Every `traffic` value in the output carries `traffic_source` beside it.
TRAFFIC_SOURCE = "profiles/hbm_traffic_skinny_c2_gemm256_c4_quantize.md (rocprofv3 --pmc; a constant, not this run)"
PROFILED_TRAFFIC_BYTES = {"c2_decode": int((14858.5 * 2.0 + 28.0) * 1024), "c4_prefill": int((109777.3 * 2.0 + 57344.0) * 1024),
                          "quantize": int((57412.5 * 2.0 + 36364.4) * 1024), "mlp_decode": int((29675.0 * 2.0 + 28.0) * 1024)}
# The reference's own MLAS kernel on the headline shape, timed by the survey on an 8-vCPU Sapphire-Rapids-class host
# (standalone MLAS build, SQNBIT_CompFp32, N sliced over 8 threads): quoted beside the port so that the port's
# figure is not read as the reference's.
REFERENCE_MLAS_US_SURVEY = {"us_per_call": 1353.0, "threads": 8, "algorithmic_GBs": 23.1,
                            "source": "the baseline survey of the reference (its container, not this host)"}
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published (no sparsity)
LAYERS = 32


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


class Problem:
    """One MatMulNBits shape with `copies` independently packed weight matrices, run through the C ABI."""

    def __init__(self, case, copies: int, torch, lib_mod):
        from onnxruntime_amd.matmul_nbits import MatMulNBits
        self.torch, self.case = torch, case
        self.lib = lib_mod.load()
        self.lib_mod = lib_mod
        tdt = torch.float16 if case.dtype == np.float16 else torch.float32
        self.dt = lib_mod.DTYPE_FLOAT16 if case.dtype == np.float16 else lib_mod.DTYPE_FLOAT
        dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()
        self.has_zp = int(case.zero_points is not None)
        b, s, z = dev(case.B), dev(case.scales), dev(case.zero_points)
        self.packed = []
        t0 = time.perf_counter()
        for i in range(copies):
            op = MatMulNBits(case.K, case.N, case.bits, case.block_size, dtype=tdt,
                             has_zero_points=bool(self.has_zp), has_bias=case.bias is not None)
            # distinct contents per copy (rolled columns) so no two copies alias in any cache
            bi = torch.roll(b, shifts=i, dims=0) if i else b
            assert op.PrePack(bi, s, z)
            self.packed.append(op.packed)
        torch.cuda.synchronize()
        self.prepack_ms = (time.perf_counter() - t0) * 1e3 / copies   # host view: allocation, roll and launch included

        from onnxruntime_amd.matmul_nbits import _stream_ptr
        stream = _stream_ptr(b.device)

        def repack():  # device view: the pack kernels alone, into the buffers that exist by now
            for pk in self.packed:
                lib_mod.check(self.lib.MnbPackQuantBData(case.N, case.K, case.bits, case.block_size, self.dt, _ptr(b),
                                                         _ptr(s), _ptr(z), _ptr(pk), stream))
        self.prepack_device_us = time_steps(torch, repack, 3, 1) / copies * 1e3
        for i, pk in enumerate(self.packed):  # restore the distinct contents
            bi = torch.roll(b, shifts=i, dims=0) if i else b
            lib_mod.check(self.lib.MnbPackQuantBData(case.N, case.K, case.bits, case.block_size, self.dt, _ptr(bi),
                                                     _ptr(s), _ptr(z), _ptr(pk), stream))
        torch.cuda.synchronize()
        self.a = dev(case.A.reshape(-1, case.K))
        self.bias = dev(case.bias)
        self.M = self.a.shape[0]
        self.y = [torch.empty(self.M, case.N, dtype=tdt, device="cuda") for _ in range(copies)]
        wsz = self.lib.MnbGemmWorkspaceSize(self.M, case.N, case.K, case.bits, case.block_size, self.has_zp, self.dt)
        self.wsz = wsz
        self.ws = torch.zeros(max(wsz, 256), dtype=torch.uint8, device="cuda")
        self.kernel = self.lib.MnbGemmKernelName(self.M, case.N, case.K, case.bits, case.block_size, self.dt).decode()

    def launch(self, i: int):
        c = self.case
        stream = ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)
        rc = self.lib.MnbGemm(self.M, c.N, c.K, c.bits, c.block_size, self.has_zp, self.dt, _ptr(self.a), c.K,
                              _ptr(self.packed[i]), _ptr(self.bias), _ptr(self.y[i]), c.N, _ptr(self.ws), self.wsz,
                              stream)
        self.lib_mod.check(rc)

    def step(self):
        for i in range(len(self.packed)):
            self.launch(i)


def time_steps(torch, run_step, steps: int, warmup: int, warm_ms: float = 0.0) -> float:
    """Milliseconds per step, HIP events on the launch stream, barrier + synchronize on both sides.

    warm_ms > 0 keeps the warm-up going until that much wall time has passed: from idle the matrix-core clock needs
    about 15 ms of load to settle (measured on the M=2048 GEMM: 305, 241, 230, 225, 225 ... us per launch over
    consecutive groups of 20 launches), so a compute-bound leg that is timed after a handful of launches reports the
    ramp, not the kernel.  The decode GEMV shows no such ramp (8.34-8.42 us per launch from the first replay on)."""
    for _ in range(warmup):
        run_step()
    torch.cuda.synchronize()
    if warm_ms > 0:
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < warm_ms:
            run_step()
            torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        run_step()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def load_probe():
    """libmnb_probe.so: the read-bandwidth and matrix-core-rate probes (onnxruntime_amd/csrc/mnb_probe.h)."""
    path = ROOT / "onnxruntime_amd" / "libmnb_probe.so"
    if not path.exists():
        raise RuntimeError(f"{path} is missing: build it with `python -m onnxruntime_amd.build`")
    lib = ctypes.CDLL(str(path))
    lib.MnbProbeReadBandwidth.restype = ctypes.c_int
    lib.MnbProbeReadBandwidth.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeReadBandwidthResident.restype = ctypes.c_int
    lib.MnbProbeReadBandwidthResident.argtypes = lib.MnbProbeReadBandwidth.argtypes
    lib.MnbProbeMfmaRate.restype = ctypes.c_int
    lib.MnbProbeMfmaRate.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeMfmaRateOperands.restype = ctypes.c_int
    lib.MnbProbeMfmaRateOperands.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeIssueOverlap.restype = ctypes.c_int
    lib.MnbProbeIssueOverlap.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                         ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeDequantMfma16.restype = ctypes.c_int
    lib.MnbProbeDequantMfma16.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeShaderClockStart.restype = ctypes.c_int
    lib.MnbProbeShaderClockStart.argtypes = [ctypes.c_double]
    lib.MnbProbeShaderClockFinish.restype = ctypes.c_int
    lib.MnbProbeShaderClockFinish.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    lib.MnbProbeRelease.restype = None
    lib.MnbProbeRelease.argtypes = []
    return lib


def graph_of(torch, run_step):
    """Captures one step into a HIP graph (the launches are ~5 us each: Python cannot issue them that fast)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_step()  # warm every code path on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        run_step()
    return g


def graph_of_chains(torch, launch, n_launches: int, chains: int):
    """The same launches as independent chains inside one HIP graph (launch i on chain i % chains): what a runtime
    with several streams does with GEMVs that do not depend on each other."""
    side = torch.cuda.Stream()
    subs = [torch.cuda.Stream() for _ in range(chains - 1)]
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        streams = [side] + subs
        for s in subs:
            s.wait_stream(side)
        for i in range(n_launches):
            with torch.cuda.stream(streams[i % chains]):
                launch(i)
        for s in subs:
            side.wait_stream(s)
    return g


def cpu_baseline(case, budget_s: float, threads: int):
    """The oracle (a port of the reference arithmetic) timed on this host for a bounded number of calls."""
    from oracle import oracle
    oracle.build()
    run = lambda: oracle.C.matmul(case.A, case.B, case.scales, case.zero_points, case.bias, case.N, case.K,
                                  case.bits, case.block_size, nthreads=threads)
    run()
    t0 = time.perf_counter()
    n = 0
    while True:
        run()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 200:
            break
    return el / n, n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the M=2048 GEMM")
    ap.add_argument("--no-ceilings", action="store_true",
                    help="skip the read-only / MFMA-only probe kernels that report what the machine sustains")
    ap.add_argument("--no-quantize", action="store_true", help="skip the blockwise quantiser (producer of the format)")
    ap.add_argument("--no-fused", action="store_true", help="skip the fused gate/up projection (MatMulNBitsMlp)")
    ap.add_argument("--no-sizes", action="store_true", help="skip the decode kernel on the larger gate+up matrices")
    ap.add_argument("--no-bf16", action="store_true", help="skip the bfloat16 rows")
    ap.add_argument("--no-int8", action="store_true",
                    help="skip the int8-activation route (accuracy_level 4) beside the full-accuracy one")
    ap.add_argument("--no-plugin", action="store_true", help="skip the leg through the plugin-EP boundary")
    ap.add_argument("--sweep", action="store_true", help="also time the other configurations (printed to stderr)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (a kernel of known traffic, for scaling the "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters); nothing else changes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the op shards along N without communication; nothing "
              "here uses a second device). Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch
    from onnxruntime_amd import _lib, synthetic
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    _lib.load()

    if args.calibrate_copy:
        src = torch.full((256 << 20,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    # ---- decode GEMV (headline) ------------------------------------------------------------------------------
    c2 = synthetic.config_c2(seed=0)
    p2 = Problem(c2, LAYERS, torch, _lib)
    g2 = graph_of(torch, p2.step)
    ms_step = time_steps(torch, g2.replay, args.steps, args.warmup)
    bytes_per_launch = c2.algorithmic_bytes()
    us_per_launch = ms_step * 1e3 / LAYERS
    gbs = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    # same launches with the weights resident in the Infinity Cache (one matrix re-used), for reference only
    g2hot = graph_of(torch, lambda: [p2.launch(0) for _ in range(LAYERS)])
    ms_hot = time_steps(torch, g2hot.replay, args.steps, args.warmup)

    # the same chain four times over in one graph (128 launches): what a step loses to the hand-over from one graph
    # replay to the next, which is not part of any launch (reported beside the headline)
    g2long = graph_of(torch, lambda: [p2.launch(i % LAYERS) for i in range(4 * LAYERS)])
    ms_long = time_steps(torch, g2long.replay, max(2, args.steps // 4), 1)
    del g2long

    # and as two independent chains of 16: the head and tail of one launch overlap with its neighbour's streaming.
    # Reported beside the headline, never as the headline: `value` is the serialised chain.
    g2two = graph_of_chains(torch, p2.launch, LAYERS, 2)
    ms_two = time_steps(torch, g2two.replay, args.steps, args.warmup)
    del g2two

    out = {
        "metric": "int4 MatMulNBits decode GEMV (M=1, K=4096, N=14336) algorithmic HBM GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: MatMulNBits M=1 K=4096 N=14336 bits=4 block_size=128 symmetric fp16; "
                        f"one step = {LAYERS} launches on {LAYERS} distinct packed weight matrices (HIP graph)",
            "launches_per_step": LAYERS,
            "algorithmic_bytes_per_launch": bytes_per_launch,
            "kernel": p2.kernel,
            "prepack_ms_per_matrix": round(p2.prepack_ms, 3),
            "prepack_device_us_per_matrix": round(p2.prepack_device_us, 1),
            "us_per_launch_weights_in_infinity_cache": round(ms_hot * 1e3 / LAYERS, 3),
            "us_per_launch_in_graphs_of_128_launches": round(ms_long * 1e3 / (4 * LAYERS), 3),
            "us_per_launch_as_two_independent_chains": round(ms_two * 1e3 / LAYERS, 3),
            "GBs_as_two_independent_chains": round(bytes_per_launch / (ms_two * 1e-3 / LAYERS) / 1e9, 1),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": PROFILED_TRAFFIC_BYTES["c2_decode"], "traffic_source": TRAFFIC_SOURCE,
            "kernel": p2.kernel,
            "us_per_launch": round(us_per_launch, 3),
        },
    }
    del g2, g2hot, p2
    torch.cuda.empty_cache()

    # ---- what this GPU sustains with the plainest kernels (context for the fractions above and below) ----------
    if not args.no_ceilings:
        probe = load_probe()
        v = ctypes.c_double(0.0)
        sweep_rows = []
        for threads in (256, 512, 1024):
            for inflight in (4, 8, 16, 32):
                for batches in (1, 2, 4):
                    rc = probe.MnbProbeReadBandwidth(bytes_per_launch, LAYERS, threads, inflight, batches,
                                                     ctypes.byref(v))
                    assert rc == 0, f"read probe failed ({rc})"
                    sweep_rows.append((v.value, threads, inflight, batches))
        best = max(sweep_rows)
        # the same bytes waiting in the Infinity Cache (every launch re-reads one buffer): the eight best configurations
        resident_rows = []
        for _, threads, inflight, batches in sorted(sweep_rows, reverse=True)[:8]:
            assert probe.MnbProbeReadBandwidthResident(bytes_per_launch, LAYERS, threads, inflight, batches,
                                                       ctypes.byref(v)) == 0
            resident_rows.append((v.value, threads, inflight, batches))
        probe.MnbProbeRelease()
        # 1 GiB per launch, where launch ramp and tail no longer count: the same 36 configurations
        big_rows = []
        for threads in (256, 512, 1024):
            for inflight in (4, 8, 16, 32):
                for batches in (1, 2, 4):
                    assert probe.MnbProbeReadBandwidth(1 << 30, 2, threads, inflight, batches, ctypes.byref(v)) == 0
                    big_rows.append((v.value, threads, inflight, batches))
        big_best = max(big_rows)
        read_big = big_best[0]
        probe.MnbProbeRelease()
        out["roofline"]["measured_ceiling"] = {
            "read_only_kernel_same_bytes_per_launch_GBs": round(best[0], 1),
            "read_only_kernel_best_config": {"threads": best[1], "loads_in_flight": best[2], "batches": best[3]},
            "read_only_kernel_sweep_GBs_min_median_max": [round(x, 1) for x in (
                min(sweep_rows)[0], sorted(sweep_rows)[len(sweep_rows) // 2][0], best[0])],
            "read_only_kernel_configs_swept": len(sweep_rows),
            "read_only_kernel_same_bytes_in_infinity_cache_GBs": round(max(resident_rows)[0], 1),
            "read_only_kernel_1GiB_per_launch_GBs": round(read_big, 1),
            "read_only_kernel_1GiB_best_config": {"threads": big_best[1], "loads_in_flight": big_best[2],
                                                  "batches": big_best[3]},
            "read_only_kernel_1GiB_sweep_GBs_min_median_max": [round(x, 1) for x in (
                min(big_rows)[0], sorted(big_rows)[len(big_rows) // 2][0], big_best[0])],
            "read_only_kernel_1GiB_frac_of_hbm_peak": round(read_big / HBM_PEAK_GBS, 4),
            "frac_of_read_only_kernel": round(gbs / best[0], 4) if best[0] > 0 else None,
        }
        if args.sweep:
            for r in sorted(sweep_rows, reverse=True):
                print(f"read probe: {r[0]:8.1f} GB/s threads={r[1]} loads_in_flight={r[2]} batches={r[3]}",
                      file=sys.stderr)
            for r in sorted(big_rows, reverse=True):
                print(f"read probe 1 GiB: {r[0]:8.1f} GB/s threads={r[1]} loads_in_flight={r[2]} batches={r[3]}",
                      file=sys.stderr)
            for r in sorted(resident_rows, reverse=True):
                print(f"read probe, data in the Infinity Cache: {r[0]:8.1f} GB/s threads={r[1]} loads_in_flight={r[2]} "
                      f"batches={r[3]}", file=sys.stderr)

    # ---- prefill GEMM ----------------------------------------------------------------------------------------
    if not args.no_prefill:
        c4 = synthetic.config_c4(seed=0)
        p4 = Problem(c4, 2, torch, _lib)
        k4 = max(50, args.steps)  # 100+ launches, about 25 ms
        ms4 = time_steps(torch, p4.step, k4, max(1, args.warmup // 2), warm_ms=30.0) / 2
        tflops = c4.flops() / (ms4 * 1e-3) / 1e12
        out["prefill"] = {
            "workload": "BASELINE configs[3]: M=2048 K=4096 N=14336 bits=4 block_size=32 zero_points bias fp16",
            "value": round(tflops, 1),
            "unit": "TFLOP/s",
            "ms_per_launch": round(ms4, 4),
            "kernel": p4.kernel,
            "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_FP16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tflops / MFMA_FP16_PEAK_TFLOPS, 4),
                         "traffic": PROFILED_TRAFFIC_BYTES["c4_prefill"], "traffic_source": TRAFFIC_SOURCE},
        }
        if not args.no_ceilings:
            probe = load_probe()
            v = ctypes.c_double(0.0)
            assert probe.MnbProbeMfmaRate(0, ctypes.byref(v)) == 0
            mfma_const = v.value
            assert probe.MnbProbeMfmaRate(1, ctypes.byref(v)) == 0
            mfma_rand = v.value
            # the same loop on the operand classes of this kernel: A bell-shaped activations (class 3), B what the
            # kernel feeds (dequantised weights with a scale per column, class 4), what it would feed if the scale were
            # applied to the sums instead (integers, 5; the decode kernel's raw halves, 6), and zeros
            by_class = {}
            for name, (ca, cb) in {"activations_x_dequantised_weights": (3, 4), "activations_x_integer_weights": (3, 5),
                                   "activations_x_raw_magic_halves": (3, 6), "dequantised_weights_x_activations": (4, 3),
                                   "zero_x_dequantised_weights": (2, 4)}.items():
                assert probe.MnbProbeMfmaRateOperands(ca, cb, ctypes.byref(v)) == 0
                by_class[name] = round(v.value, 1)
            # the same kernel, same launches, on activations that are all zero: the instruction stream is identical,
            # only the switching activity of the operands (and with it the clock the power limit allows) differs
            a_saved = p4.a.clone()
            p4.a.zero_()
            ms4_zero = time_steps(torch, p4.step, k4, max(1, args.warmup // 2), warm_ms=30.0) / 2
            tflops_zero = c4.flops() / (ms4_zero * 1e-3) / 1e12

            def clock_during(run_step, steps):
                """GHz of the shader clock while `steps` steps run: a single wavefront on a stream of its own compares
                the shader clock's cycle counter with the constant 100 MHz counter for 12 ms (chip already warm)."""
                ghz, sampled = ctypes.c_double(0.0), ctypes.c_double(0.0)
                assert probe.MnbProbeShaderClockStart(12.0) == 0
                for _ in range(steps):
                    run_step()
                torch.cuda.synchronize()
                assert probe.MnbProbeShaderClockFinish(ctypes.byref(ghz), ctypes.byref(sampled)) == 0
                return round(ghz.value, 3)

            p4.a.zero_()
            clock_zero = clock_during(p4.step, k4)
            p4.a.copy_(a_saved)
            clock_random = clock_during(p4.step, k4)
            del a_saved
            # What the kernel's instruction mix costs in issue slots, with nothing else in the way: two wavefronts per
            # SIMD, per matrix instruction two independent vector instructions (the dequantisation) and one 1 KB LDS
            # read (its A operand), issued a whole loop iteration ahead of its use; constant operands.
            slot = {}
            for name, (valu, lds) in {"mfma_only": (0, 0), "mfma_2_vector": (2, 0), "mfma_lds_operand": (0, 2),
                                      "mfma_2_vector_lds_operand": (2, 2)}.items():
                assert probe.MnbProbeIssueOverlap(valu, 1, 2, lds, ctypes.byref(v)) == 0
                slot[name] = v.value
            out["prefill"]["roofline"]["measured_ceiling"] = {
                "issue_probe_ns_per_matrix_instruction_per_wavefront_two_per_simd": {k: round(x, 2)
                                                                                    for k, x in slot.items()},
                "issue_probe_instruction_mix_of_this_kernel_vs_mfma_only": round(
                    slot["mfma_only"] / slot["mfma_2_vector_lds_operand"], 4),
                "mfma_only_loop_constant_operands_TFLOPs": round(mfma_const, 1),
                "mfma_only_loop_random_operands_TFLOPs": round(mfma_rand, 1),
                "frac_of_mfma_only_random": round(tflops / mfma_rand, 4) if mfma_rand > 0 else None,
                "mfma_only_loop_TFLOPs_by_operand_class": by_class,
                "frac_of_mfma_only_on_this_kernels_operands": round(
                    tflops / by_class["activations_x_dequantised_weights"], 4),
                "same_kernel_zero_activations_TFLOPs": round(tflops_zero, 1),
                "same_kernel_zero_activations_ms_per_launch": round(ms4_zero, 4),
                "shader_clock_ghz_during_these_launches": clock_random,
                "shader_clock_ghz_during_the_zero_activation_launches": clock_zero,
            }
        del p4
        torch.cuda.empty_cache()

    # ---- blockwise quantiser: fp16 [K, N] weights -> the operands of configs[1] --------------------------------
    if not args.no_quantize:
        from onnxruntime_amd.matmul_nbits import quantize_blockwise
        Kq, Nq, copies = c2.K, c2.N, 4
        gen = torch.Generator(device="cuda").manual_seed(0)
        ws = [torch.randn(Kq, Nq, generator=gen, device="cuda", dtype=torch.float16) * 0.05 for _ in range(copies)]

        def qstep():
            for w in ws:  # 4 x 117 MB of distinct sources: beyond the Infinity Cache
                quantize_blockwise(w, c2.bits, c2.block_size, symmetric=True)

        msq = time_steps(torch, qstep, max(4, args.steps // 5), 2, warm_ms=20.0) / copies
        kbq = Kq // c2.block_size
        qbytes = Kq * Nq * 2 + Nq * kbq * (c2.block_size * c2.bits // 8) + Nq * kbq * 2
        out["quantize"] = {
            "workload": "MlasQuantizeBlockwise semantics: fp16 [4096, 14336] -> int4 block_size=128 symmetric",
            "value": round(qbytes / (msq * 1e-3) / 1e9, 1),
            "unit": "GB/s",
            "ms_per_launch": round(msq, 4),
            "kernel": "mnb_quantize_kernel",
            "roofline": {"bound": "hbm", "achieved": round(qbytes / (msq * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(qbytes / (msq * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": PROFILED_TRAFFIC_BYTES["quantize"], "traffic_source": TRAFFIC_SOURCE},
        }
        # ---- and back: MlasDequantizeBlockwise semantics on the quantiser's output (4 distinct operand sets) --------
        from onnxruntime_amd.matmul_nbits import dequantize_blockwise
        qs = [quantize_blockwise(w, c2.bits, c2.block_size, symmetric=True) for w in ws]
        del ws
        torch.cuda.empty_cache()

        def dstep():
            for (b, sc, z) in qs:  # the allocator hands every call the 117 MB block the previous result just freed
                dequantize_blockwise(b, sc, z, Nq, Kq, c2.bits, c2.block_size)

        msd = time_steps(torch, dstep, max(4, args.steps // 5), 2, warm_ms=20.0) / copies
        out["dequantize"] = {
            "workload": "MlasDequantizeBlockwise semantics: int4 block_size=128 symmetric [14336, 32, 64] -> fp16 [14336, 4096]",
            "value": round(qbytes / (msd * 1e-3) / 1e9, 1),
            "unit": "GB/s",
            "ms_per_launch": round(msd, 4),
            "kernel": "mnb_dequant_canonical_vec_kernel",
            "roofline": {"bound": "hbm", "achieved": round(qbytes / (msd * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(qbytes / (msd * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None},
        }
        del qs
        torch.cuda.empty_cache()

    # ---- MatMulNBitsMlp: the gate and up projections of configs[1]'s shape in one launch ------------------------
    if not args.no_fused:
        from onnxruntime_amd.matmul_nbits import MatMulNBitsMlp
        copies = 6   # 6 x 60 MB of distinct weights: beyond the Infinity Cache
        dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
        up = synthetic.make_case(1, c2.N, c2.K, c2.bits, c2.block_size, np.float16, seed=1)
        gb, gs, ub, us = dev(c2.B), dev(c2.scales), dev(up.B), dev(up.scales)
        ops = []
        for i in range(copies):
            op = MatMulNBitsMlp(c2.K, c2.N, c2.bits, c2.block_size)
            assert op.PrePack(torch.roll(gb, i, 0), gs, None, torch.roll(ub, i, 0), us, None)
            ops.append(op)
        a1 = dev(c2.A.reshape(1, c2.K))
        skip1 = dev(up.A.reshape(1, c2.K))
        gamma = torch.ones(c2.K, dtype=torch.float16, device="cuda")
        fbytes = 2 * (c2.N * c2.k_blocks * (c2.block_size * c2.bits // 8) + c2.N * c2.k_blocks * 2) + \
            c2.K * 2 + c2.N * 2
        legs = {}
        for name, kw in (("plain", {}), ("skip_norm", dict(skip=skip1, norm_scale=gamma, want_skip_sum=True))):
            def fstep():
                for op in ops:
                    op.Compute(a1, **kw)
            g = graph_of(torch, fstep)
            msf = time_steps(torch, g.replay, max(4, args.steps // 2), 2) / copies
            legs[name] = msf
        gbs_f = fbytes / (legs["plain"] * 1e-3) / 1e9
        out["mlp_decode"] = {
            "workload": "MatMulNBitsMlp M=1 K=4096 N=14336 bits=4 block_size=128 fp16: silu(A gate^T) * (A up^T), "
                        "gate and up packed as one matrix",
            "value": round(gbs_f, 1),
            "unit": "GB/s",
            "ms_per_launch": round(legs["plain"], 5),
            "ms_per_launch_with_skip_layer_norm_prologue": round(legs["skip_norm"], 5),
            "kernel": "mnb_skinny_kernel",
            "roofline": {"bound": "hbm", "achieved": round(gbs_f, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs_f / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC_BYTES["mlp_decode"], "traffic_source": TRAFFIC_SOURCE},
        }
        del ops
        torch.cuda.empty_cache()

    # ---- the same decode kernel on larger matrices: how the fixed part of a launch weighs against its size ----------
    if not args.no_sizes:
        rows = []
        # (the 2-bit rows stream the copy of the weights in their own width: half the bytes of the 4-bit rows)
        # (the down rows run single-tile slabs, where the activations reach the operand registers through LDS: one load per
        # chunk of up to four rows)
        for label, bits, bs, shape, M5 in (("gate+up int4 bs128 zp", 4, 128, "gate_up", 1),
                                           ("gate+up int8 bs64 zp", 8, 64, "gate_up", 1),
                                           ("gate+up int2 bs128 zp", 2, 128, "gate_up", 1),
                                           ("configs[1] shape as int2 bs128 zp", 2, 128, None, 1),
                                           ("down int4 bs128 zp", 4, 128, "down", 1),
                                           ("down int4 bs128 zp", 4, 128, "down", 4),
                                           ("down int2 bs128 zp", 2, 128, "down", 1)):
            K5, N5 = synthetic.C5_SHAPES[shape] if shape else (c2.K, c2.N)
            case = synthetic.make_case(M5, N5, K5, bits, bs, np.float16, has_zp=True, seed=0)
            copies = 8 if shape == "gate_up" else 32  # distinct weights beyond the 256 MB Infinity Cache
            p5 = Problem(case, copies, torch, _lib)
            per_graph = max(copies, 32)  # (a graph replay hands over to the next in several microseconds: 32 launches share it)
            g5 = graph_of(torch, lambda: [p5.launch(i % copies) for i in range(per_graph)])
            us5 = time_steps(torch, g5.replay, max(4, args.steps // 2), 2) / per_graph * 1e3
            gb5 = case.algorithmic_bytes() / (us5 * 1e-6) / 1e9
            rows.append({"workload": f"{'BASELINE configs[4] ' if shape else ''}M={M5} K={K5} N={N5} {label} fp16", "kernel": p5.kernel,
                         "algorithmic_bytes_per_launch": case.algorithmic_bytes(), "us_per_launch": round(us5, 3),
                         "value": round(gb5, 1), "unit": "GB/s", "frac_of_hbm_peak": round(gb5 / HBM_PEAK_GBS, 4)})
            del g5, p5
            torch.cuda.empty_cache()
        out["decode_sizes"] = rows

    # ---- accuracy_level 4: int8 activations against the full-accuracy route on the same problems ----------------
    if not args.no_int8:
        rows = []
        lib = _lib.load()
        # (blocks of 32 are declined by MnbGemmInt8: 80 vector instructions behind every matrix instruction)
        for label, M8, N8, K8, bs8 in (("configs[3] shape with 64-wide blocks", 2048, 14336, 4096, 64),
                                       ("configs[4] gate+up M=1024, block 128", 1024, 28672, 4096, 128),
                                       ("the same with 256-wide blocks", 1024, 28672, 4096, 256)):
            case = synthetic.make_case(M8, N8, K8, 4, bs8, np.float16, has_zp=True, seed=0)
            p8 = Problem(case, 1, torch, _lib)
            ms_full = time_steps(torch, p8.step, 20, 1, warm_ms=30.0)
            need = lib.MnbGemmInt8WorkspaceSize(M8, N8, K8, 4, bs8, 1, _lib.DTYPE_FLOAT16)
            ws8 = torch.empty(need, dtype=torch.uint8, device="cuda")
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

            def int8_step():
                _lib.check(lib.MnbGemmInt8(M8, N8, K8, 4, bs8, 1, _lib.DTYPE_FLOAT16, _ptr(p8.a), K8, _ptr(p8.packed[0]),
                                           None, _ptr(p8.y[0]), N8, _ptr(ws8), need, stream))
            ms_int8 = time_steps(torch, int8_step, 20, 1, warm_ms=30.0)
            rows.append({"workload": f"M={M8} K={K8} N={N8} int4 zero_points fp16, {label}",
                         "full_accuracy_kernel": p8.kernel, "full_accuracy_ms": round(ms_full, 4),
                         "int8_activations_ms": round(ms_int8, 4),
                         "int8_over_full": round(ms_int8 / ms_full, 3)})
            del p8, ws8
            torch.cuda.empty_cache()
        out["accuracy_level_4"] = rows

    # ---- bfloat16 models: configs[1]'s and configs[3]'s shapes through the variant entry points --------------------
    if not args.no_bf16:
        from onnxruntime_amd.matmul_nbits import MatMulNBits
        lib = _lib.load()
        rows = []
        for label, case, copies in (("configs[1] shape (M=1, int4 bs128 symmetric)", c2, 16),
                                    ("configs[3] shape (M=2048, int4 bs32 zero_points bias)",
                                     synthetic.config_c4(seed=0), 2)):
            dev = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()
            b, z = dev(case.B), dev(case.zero_points)
            sc = dev(case.scales.astype(np.float32)).to(torch.bfloat16)
            a = dev(case.A.reshape(-1, case.K).astype(np.float32)).to(torch.bfloat16)
            bias = None if case.bias is None else dev(case.bias.astype(np.float32)).to(torch.bfloat16)
            ops = []
            for i in range(copies):
                op = MatMulNBits(case.K, case.N, case.bits, case.block_size, dtype=torch.bfloat16,
                                 has_zero_points=z is not None, has_bias=bias is not None)
                assert op.PrePack(torch.roll(b, i, 0) if i else b, sc, z, None)
                ops.append(op)
            Mb = a.shape[0]
            ys = [torch.empty(Mb, case.N, dtype=torch.bfloat16, device="cuda") for _ in ops]

            def bstep():
                for op, y in zip(ops, ys):
                    op.Compute(a, bias=bias, out=y)
            bstep()
            if Mb <= 16:
                g = graph_of(torch, bstep)
                ms_b = time_steps(torch, g.replay, max(4, args.steps // 2), 2) / copies
            else:
                ms_b = time_steps(torch, bstep, 50, 2, warm_ms=30.0) / copies
            # algorithmic bytes: the packed matrix carries fp32 scales (and zero points) for bfloat16 models
            kb = case.k_blocks
            abytes = case.N * kb * (case.block_size * case.bits // 8) + case.N * kb * (8 if z is not None else 4) + \
                Mb * case.K * 2 + Mb * case.N * 2 + (case.N * 2 if bias is not None else 0)
            rows.append({"workload": f"bfloat16, {label}",
                         "kernel": lib.MnbVariantGemmKernelName(ctypes.byref(ops[0].plan), Mb).decode(),
                         "us_per_launch": round(ms_b * 1e3, 3),
                         "GBs": round(abytes / (ms_b * 1e-3) / 1e9, 1),
                         "TFLOPs": round(2.0 * Mb * case.N * case.K / (ms_b * 1e-3) / 1e12, 1)})
            del ops, ys
            torch.cuda.empty_cache()
        out["bfloat16"] = rows

    # ---- the same decode call through the plugin-EP boundary ---------------------------------------------------
    # Everything above enters the library at MnbGemm (ctypes).  ONNX Runtime enters at OrtKernelImpl::Compute
    # (plugin_ep/ep_kernel_registration.cc:78-80): input and shape queries through the C API, output allocation from
    # the session's arena, the workspace request, then the same MnbGemm.  The host test double plays ONNX Runtime's
    # part (tests/ep_host): CreateEpFactories -> ... -> PrePackWeight -> Compute, called back to back on one
    # device-resident activation, one packed matrix (which therefore stays in the Infinity Cache: compare with
    # us_per_launch_weights_in_infinity_cache, not with the headline).
    if not args.no_plugin:
        sys.path.insert(0, str(ROOT / "tests"))
        try:
            from ep_host import host
            have_host = host.available()
        except Exception:  # noqa: BLE001 - the leg is optional
            have_host = False
        if have_host:
            rows = {}
            for label, case in (("decode M=1 (configs[1])", c2), ("M=64 K=4100 N=6144 int4 bs128 zp (staged activations: a workspace per call)",
                                                                   synthetic.make_case(64, 6144, 4100, 4, 128, np.float16, has_zp=True, seed=3))):  # (K not a whole number of chunks)
                host.time_next_run(50, 400)
                _, trace = host.run_matmul_nbits(case.N, case.K, case.bits, case.block_size, case.A, case.B,
                                                 case.scales, case.zero_points, None, case.bias)
                st = host.last_run_stats()
                # the eager ctypes call on the same problem, for the difference
                op = Problem(case, 1, torch, _lib)
                for _ in range(50):
                    op.launch(0)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                t0 = time.perf_counter()
                e0.record()
                for _ in range(400):
                    op.launch(0)
                e1.record()
                t1 = time.perf_counter()
                torch.cuda.synchronize()
                rows[label] = {
                    "kernel": op.kernel,
                    "compute_calls_timed": int(st["timed_computes"]),
                    "host_us_per_Compute": round(st["host_us_per_compute"], 2),
                    "device_us_per_Compute": round(st["device_us_per_compute"], 2),
                    "wall_us_per_Compute": round(st["wall_us_per_compute"], 2),
                    "scratch_requests_served_by_session": int(st["scratch_served"]),
                    "provider_allocations_while_timed": 0 if "ep_allocs_while_timed=0" in trace else None,
                    "ctypes_MnbGemm_host_us_per_call": round((t1 - t0) / 400 * 1e6, 2),
                    "ctypes_MnbGemm_device_us_per_call": round(e0.elapsed_time(e1) / 400 * 1e3, 2),
                }
                del op
            out["plugin_boundary"] = {
                "path": "tests/ep_host host double: CreateEpFactories -> CreateEp -> kernel registry -> PrePackWeight -> "
                        "OrtKernelImpl::Compute, back to back on one stream, outputs and workspace from the "
                        "session's arena (KernelContext_GetOutput / KernelContext_GetScratchBuffer)",
                "rows": rows,
            }
        else:
            out["plugin_boundary"] = None

    # ---- the other configurations (not part of the JSON contract) ---------------------------------------------
    if args.sweep:
        sweep(torch, _lib, synthetic)

    # ---- CPU baseline ----------------------------------------------------------------------------------------
    if not args.no_cpu:
        threads = max(1, min(16, os.cpu_count() or 1))
        sec, n = cpu_baseline(c2, args.cpu_seconds, threads)
        out["cpu_baseline"] = {
            "value": round(bytes_per_launch / sec / 1e9, 2),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"{n} calls of the same M=1 K=4096 N=14336 problem on the C oracle, N sliced over {threads} "
                      f"threads, {sec * 1e3:.2f} ms per call",
            "reference_mlas_us_survey": REFERENCE_MLAS_US_SURVEY,
        }
    print(json.dumps(out))
    return 0


def sweep(torch, _lib, synthetic):
    """Times BASELINE configs 1, 3 and 5 (one launch each, rotating weight copies); table on stderr."""
    from onnxruntime_amd.synthetic import make_case
    rows = []

    def copies_from_hbm(case):
        """Distinct packed matrices whose total lies beyond twice the 256 MB Infinity Cache: every launch streams from HBM."""
        return max(8, min(64, -(-600_000_000 // case.algorithmic_bytes())))

    def one(name, case, copies):
        copies = copies or copies_from_hbm(case)
        p = Problem(case, copies, torch, _lib)
        if p.M <= 64:
            per_graph = max(copies, 32)  # (as in the decode legs: the hand-over between graph replays is shared by 32 launches)
            g = graph_of(torch, lambda: [p.launch(i % copies) for i in range(per_graph)])
            ms = time_steps(torch, g.replay, 20, 3) / per_graph
        else:
            ms = time_steps(torch, p.step, 20, 1, warm_ms=30.0) / copies
        gb = case.algorithmic_bytes() / (ms * 1e-3) / 1e9
        tf = case.flops() / (ms * 1e-3) / 1e12
        rows.append((name, p.kernel, ms * 1e3, gb, tf))
        print(f"{name:44s} {p.kernel:26s} {ms * 1e3:10.2f} us {gb:9.1f} GB/s {tf:9.2f} TFLOP/s", file=sys.stderr)
        del p
        torch.cuda.empty_cache()

    # the streaming kernels' instruction mix on its own (two wavefronts per SIMD): per 32-bit word of 4-bit weights and
    # column tile, 13 vector instructions make the operand and 4 matrix instructions (64 rows) use it
    probe, v = load_probe(), ctypes.c_double(0.0)
    for mode, what in enumerate(("4 matrix instructions alone", "13 vector instructions alone",
                                 "operand made in front of its matrix instructions",
                                 "next operand made between the matrix instructions")):
        assert probe.MnbProbeDequantMfma16(mode, 2, ctypes.byref(v)) == 0
        print(f"streaming mix probe: {v.value:6.2f} ns per step of two wavefronts on a SIMD, {what}", file=sys.stderr)
    c1 = synthetic.config_c1()
    one("C1 fp32 M=1 4096x4096 bs32 zp", c1, copies_from_hbm(c1))
    for nm, (K, N) in synthetic.C3_SHAPES.items():
        for M in (1, 2, 4, 8, 16):
            case = make_case(M, N, K, 4, 64, np.float16, has_zp=True)
            one(f"C3 {nm} M={M} K={K} N={N} bs64 zp", case, copies_from_hbm(case))
    for bits, bs in ((4, 128), (8, 64)):
        for nm, (K, N) in synthetic.C5_SHAPES.items():
            for M in (1, 64, 256, 1024, 4096):
                copies = 0 if M <= 64 else 1  # (0: as many as stream from HBM, from the case itself)
                one(f"C5 {nm} M={M} K={K} N={N} b{bits} bs{bs} zp",
                    make_case(M, N, K, bits, bs, np.float16, has_zp=True), copies)
    return rows


if __name__ == "__main__":
    sys.exit(main())
