"""Drivers for calibration libraries: see the package docstring."""
from __future__ import annotations

import ctypes
import os
import sys
import time

import numpy as np
import torch

from onnxruntime_amd import _lib
from onnxruntime_amd.matmul_nbits import MatMulNBits
from onnxruntime_amd.synthetic import make_case

ENV_KEYS = ("MNB_GEMM256_PLAN", "MNB_GEMM256_WAVES", "MNB_GEMM256_WAVE_ROWS", "MNB_GEMM32", "MNB_GEMV16_NW",
            "MNB_MID_DIRECT", "MNB_MID_MAX_M", "MNB_MID_PLAN", "MNB_MID_SHARED", "MNB_NATIVE_ROUTE", "MNB_ROWS16_M",
            "MNB_ROWS16_NW", "MNB_ROWS16_T", "MNB_SKINNY_A4", "MNB_SKINNY_ALDS_FROM", "MNB_SKINNY_MODE", "MNB_SKINNY_NW",
            "MNB_SKINNY_PLAN", "MNB_SKINNY_T4LDS", "MNB_SKINNY_WIDE_EXACT")


def load(path: str):
    product = _lib.load()
    if path == "product":
        return product
    lib = ctypes.CDLL(path)
    for name in ("MnbGemm", "MnbGemmWorkspaceSize", "MnbGemmKernelName"):
        getattr(lib, name).restype = getattr(product, name).restype
        getattr(lib, name).argtypes = getattr(product, name).argtypes
    return lib


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _dev(x):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class Problem:
    """One problem; `copies` > 1 keeps that many copies of the packed matrix and successive calls walk through them
    (weights then stream from HBM instead of waiting in the Infinity Cache)."""

    def __init__(self, M, N, K, bits, bs, zp=True, bias=True, copies=1):
        c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=bias, seed=1)
        op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=zp, has_bias=bias)
        assert op.PrePack(_dev(c.B), _dev(c.scales), _dev(c.zero_points))
        self.dims, self.zp = (M, N, K, bits, bs), int(zp)
        self.a, self.bias = _dev(c.A), _dev(c.bias)
        self.packed = [op.packed] + [op.packed.clone() for _ in range(copies - 1)]

    def caller(self, lib):
        M, N, K, bits, bs = self.dims
        need = lib.MnbGemmWorkspaceSize(M, N, K, bits, bs, self.zp, _lib.DTYPE_FLOAT16)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
        y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        turn = [0]

        def call():
            packed = self.packed[turn[0] % len(self.packed)]
            turn[0] += 1
            return lib.MnbGemm(M, N, K, bits, bs, self.zp, _lib.DTYPE_FLOAT16, _ptr(self.a), K, _ptr(packed),
                               _ptr(self.bias), _ptr(y), N, _ptr(ws) if need else None, need, _stream())
        return call, y


def set_env(variant: dict):
    for k in ENV_KEYS:
        os.environ.pop(k, None)
    os.environ.update(variant)


def one(argv):
    lib = load(argv[0])
    M, N, K, bits, bs, zp = map(int, argv[1:7])
    launches = int(argv[argv.index("--launches") + 1]) if "--launches" in argv else 30
    copies = int(argv[argv.index("--copies") + 1]) if "--copies" in argv else 1   # > 1: weights stream from HBM
    call, _ = Problem(M, N, K, bits, bs, bool(zp), bias=False, copies=copies).caller(lib)
    print("kernel:", lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16).decode(), flush=True)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.05:   # the matrix-core clock settles
        assert call() == 0
        torch.cuda.synchronize()
    for _ in range(launches):
        assert call() == 0
    torch.cuda.synchronize()


def ab(argv):
    libs = [(p, load(p)) for p in argv[0].split(";")]
    envs = [dict(kv.split("=", 1) for kv in v.split("+") if kv) for v in argv[1].split(";")]
    shapes = [tuple(map(int, s.split(","))) for s in argv[2].split(";")]   # M,N,K,bits,block[,zero points[,copies]]
    variants = [(f"{p.split('/')[-1]} {e or ''}".strip(), lib, e) for p, lib in libs for e in envs]
    for shape in shapes:
        M, N, K, bits, bs = shape[:5]
        zp = bool(shape[5]) if len(shape) > 5 else True
        copies = shape[6] if len(shape) > 6 else 1
        prob = Problem(M, N, K, bits, bs, zp=zp, bias=zp, copies=copies)
        calls, outs = [], []
        for name, lib, env in variants:
            set_env(env)
            call, y = prob.caller(lib)
            print("run", name, (M, N, K, bits, bs), flush=True)   # (names the case should the launch fault)
            assert call() == 0
            torch.cuda.synchronize()
            calls.append(call)
            outs.append(y)
        same = [bool(torch.equal(outs[0], y)) for y in outs[1:]]
        best = [[] for _ in variants]
        for _ in range(4):
            for i, (name, lib, env) in enumerate(variants):
                set_env(env)
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < 0.03:
                    calls[i]()
                    torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for _ in range(max(20, copies)):
                        assert calls[i]() == 0
                g.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                g.replay()
                g.replay()
                e1.record()
                torch.cuda.synchronize()
                best[i].append(e0.elapsed_time(e1) / (2 * max(20, copies)) * 1e3)
        print(f"M={M} N={N} K={K} b{bits} bs{bs} zp={int(zp)} copies={copies}: " + "  ".join(
            f"[{variants[i][0]}] {min(b):.1f} us" for i, b in enumerate(best)) + f"  bit-identical to the first: {same}",
            flush=True)


def stamps(argv):
    """Anatomy of a direct decode launch from a library built with -DMNB_STAMPS: M N K BITS BLOCK ZP [COPIES].
    A HIP graph of COPIES launches over as many copies of the packed matrix is replayed; the readings are those of
    its last launch (100 MHz counter: 10 ns steps), printed relative to the first wavefront's entry."""
    lib = load(argv[0])
    M, N, K, bits, bs, zp = map(int, argv[1:7])
    # the readings live in the translation unit that holds the kernels of the weight format
    unit = {4: "w4zp" if zp else "w4", 8: "w8", 2: "w2"}[bits]
    read_stamps = getattr(lib, "MnbCalibrationReadStamps_" + unit)
    read_stamps.restype = ctypes.c_int
    read_stamps.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    copies = int(argv[7]) if len(argv) > 7 else 32
    call, _ = Problem(M, N, K, bits, bs, bool(zp), bias=False, copies=copies).caller(lib)
    print("kernel:", lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16).decode(), flush=True)
    assert call() == 0
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(copies):
            assert call() == 0
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    print(f"{e0.elapsed_time(e1) / copies * 1e3:.2f} us per launch with the readings compiled in", flush=True)
    points, waves, groups = 8, 16, 4096
    buf = np.zeros(groups * waves * points, dtype=np.uint64)
    assert read_stamps(buf.ctypes.data_as(ctypes.c_void_p), buf.size) == 0
    t = buf.reshape(groups, waves, points).astype(np.int64)
    live = t[:, :, 0] != 0
    t0 = t[:, :, 0][live].min()
    us = (t - t0) / 100.0
    names = ["entry", "loads issued", "first chunk computed", "last chunk computed", "partials in LDS",
             "past the barrier", "sums stored"]
    print(f"{int(live.sum())} wavefronts in {int(live.any(axis=1).sum())} workgroups; microseconds after the first entry")
    print(f"{'point':24s} {'min':>7s} {'p10':>7s} {'median':>7s} {'p90':>7s} {'max':>7s}")
    for i, name in enumerate(names):
        if not (t[:, :, i][live] != 0).all():   # (points 1-3 exist only where a wavefront's chunks are straight-line code)
            print(f"{name:24s} not recorded by this instantiation")
            continue
        v = us[:, :, i][live]
        print(f"{name:24s} {v.min():7.2f} {np.percentile(v, 10):7.2f} {np.median(v):7.2f} {np.percentile(v, 90):7.2f} "
              f"{v.max():7.2f}")
    ends = np.where(live, us[:, :, 6], -1).max(axis=1)
    ends = ends[live.any(axis=1)]
    print(f"workgroup ends: min {ends.min():.2f}  median {np.median(ends):.2f}  max {ends.max():.2f}")
    lag = (us[:, :, 5] - us[:, :, 4])[live]
    print(f"wait at the barrier per wavefront: median {np.median(lag):.2f}  p90 {np.percentile(lag, 90):.2f}  "
          f"max {lag.max():.2f}")


if __name__ == "__main__":
    {"one": one, "ab": ab, "stamps": stamps}[sys.argv[1]](sys.argv[2:])
