"""The C ABI under HIP graph capture (every kernel family, replayed with eager work in between) and the plugin EP
driven from several host threads at once."""
import threading

import numpy as np
import pytest
import torch

from ep_host import host
from gpu_util import check_against_oracle, dev, make_op
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K,bits,bs,dtype", [
    (1, 512, 1024, 4, 128, np.float16),     # matrix-core decode kernel
    (3, 300, 520, 8, 32, np.float32),       # fp32 GEMV
    (40, 384, 1024, 4, 32, np.float16),     # weight-streaming kernel (staging kernel + main kernel, workspace)
    (300, 512, 1024, 4, 64, np.float16),    # tile GEMM or streaming kernel, by the cost estimate
    (20, 100, 200, 4, 16, np.float32),      # generic kernel
    (1024, 4096, 4096, 8, 64, np.float16),  # tile GEMM with tiles cut along K (flag-clearing kernel + main kernel)
    (600, 1500, 512, 4, 128, np.float16),   # tile GEMM, ragged
    (24, 700, 1024, 4, 32, np.float32),     # fp32 rows through the fp32 matrix cores
    (1024, 4096, 4096, 4, 128, np.float16),  # tile GEMM on 128 x 128 tiles of four wavefronts
])
def test_gemm_replays_from_a_hip_graph(M, N, K, bits, bs, dtype):
    c = make_case(M, N, K, bits, bs, dtype, has_zp=True, has_bias=True, seed=M + N)
    op = make_op(c)
    bias = dev(c.bias)
    a1, a2 = dev(c.A), dev(c.A[::-1].copy())
    a = a1.clone()
    y = op.Compute(a, bias=bias)                      # eager: also sizes the workspace outside the capture
    want1 = y.clone()
    want2 = op.Compute(a2, bias=bias).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            op.Compute(a, bias=bias, out=y)
    for rep in range(4):                              # replays, with eager work and new inputs in between
        src, want = (a1, want1) if rep % 2 == 0 else (a2, want2)
        a.copy_(src)
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {rep}"
        _ = op.Compute(a2, bias=bias)                 # eager call of the same op between replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("kind,zp_kind,M,N,K", [
    ("bf16", "u8", 7, 520, 1024),          # decode kernel on bfloat16
    ("bf16", "none", 90, 700, 1000),       # streaming kernel (staging kernel + main kernel, workspace)
    ("bf16", "u8", 1024, 4096, 4096),      # tile GEMM
    ("f16", "typed", 40, 300, 512),        # fp16 with zero points in the activation type
])
def test_variant_gemm_replays_from_a_hip_graph(kind, zp_kind, M, N, K):
    from test_gpu_variants import make, to_dev, TORCH
    from onnxruntime_amd import MatMulNBits
    c = make(kind, N, K, 4, 32, zp_kind, "none", M, seed=M, bias=True)
    zp_dtype = torch.uint8 if zp_kind != "typed" else TORCH[kind]
    op = MatMulNBits(K, N, bits=4, block_size=32, dtype=TORCH[kind], has_zero_points=c["zp"] is not None,
                     has_bias=True, zero_points_dtype=zp_dtype)
    d = {k: to_dev(v) for k, v in c.items()}
    assert op.PrePack(d["B"], d["scales"], d["zp"], None)
    a1, a2 = d["A"], d["A"].flip(0).contiguous()
    a = a1.clone()
    y = op.Compute(a, bias=d["bias"])                 # eager: also sizes the workspace outside the capture
    want1 = y.clone()
    want2 = op.Compute(a2, bias=d["bias"]).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            op.Compute(a, bias=d["bias"], out=y)
    bits = torch.int16
    for rep in range(4):
        src, want = (a1, want1) if rep % 2 == 0 else (a2, want2)
        a.copy_(src)
        y.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(bits), want.view(bits)), f"replay {rep}"
        _ = op.Compute(a2, bias=d["bias"])
        torch.cuda.synchronize()


@pytest.mark.skipif(not host.available(), reason="plugin EP or host shim not built")
def test_plugin_sessions_on_concurrent_threads(oracle):
    cases = [make_case(M, 192, 256, bits, 32, dt, has_zp=True, has_bias=bool(M % 2), seed=M)
             for M, bits, dt in [(1, 4, np.float16), (5, 8, np.float32), (33, 4, np.float16), (2, 4, np.float32)]]
    results, errors = [None] * len(cases), []

    def work(i):
        try:
            c = cases[i]
            for _ in range(5):
                y, _ = host.run_matmul_nbits(c.N, c.K, c.bits, c.block_size, c.A, c.B, c.scales, c.zero_points,
                                             None, c.bias, repeat=2)
            results[i] = y
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for c, y in zip(cases, results):
        check_against_oracle(oracle, c, y)
