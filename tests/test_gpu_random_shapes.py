"""Seeded random sweep over shapes, alignments and operator variants: every case goes through the C ABI and is held
to the oracle with the usual gates.  The point is breadth: ragged N and K, odd row pitches, misaligned activations,
every kernel family and both fused operators, drawn independently of the hand-picked cases elsewhere."""
import numpy as np
import pytest
import torch

from gpu_util import FP16_GATE, FP32_GATE, check_against_oracle, dev, tdtype
from onnxruntime_amd.matmul_nbits import MatMulNBits, MatMulNBitsMlp, MatMulNBitsQkv
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu

M_CHOICES = [1, 2, 3, 5, 8, 15, 16, 17, 31, 33, 64, 100, 129, 257]


def _draw(rng):
    bits = int(rng.choice([2, 4, 8]))
    bs = int(rng.choice([16, 32, 64, 128, 256]))
    dtype = np.float16 if rng.random() < 0.7 else np.float32
    M = int(rng.choice(M_CHOICES))
    N = int(rng.integers(1, 700))
    K = int(rng.integers(1, 1500)) if rng.random() < 0.5 else int(rng.choice([64, 128, 256, 512, 1024, 2048, 2112, 3072, 4096, 4224, 6144]))
    return M, N, K, bits, bs, dtype


def _strided_activation(rng, A):
    """A copy of A on the device with a random row pitch and a random element offset (alignment of the base)."""
    M, K = A.shape
    pitch = K + int(rng.choice([0, 0, 1, 3, 8, 24]))
    offset = int(rng.choice([0, 0, 1, 4, 8]))
    buf = torch.zeros(offset + M * pitch + 8, dtype=tdtype(A.dtype), device="cuda")
    view = buf[offset:offset + M * pitch].view(M, pitch)[:, :K]
    view.copy_(dev(A))
    return view


@pytest.mark.parametrize("seed", range(160))
def test_random_matmul_nbits(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    M, N, K, bits, bs, dtype = _draw(rng)
    zp, bias = bool(rng.random() < 0.5), bool(rng.random() < 0.5)
    c = make_case(M, N, K, bits, bs, dtype, has_zp=zp, has_bias=bias, seed=seed)
    op = MatMulNBits(K, N, bits, bs, dtype=tdtype(dtype), has_zero_points=zp, has_bias=bias)
    a = _strided_activation(rng, c.A)
    if rng.random() < 0.75:
        assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
        y = op.Compute(a, bias=dev(c.bias))
    else:
        y = op.Compute(a, dev(c.B), dev(c.scales), dev(c.zero_points), dev(c.bias))
    torch.cuda.synchronize()
    check_against_oracle(oracle, c, y.cpu().numpy())


@pytest.mark.parametrize("seed", range(96))
def test_random_fused_projections(oracle, seed):
    rng = np.random.default_rng(5000 + seed)
    M, N, K, bits, bs, dtype = _draw(rng)
    N = max(N // 2, 1)
    prologue = rng.choice(["none", "simplified", "skip"])
    gamma = rng.uniform(0.5, 1.5, K).astype(dtype) if prologue != "none" else None
    skip_rows = M if rng.random() < 0.7 else 1
    skip = rng.standard_normal((skip_rows, K)).astype(dtype) if prologue == "skip" else None
    mats = [make_case(M, n, K, bits, bs, dtype, has_bias=bool(rng.random() < 0.5), seed=seed * 7 + i)
            for i, n in enumerate((N, N, max(N // 3, 1)))]
    A = mats[0].A
    a = _strided_activation(rng, A)
    norm = None if prologue == "none" else (skip, gamma, 1e-5)
    act = A if norm is None else oracle.C.simplified_layer_norm(A, skip, gamma, 1e-5)
    want_sum = prologue == "skip" and rng.random() < 0.5

    def gate(got, c, n):
        y64, bound = oracle.C.matmul_f64(act, c.B, c.scales, None, c.bias, n, K, bits, bs, nthreads=8)
        err = np.abs(got.astype(np.float64) - y64)
        if dtype == np.float32:
            # the device normalises with a tree sum: its activation differs from the oracle's in the last bits
            assert float(np.max(err / (bound + 1e-30))) <= FP32_GATE * (1 if norm is None else 2)
        else:
            # one fp16 ulp of difference in a few normalised activations is inside the gate
            assert float(np.linalg.norm(err) / max(np.linalg.norm(y64), 1e-30)) <= FP16_GATE

    if seed % 2 == 0:
        g, u = mats[0], mats[1]
        op = MatMulNBitsMlp(K, N, bits, bs, epsilon=1e-5, dtype=tdtype(dtype))
        assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), dev(u.bias))
        out = op.Compute(a, skip=dev(skip), norm_scale=dev(gamma), want_skip_sum=want_sum)
        torch.cuda.synchronize()
        y = (out[0] if want_sum else out).cpu().numpy()
        g64, gb = oracle.C.matmul_f64(act, g.B, g.scales, None, g.bias, N, K, bits, bs, nthreads=8)
        u64, ub = oracle.C.matmul_f64(act, u.B, u.scales, None, u.bias, N, K, bits, bs, nthreads=8)
        sig = 1.0 / (1.0 + np.exp(-g64))
        ref = g64 * sig * u64
        err = np.abs(y.astype(np.float64) - ref)
        bound = 1.1 * np.abs(u64) * gb + np.abs(g64 * sig) * ub
        if dtype == np.float32:
            assert float(np.max(err / (bound + 1e-30))) <= FP32_GATE * (1 if norm is None else 2)
        else:
            assert np.all(err <= 1.5e-3 * bound + 2.0 ** -10 * np.abs(ref) + 1e-7)
    else:
        q, k, v = mats
        Nkv = v.N
        kk = make_case(M, Nkv, K, bits, bs, dtype, has_bias=k.bias is not None, seed=seed * 7 + 5)
        op = MatMulNBitsQkv(K, N, Nkv, bits, bs, epsilon=1e-5, dtype=tdtype(dtype))
        assert op.PrePack(dev(q.B), dev(q.scales), dev(q.bias), dev(kk.B), dev(kk.scales), dev(kk.bias), dev(v.B),
                          dev(v.scales), dev(v.bias))
        out = op.Compute(a, skip=dev(skip), norm_scale=dev(gamma), want_skip_sum=want_sum)
        torch.cuda.synchronize()
        for got, c, n in zip(out[:3], (q, kk, v), (N, Nkv, Nkv)):
            gate(got.cpu().numpy(), c, n)
    if want_sum:
        sm = out[-1].cpu().numpy()
        assert np.array_equal(sm, (A.astype(np.float32) + np.resize(skip.astype(np.float32), A.shape)).astype(dtype))


@pytest.mark.parametrize("seed", range(40))
def test_random_wide_matrices(oracle, seed):
    """Wide fp16 matrices with more than sixteen rows: the widths at which the streaming kernel shares the activations
    through LDS, at which the tile GEMM runs 128- and 256-row tiles or cuts tiles along K, and the ragged widths
    between them.  A random sample of rows against the oracle (rows are independent)."""
    rng = np.random.default_rng(9000 + seed)
    bits = int(rng.choice([4, 4, 8, 2]))
    bs = int(rng.choice([32, 64, 128]))
    M = int(rng.choice([17, 31, 33, 64, 65, 100, 129, 257, 600]))
    N = int(rng.integers(4500, 30000))
    if rng.random() < 0.4:
        N = (N // 128) * 128
    K = int(rng.choice([1024, 1152, 1408, 2048, 2080, 4096]))
    zp, bias = bool(rng.random() < 0.5), bool(rng.random() < 0.5)
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=bias, seed=seed)
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=zp, has_bias=bias)
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    a = _strided_activation(rng, c.A) if rng.random() < 0.5 else dev(c.A)
    y = op.Compute(a, bias=dev(c.bias))
    torch.cuda.synchronize()
    rows = np.sort(rng.choice(M, size=min(M, 24), replace=False))
    check_against_oracle(oracle, c, y.cpu().numpy()[rows], A=c.A[rows])
