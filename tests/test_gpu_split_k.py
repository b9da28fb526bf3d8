"""The tile GEMM with tiles cut along K across workgroups (few tiles of a tall problem, workspace given): the same
results as without the cut up to fp32 summation order, exact where one side of every sum is zero, the same from run to
run, and right against the oracle.  Counterpart of the reference's work partitioning, which cuts M and N only
(onnxruntime/core/mlas/lib/qnbitgemm.cpp:1600-1809)."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import FP16_GATE, dev
from onnxruntime_amd import _lib
from onnxruntime_amd.matmul_nbits import MatMulNBits, MatMulNBitsMlp
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _gemm(case, op, a, bias, with_workspace):
    lib = _lib.load()
    M = a.shape[0]
    has_zp = int(case.zero_points is not None)
    need = lib.MnbGemmWorkspaceSize(M, case.N, case.K, case.bits, case.block_size, has_zp, _lib.DTYPE_FLOAT16)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda") if with_workspace else None
    y = torch.full((M, case.N), float("nan"), dtype=torch.float16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.MnbGemm(M, case.N, case.K, case.bits, case.block_size, has_zp, _lib.DTYPE_FLOAT16, _ptr(a), case.K,
                           _ptr(op.packed), _ptr(bias), _ptr(y), case.N, _ptr(ws), need if with_workspace else 0, stream))
    torch.cuda.synchronize()
    return y, need


# M, N, K, bits, block size: two and four parts, 128- and 256-row tiles, ragged M / N, 8-bit weights
SHAPES = [(768, 4096, 4096, 8, 64), (1000, 4000, 8192, 4, 32), (512, 8192, 8192, 4, 64), (1024, 4096, 14336, 4, 128),
          (1024, 4096, 8192, 8, 64), (1000, 4090, 14336, 8, 32), (512, 4096, 14336, 8, 64)]


@pytest.mark.parametrize("M,N,K,bits,bs", SHAPES)
def test_split_matches_unsplit_and_oracle(oracle, M, N, K, bits, bs):
    lib = _lib.load()
    assert lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16).decode() == "mnb_gemm256_kernel"
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, has_bias=True, seed=M + K)
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=True, has_bias=True)
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    a, bias = dev(c.A), dev(c.bias)
    y_split, need = _gemm(c, op, a, bias, True)
    assert need > 0, "this shape is meant to take the split"
    y_plain, _ = _gemm(c, op, a, bias, False)
    assert not torch.isnan(y_split).any()
    rel = ((y_split.float() - y_plain.float()).norm() / y_plain.float().norm()).item()
    assert 0 < rel < 1e-4, rel                       # another summation order, nothing more
    y_again, _ = _gemm(c, op, a, bias, True)
    assert torch.equal(y_again.view(torch.int16), y_split.view(torch.int16))      # the same from run to run
    rows = np.unique(np.concatenate([np.linspace(0, M - 1, 6).astype(int), [255, 256, M - 1]]))
    y64, _ = oracle.C.matmul_f64(c.A[rows], c.B, c.scales, c.zero_points, c.bias, N, K, bits, bs, nthreads=8)
    got = y_split[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.float64)
    assert np.linalg.norm(got - y64) / np.linalg.norm(y64) <= FP16_GATE


@pytest.mark.parametrize("M,N,K,bits,bs", [(1024, 4096, 8192, 4, 128), (1024, 4096, 8192, 8, 64)])
def test_unit_vectors_come_back_exactly_through_the_split(oracle, M, N, K, bits, bs):
    """Row m of A is the unit vector e_k(m): every partial sum but one is zero, so Y[m] is column k(m) of the
    dequantised weights bit for bit, whichever part of the tile k(m) falls into."""
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, seed=3)
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=True)
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    ks = (np.arange(M) * 37 + 5) % K                                         # spread over all parts of K
    ks[:8] = [0, 1, K // 4 - 1, K // 4, K // 2 - 1, K // 2, K - 2, K - 1]    # and the borders of the parts
    A = np.zeros((M, K), np.float16)
    A[np.arange(M), ks] = 1
    c.A, c.bias = A, None
    y, need = _gemm(c, op, dev(A), None, True)
    assert need > 0
    w = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs)    # [N, K] fp16
    want = np.ascontiguousarray(w[:, ks].T)
    assert np.array_equal(y.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_fused_gate_up_through_the_split(oracle):
    """MatMulNBitsMlp on a shape whose packed matrix (gate and up interleaved) takes the split: the epilogue that
    applies silu(gate) * up sees complete sums."""
    M, N, K, bits, bs = 1024, 2048, 8192, 4, 32
    g = make_case(M, N, K, bits, bs, np.float16, has_bias=True, seed=5)
    u = make_case(M, N, K, bits, bs, np.float16, has_bias=True, seed=6)
    op = MatMulNBitsMlp(K, N, bits, bs, dtype=torch.float16)
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), dev(u.bias))
    lib = _lib.load()
    assert lib.MnbGemmKernelName(M, 2 * N, K, bits, bs, _lib.DTYPE_FLOAT16).decode() == "mnb_gemm256_kernel"
    assert lib.MnbGemmWorkspaceSize(M, 2 * N, K, bits, bs, 0, _lib.DTYPE_FLOAT16) > 0
    y = op.Compute(dev(g.A)).cpu().numpy().astype(np.float64)
    rows = np.array([0, 1, 255, 256, 511, 1000, 1023])
    want = oracle.C.mlp(g.A[rows], (g.B, g.scales, g.bias), (u.B, u.scales, u.bias), N, K, bits, bs).astype(np.float64)
    assert np.linalg.norm(y[rows] - want) / np.linalg.norm(want) <= FP16_GATE
    assert np.isfinite(y).all()


def _tile_plan(M, N, K, bits, bs):
    lib = _lib.load()
    r, c, p = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _lib.check(lib.MnbGemmTilePlan(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, ctypes.byref(r), ctypes.byref(c),
                                   ctypes.byref(p)))
    return r.value, c.value, p.value


def test_the_shapes_above_are_cut_along_k():
    for (M, N, K, bits, bs) in SHAPES:
        rows, cols, parts = _tile_plan(M, N, K, bits, bs)
        assert cols == 256 and parts > 1, (M, N, K, bits, bs, rows, cols, parts)


# problems whose 256-column tiles would leave half of the compute units idle: 128 x 128 tiles of four wavefronts
NARROW = [(1024, 4096, 4096, 4, 128), (512, 6144, 4096, 4, 32), (1000, 4000, 4096, 8, 64), (1024, 4096, 4096, 8, 16),
          (250, 14300, 4096, 4, 64)]


@pytest.mark.parametrize("M,N,K,bits,bs", NARROW)
def test_narrow_tiles_against_the_oracle_and_unit_vectors(oracle, M, N, K, bits, bs):
    assert _tile_plan(M, N, K, bits, bs) == (128, 128, 1)
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, has_bias=True, seed=M + N)
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=True, has_bias=True)
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    y, need = _gemm(c, op, dev(c.A), dev(c.bias), True)
    assert need == 0 and not torch.isnan(y).any()
    rows = np.unique(np.concatenate([np.linspace(0, M - 1, 7).astype(int), [127, 128, M - 1]]))
    y64, _ = oracle.C.matmul_f64(c.A[rows], c.B, c.scales, c.zero_points, c.bias, N, K, bits, bs, nthreads=8)
    got = y[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.float64)
    assert np.linalg.norm(got - y64) / np.linalg.norm(y64) <= FP16_GATE
    # unit-vector rows: column k(m) of the dequantised weights, bit for bit
    ks = (np.arange(M) * 37 + 5) % K
    A = np.zeros((M, K), np.float16)
    A[np.arange(M), ks] = 1
    y1, _ = _gemm(c, op, dev(A), None, True)
    w = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs)
    assert np.array_equal(y1.cpu().numpy().view(np.uint16), np.ascontiguousarray(w[:, ks].T).view(np.uint16))


def test_a_wait_that_gives_up_poisons_its_tile_and_is_reported(oracle):
    """The bounded cross-workgroup wait, exercised from the host's choice of arguments: a test build of the library
    (tests/hooks) leaves the lower parts of odd-numbered tiles uncomputed, so their flags stay zero, and bounds the
    wait at a few polls.  The finalising parts of those tiles give up: every kernel ends normally, exactly the
    odd-numbered tiles hold NaN, the even ones the product's own bits, and MnbGemmWorkspaceStatus reports it."""
    from pathlib import Path
    hooks_path = Path(__file__).resolve().parent / "hooks" / "libmnb_test_hooks.so"
    assert hooks_path.exists(), "tests/hooks/libmnb_test_hooks.so is missing: python -m tests.hooks.build"
    lib = _lib.load()
    hooked = ctypes.CDLL(str(hooks_path))
    for name in ("MnbGemm", "MnbGemmWorkspaceSize", "MnbGemmWorkspaceStatus", "MnbGemmTilePlan"):
        getattr(hooked, name).restype, getattr(hooked, name).argtypes = _lib.SIGNATURES[name]
    hooked.MnbTestSetSplitHooks.restype = None
    hooked.MnbTestSetSplitHooks.argtypes = [ctypes.c_int, ctypes.c_int]
    M, N, K, bits, bs = 1024, 4096, 8192, 4, 128
    tr, tc, parts = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    hooked.MnbGemmTilePlan(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, ctypes.byref(tr), ctypes.byref(tc), ctypes.byref(parts))
    assert parts.value > 1, "the case is meant to be cut along K"
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, has_bias=True, seed=7)
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=True, has_bias=True)
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    a, bias = dev(c.A), dev(c.bias)
    need = hooked.MnbGemmWorkspaceSize(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16)
    assert need == lib.MnbGemmWorkspaceSize(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16) > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gave_up = ctypes.c_int(-1)

    def run(l):
        y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        _lib.check(l.MnbGemm(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, _ptr(a), K, _ptr(op.packed), _ptr(bias), _ptr(y),
                             N, _ptr(ws), need, stream))
        torch.cuda.synchronize()
        _lib.check(l.MnbGemmWorkspaceStatus(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, _ptr(ws), need, stream,
                                            ctypes.byref(gave_up)))
        return y

    y_good = run(lib)
    assert gave_up.value == 0 and not torch.isnan(y_good).any()
    hooked.MnbTestSetSplitHooks(0, 0)                       # the hook build with its hooks off is the product
    assert torch.equal(run(hooked).view(torch.int16), y_good.view(torch.int16)) and gave_up.value == 0
    hooked.MnbTestSetSplitHooks(64, 1)                      # 64 polls, odd tiles lose their lower parts
    try:
        y_bad = run(hooked)
    finally:
        hooked.MnbTestSetSplitHooks(0, 0)
    assert gave_up.value == 1
    tiles_n = -(-N // tc.value)
    nan = torch.isnan(y_bad)
    for t in range((-(-M // tr.value)) * tiles_n):
        r0, c0 = (t // tiles_n) * tr.value, (t % tiles_n) * tc.value
        blk = (slice(r0, min(r0 + tr.value, M)), slice(c0, min(c0 + tc.value, N)))
        if t & 1:
            assert bool(nan[blk].all()), t
        else:
            assert not bool(nan[blk].any()) and torch.equal(y_bad[blk].view(torch.int16), y_good[blk].view(torch.int16)), t
    # the next healthy launch clears the report
    assert not torch.isnan(run(lib)).any() and gave_up.value == 0
