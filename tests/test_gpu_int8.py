"""accuracy_level 4 on the device (MnbGemmInt8, through the C ABI): the int8-activation route against the oracle's
restatement of the reference's scalar statement of it.  Every output is accumulated by one lane, block by block in k
order, with the oracle's operations and roundings, so the comparison is bit for bit (zeros of either sign compare
equal: a padded block adds +0 to a sum that may be -0)."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import dev
from onnxruntime_amd import _lib
from onnxruntime_amd.matmul_nbits import MatMulNBits, MnbError
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu


def _run(c, has_zp, has_bias, a=None):
    op = MatMulNBits(c.K, c.N, 4, c.block_size, accuracy_level=4, dtype=torch.float16, has_zero_points=has_zp,
                     has_bias=has_bias, int8_activations=True)
    assert op.int8_activations
    assert op.PrePack(dev(c.B), dev(c.scales), dev(c.zero_points))
    y = op.Compute(dev(c.A) if a is None else a, bias=dev(c.bias))
    torch.cuda.synchronize()
    return y.cpu().numpy()


SHAPES = [  # M, N, K, block size, zero points, bias
    (1, 128, 128, 64, False, False), (5, 200, 256, 64, True, True), (130, 257, 384, 64, True, True),
    (64, 512, 1024, 128, False, True), (257, 130, 512, 256, True, False), (33, 96, 200, 64, True, True),
    (200, 300, 4096, 128, True, True), (129, 64, 1000, 64, False, False), (16, 4096, 4096, 128, False, False),
]


@pytest.mark.parametrize("M,N,K,bs,has_zp,has_bias", SHAPES)
def test_bit_exact_against_the_oracle(oracle, M, N, K, bs, has_zp, has_bias):
    c = make_case(M, N, K, 4, bs, np.float16, has_zp=has_zp, has_bias=has_bias, seed=M + N + K)
    got = _run(c, has_zp, has_bias)
    want = oracle.C.matmul_int8(c.A, c.B, c.scales, c.zero_points, c.bias, N, K, bs, nthreads=8)
    assert got.shape == want.shape
    assert np.array_equal(got, want), (np.abs(got.astype(np.float64) - want.astype(np.float64)).max(),
                                       int((got != want).sum()))


def test_llama_projection_shape_rows_sampled(oracle):
    """BASELINE configs[4] gate+up at M = 1024 (int4, block 128, zero points): sampled rows bit for bit."""
    M, N, K, bs = 1024, 28672, 4096, 128
    c = make_case(M, N, K, 4, bs, np.float16, has_zp=True, seed=11)
    got = _run(c, True, False)
    rows = np.array([0, 1, 127, 128, 511, 1000, 1023])
    want = oracle.C.matmul_int8(c.A[rows], c.B, c.scales, c.zero_points, None, N, K, bs, nthreads=8)
    assert np.array_equal(got[rows], want)
    assert np.isfinite(got).all()


def test_strided_and_unaligned_activations(oracle):
    M, N, K, bs = 20, 160, 264, 64
    c = make_case(M, N, K, 4, bs, np.float16, has_zp=True, has_bias=True, seed=2)
    wide = torch.zeros(M, K + 3, dtype=torch.float16, device="cuda")
    wide[:, :K] = dev(c.A)
    got = _run(c, True, True, a=wide[:, :K])                     # row pitch K + 3: rows are not 16-byte aligned
    want = oracle.C.matmul_int8(c.A, c.B, c.scales, c.zero_points, c.bias, N, K, bs)
    assert np.array_equal(got, want)


def test_exact_ties_and_zero_rows(oracle):
    """Rows made of half-way values (in units of the block's scale) and an all-zero row."""
    M, N, K, bs = 4, 64, 128, 64
    c = make_case(M, N, K, 4, bs, np.float16, has_zp=True, seed=5)
    t = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 127.0] + [3.5] * 55)
    A = np.zeros((M, K), np.float16)
    A[0] = np.tile(t * 0.25, K // bs)
    A[1] = np.tile(-t * 2.0, K // bs)
    A[3] = c.A[3]
    c.A = A
    got = _run(c, True, False)
    want = oracle.C.matmul_int8(A, c.B, c.scales, c.zero_points, None, N, K, bs)
    assert np.array_equal(got, want)
    assert not got[2].any()


def test_differs_from_the_full_accuracy_route_within_the_rounding_bound(oracle):
    M, N, K, bs = 8, 256, 1024, 128
    c = make_case(M, N, K, 4, bs, np.float16, has_zp=True, seed=8)
    y8 = _run(c, True, False).astype(np.float64)
    y0, _ = oracle.C.matmul_f64(c.A, c.B, c.scales, c.zero_points, None, N, K, 4, bs)
    _, sa = oracle.C.quantize_a_int8(c.A, bs)
    w = np.abs(oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, 4, bs).astype(np.float64))
    bound = (sa.astype(np.float64) / 2) @ w.reshape(N, K // bs, bs).sum(axis=2).T
    err = np.abs(y8 - y0)
    assert (err <= bound * 1.001 + np.abs(y0) * 2.0 ** -10 + 1e-6).all()
    assert err.max() > 0


def test_unsupported_configurations_are_declined_not_approximated():
    lib = _lib.load()
    # (blocks of 32 included: 80 vector instructions behind every matrix instruction; declined, see the header)
    for bits, bs, dt in ((8, 64, _lib.DTYPE_FLOAT16), (4, 16, _lib.DTYPE_FLOAT16), (4, 64, _lib.DTYPE_FLOAT),
                         (2, 64, _lib.DTYPE_FLOAT16), (4, 32, _lib.DTYPE_FLOAT16)):
        assert lib.MnbGemmInt8WorkspaceSize(4, 64, 64, bits, bs, 0, dt) == 0
        x = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
        p = ctypes.c_void_p(x.data_ptr())
        rc = lib.MnbGemmInt8(4, 64, 64, bits, bs, 0, dt, p, 64, p, None, p, 64, p, x.numel(), None)
        assert rc == _lib.NOT_IMPLEMENTED
        assert "int8 activations are implemented for 4-bit weights" in lib.MnbGetLastErrorMessage().decode()
    # the host class falls back to the full-accuracy route for them
    op = MatMulNBits(64, 64, 8, 64, accuracy_level=4, dtype=torch.float16, int8_activations=True)
    c = make_case(4, 64, 64, 8, 64, np.float16, seed=1)
    assert op.PrePack(dev(c.B), dev(c.scales), None)
    assert op.Compute(dev(c.A)).shape == (4, 64)


def test_workspace_is_checked():
    lib = _lib.load()
    need = lib.MnbGemmInt8WorkspaceSize(4, 64, 64, 4, 64, 0, _lib.DTYPE_FLOAT16)
    assert need > 0
    x = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = ctypes.c_void_p(x.data_ptr())
    assert lib.MnbGemmInt8(4, 64, 64, 4, 64, 0, _lib.DTYPE_FLOAT16, p, 64, p, None, p, 64, p, need - 1, None) == _lib.INVALID_ARGUMENT
    assert "MnbGemmInt8WorkspaceSize" in lib.MnbGetLastErrorMessage().decode()
