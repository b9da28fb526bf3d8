"""2-bit weights (bits = 2: four elements per byte, zero points four per byte, default zero point 2;
onnxruntime/core/mlas/lib/q4_dq.cpp:318-333, 587-641).  The device library widens them to nibbles when it packs, so
every kernel family is exercised; results are held to the oracle like the other widths.  The reference's own 2-bit
tests (onnxruntime/test/contrib_ops/matmul_2bits_test.cc) draw random data and compute the expectation in the test,
so there are no stored vectors to replay: the oracle's 2-bit unpack is pinned in tests/test_oracle_matmul.py by the
exhaustive (q, zp) table and the independent numpy restatement."""
import numpy as np
import pytest
import torch

from ep_host import host
from gpu_util import check_against_oracle, dev, make_op, run_case, tdtype
from onnxruntime_amd.matmul_nbits import MatMulNBitsMlp, dequantize_blockwise, quantize_blockwise
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu


def _bits_view(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("zp", [False, True])
def test_dequant_bit_exact(oracle, dtype, bs, zp):
    for (N, K) in [(8, 64), (33, 93), (300, 260), (5, 1234)]:
        c = make_case(1, N, K, 2, bs, dtype, has_zp=zp, seed=N + K)
        want = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, 2, bs)
        got = dequantize_blockwise(dev(c.B), dev(c.scales), dev(c.zero_points), N, K, 2, bs).cpu().numpy()
        assert np.array_equal(_bits_view(got), _bits_view(want)), "canonical dequantise"
        got_p = make_op(c).dequantize_packed().cpu().numpy()
        assert np.array_equal(_bits_view(got_p), _bits_view(want)), "packed dequantise"


def test_exhaustive_q_zp():
    """All 4 x 4 (q, zp) pairs against integer arithmetic."""
    N, bs = 4, 16
    K = 4 * bs
    q = np.broadcast_to(np.arange(K)[None, :] % 4, (N, K))
    zpv = (np.arange(N)[:, None] + np.arange(4)[None, :]) % 4          # [N, k_blocks]
    B = np.zeros((N, 4, bs // 4), np.uint8)
    qq = q.reshape(N, 4, bs // 4, 4)
    for j in range(4):
        B |= (qq[..., j] << (2 * j)).astype(np.uint8)
    Z = np.zeros((N, 1), np.uint8)
    for kb in range(4):
        Z[:, 0] |= (zpv[:, kb] << (2 * kb)).astype(np.uint8)
    for dtype in (np.float16, np.float32):
        scales = np.ones((N, 4), dtype)
        got = dequantize_blockwise(dev(B), dev(scales), dev(Z), N, K, 2, bs).cpu().numpy().astype(np.int64)
        want = q.reshape(N, 4, bs) - zpv[:, :, None]
        assert np.array_equal(got.reshape(N, 4, bs), want)
        none = dequantize_blockwise(dev(B), dev(scales), None, N, K, 2, bs).cpu().numpy().astype(np.int64)
        assert np.array_equal(none.reshape(N, 4, bs), q.reshape(N, 4, bs) - 2)   # default zero point 2


CASES = [
    # M, N, K, bs, zp, bias: decode, ragged, streaming, tile GEMM
    (1, 512, 1024, 32, False, False), (1, 1000, 4096, 128, True, True), (7, 333, 200, 16, True, False),
    (16, 256, 2048, 64, False, True), (40, 520, 768, 32, True, True), (100, 72, 328, 64, False, False),
    (300, 520, 256, 128, True, True), (2048, 2048, 1024, 32, False, True),
]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("prepack", [True, False])
@pytest.mark.parametrize("M,N,K,bs,zp,bias", CASES)
def test_matmul_parity(oracle, dtype, prepack, M, N, K, bs, zp, bias):
    c = make_case(M, N, K, 2, bs, dtype, has_zp=zp, has_bias=bias, seed=M + N + K)
    check_against_oracle(oracle, c, run_case(c, prepack=prepack))


def test_through_the_plugin_and_fused(oracle):
    c = make_case(5, 320, 512, 2, 32, np.float16, has_zp=True, has_bias=True, seed=3)
    y, trace = host.run_matmul_nbits(c.N, c.K, 2, 32, c.A, c.B, c.scales, c.zero_points, None, c.bias)
    assert "claimed=1" in trace and "prepacked=1,2,3," in trace
    check_against_oracle(oracle, c, y)
    g = make_case(3, 200, 256, 2, 64, np.float16, has_bias=True, seed=4)
    u = make_case(3, 200, 256, 2, 64, np.float16, seed=5)
    op = MatMulNBitsMlp(256, 200, 2, 64)
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), None)
    y = op.Compute(dev(g.A)).cpu().numpy().astype(np.float64)
    want = oracle.C.mlp(g.A, (g.B, g.scales, g.bias), (u.B, u.scales, None), 200, 256, 2, 64).astype(np.float64)
    assert float(np.linalg.norm(y - want) / np.linalg.norm(want)) <= 5e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("bs", [16, 32, 128])
@pytest.mark.parametrize("symmetric", [True, False])
def test_quantiser_matches_the_oracle(oracle, dtype, bs, symmetric):
    K, N = 300, 70
    g = torch.Generator(device="cuda").manual_seed(bs)
    w = (torch.randn(K, N, generator=g, device="cuda") * 0.1).to(dtype)
    b, s, z = quantize_blockwise(w, 2, bs, symmetric)
    wb, ws, wz = oracle.C.quantize(w.cpu().numpy(), 2, bs, symmetric)
    assert np.array_equal(b.cpu().numpy(), wb)
    assert np.array_equal(_bits_view(s.cpu().numpy()), _bits_view(ws))
    if not symmetric:
        assert np.array_equal(z.cpu().numpy(), wz)


NATIVE = [
    # M, N, K, bs, zp, bias: decode shapes whose K is whole chunks of 256: the copy in the weights' own width
    (1, 512, 1024, 128, False, False), (1, 1000, 4096, 128, True, True), (2, 4096, 4096, 64, True, False),
    (4, 6144, 4096, 128, False, True), (1, 14336, 4096, 128, True, False), (3, 11008, 4096, 256, True, True),
    (5, 333, 256, 64, True, False), (8, 2048, 8192, 256, False, False), (9, 4100, 2048, 128, True, True),
    (16, 520, 4096, 64, False, True), (16, 4096, 14336, 128, True, False), (1, 28672, 4096, 256, True, False),
    (12, 14336, 512, 64, True, True), (7, 20480, 1024, 128, False, False),
    (1, 4096, 4096, 32, True, False), (6, 1000, 1024, 32, False, True),
]


@pytest.mark.parametrize("M,N,K,bs,zp,bias", NATIVE)
def test_decode_streams_the_native_copy(oracle, M, N, K, bs, zp, bias):
    """fp16 models, blocks of 32 and more, up to 16 rows, K a multiple of 256, aligned activations: the decode kernel
    reads the 2-bit copy of the weights (half the bytes).  Against the oracle; unit-vector rows return columns of W
    bit for bit; the nibble copy is not touched (it is overwritten first) while more than 16 rows still need it."""
    c = make_case(M, N, K, 2, bs, np.float16, has_zp=zp, has_bias=bias, seed=M + N + K)
    op = make_op(c)
    y = op.Compute(dev(c.A), bias=dev(c.bias))
    check_against_oracle(oracle, c, y.cpu().numpy())
    ks = np.random.default_rng(N).choice(K, size=M, replace=False)
    eye = np.zeros((M, K), np.float16)
    eye[np.arange(M), ks] = 1
    w = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, 2, bs)
    got = op.Compute(dev(eye)).cpu().numpy()   # (without the bias)
    assert np.array_equal(_bits_view(got), _bits_view(np.ascontiguousarray(w[:, ks].T)))
    # activations that are not 16-byte aligned take the nibble copy: the same result up to the order of the sums
    wide = torch.zeros(1 + M * (K + 3), dtype=torch.float16, device="cuda")[1:].view(M, K + 3)  # (base off by 2 bytes)
    wide[:, :K] = dev(c.A)
    y_nib = op.Compute(wide[:, :K], bias=dev(c.bias)).cpu().numpy()
    d = np.abs(y_nib.astype(np.float64) - y.cpu().numpy().astype(np.float64))
    assert d.max() <= 2e-3 * np.abs(y_nib).max() + 1e-3
    # which copy is read: garbage in the nibble section changes nothing for aligned decode calls ...
    n_pad, k_pad = -(-N // 256) * 256, -(-(-(-K // bs) * bs) // 128) * 128
    w_bytes = k_pad // 32 * n_pad * 16
    saved = op.packed[:w_bytes].clone()
    op.packed[:w_bytes] = 0x5A
    y_again = op.Compute(dev(c.A), bias=dev(c.bias))
    assert torch.equal(y_again, y)
    # ... and does for the calls that read it
    y_broken = op.Compute(wide[:, :K], bias=dev(c.bias)).cpu().numpy()
    assert not np.array_equal(y_broken, y_nib)
    op.packed[:w_bytes] = saved
    assert np.array_equal(op.Compute(wide[:, :K], bias=dev(c.bias)).cpu().numpy(), y_nib)


@pytest.mark.parametrize("M,N,K,bs", [(1, 1408, 1024, 128), (3, 200, 256, 64), (8, 4096, 4096, 256), (16, 520, 2048, 128)])
def test_fused_decode_streams_the_native_copy(oracle, M, N, K, bs):
    """MatMulNBitsMlp / MatMulNBitsQkv with 2-bit weights, up to 16 rows: the packed matrix of all projections has the
    copy in the weights' own width too, and decode reads it (the nibble copy is overwritten first)."""
    from onnxruntime_amd.matmul_nbits import MatMulNBitsQkv
    g = make_case(M, N, K, 2, bs, np.float16, has_bias=True, seed=N)
    u = make_case(M, N, K, 2, bs, np.float16, seed=N + 1)
    op = MatMulNBitsMlp(K, N, 2, bs)
    assert op.PrePack(dev(g.B), dev(g.scales), dev(g.bias), dev(u.B), dev(u.scales), None)
    n_pad, k_pad = -(-(2 * (-(-N // 16) * 16)) // 256) * 256, -(-(-(-K // bs) * bs) // 128) * 128
    op.packed[:k_pad // 32 * n_pad * 16] = 0x5A
    y = op.Compute(dev(g.A)).cpu().numpy().astype(np.float64)
    want = oracle.C.mlp(g.A, (g.B, g.scales, g.bias), (u.B, u.scales, None), N, K, 2, bs).astype(np.float64)
    assert float(np.linalg.norm(y - want) / np.linalg.norm(want)) <= 5e-3
    nkv = max(N // 4, 16)
    q, k, v = g, make_case(M, nkv, K, 2, bs, np.float16, has_bias=True, seed=N + 2), make_case(M, nkv, K, 2, bs, np.float16, seed=N + 3)
    opq = MatMulNBitsQkv(K, N, nkv, 2, bs)
    assert opq.PrePack(dev(q.B), dev(q.scales), dev(q.bias), dev(k.B), dev(k.scales), dev(k.bias), dev(v.B), dev(v.scales), None)
    outs = opq.Compute(dev(q.A))
    for got, c in zip(outs[:3], (q, k, v)):
        y64, _ = oracle.C.matmul_f64(q.A, c.B, c.scales, None, c.bias, c.N, K, 2, bs, nthreads=8)
        assert float(np.linalg.norm(got.cpu().numpy().astype(np.float64) - y64) / np.linalg.norm(y64)) <= 5e-3
