"""The device quantiser (MnbQuantizeBlockwise) against the oracle's restatement of MlasQuantizeBlockwise: every
output byte identical on seeded inputs, plus size-independent properties at a BASELINE shape."""
import numpy as np
import pytest
import torch

import tie_cases
from gpu_util import dev
from oracle.oracle import np_unpack_q, np_unpack_zp
from onnxruntime_amd.matmul_nbits import MatMulNBits, dequantize_blockwise, quantize_blockwise

pytestmark = pytest.mark.gpu


def _bits(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("symmetric", [False, True])
def test_identical_to_oracle(oracle, dtype, bits, bs, symmetric):
    for (K, N) in [(64, 8), (93, 33), (260, 300), (1234, 5), (512, 257), (200, 128), (1000, 192)]:
        rng = np.random.default_rng(K * 7 + N + bits + bs)
        W = (rng.standard_normal((K, N)) * rng.uniform(0.01, 2.0, size=(1, N))).astype(dtype)
        W[:, 0] = 0                                   # an all-zero column: scale 0
        if N > 2:
            W[:, 1] = np.abs(W[:, 1])                 # one-sided ranges: zero point clamps to 0 / maxq
            W[:, 2] = -np.abs(W[:, 2])
        Bq, s, z = oracle.C.quantize(W, bits, bs, symmetric)
        b, sc, zp = quantize_blockwise(dev(W), bits, bs, symmetric)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(sc.cpu().numpy()), _bits(s)), (K, N, "scales")
        if symmetric:
            assert zp is None and z is None
        else:
            assert np.array_equal(zp.cpu().numpy(), z), (K, N, "zero points")
        assert np.array_equal(b.cpu().numpy(), Bq), (K, N, "weights")


# (rows = K, columns = N, block) of the reference's quantise -> dequantise test, column-wise blocks
# (onnxruntime/test/mlas/unittest/test_blockq4.cpp:191-229)
QDQ_SHAPES = [(20, 1, 32), (52, 1, 32), (20, 3, 32), (52, 3, 32), (52, 3, 64), (32 * 9 + 17, 41, 32),
              (32 * 9 + 17, 41, 64), (32 * 15 + 17, 63, 128), (256, 256, 32)]
QDQ_TOLERANCE = {8: (1e-2, 5e-2), 4: (6e-2, 2e-1), 2: (2e-1, 5e-1)}   # |a - b| < err + |a| rel (test_blockq4.cpp:55-63)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("symmetric", [False, True])
def test_reference_round_trip_list(oracle, dtype, bits, symmetric):
    """MlasBlockwiseQdqTest: weights from U(-1, 1), quantise, dequantise, compare with the reference's tolerance --
    and every byte of the quantiser's and every bit of the dequantiser's output against the oracle."""
    err, rel = QDQ_TOLERANCE[bits]
    for (K, N, bs) in QDQ_SHAPES:
        rng = np.random.default_rng(192373 + K + N + bs)
        W = rng.uniform(-1.0, 1.0, size=(K, N)).astype(dtype)
        b, sc, zp = quantize_blockwise(dev(W), bits, bs, symmetric)
        w = dequantize_blockwise(b, sc, zp, N, K, bits, bs)
        torch.cuda.synchronize()
        Bq, s, z = oracle.C.quantize(W, bits, bs, symmetric)
        assert np.array_equal(b.cpu().numpy(), Bq) and np.array_equal(_bits(sc.cpu().numpy()), _bits(s)), (K, N, bs)
        assert (zp is None and z is None) or np.array_equal(zp.cpu().numpy(), z), (K, N, bs)
        w = w.cpu().numpy()
        assert np.array_equal(_bits(w), _bits(oracle.C.dequantize(Bq, s, z, N, K, bits, bs))), (K, N, bs)
        a32, b32 = W.astype(np.float32), w.T.astype(np.float32)
        assert np.all(np.abs(a32 - b32) < err + np.abs(a32) * rel), (K, N, bs, float(np.abs(a32 - b32).max()))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bs", [16, 64, 128])
@pytest.mark.parametrize("symmetric", [False, True])
def test_signed_zeros_and_nans_follow_the_sequential_scan(oracle, dtype, bs, symmetric):
    """The reference scans a block with `if (v < min) min = v; if (v > max) max = v` (q4_dq.cpp:513-516): among equal
    values the first one met stays, so the symmetric scale of an all-zero block takes its sign from the block's first
    element (+0 -> scale -0, -0 -> scale +0), zeros of either sign inside an ordinary block change nothing, and a NaN
    never enters the range.  Whole blocks and a ragged last block, every quarter of a block starting with either
    zero."""
    K, N = 3 * bs + bs // 2, 140
    rng = np.random.default_rng(bs)
    W = np.zeros((K, N), dtype)
    signs = rng.integers(0, 2, size=(K, N)).astype(bool)
    W[signs] = -0.0                                       # columns 0..69: nothing but zeros of random sign
    W[:, 70:] = rng.standard_normal((K, N - 70)).astype(dtype)
    zero_at = rng.integers(0, 4, size=(K, N - 70)) == 0   # columns 70..: ordinary values with zeros of both signs
    W[:, 70:][zero_at] = np.where(rng.integers(0, 2, size=int(zero_at.sum())).astype(bool), -0.0, 0.0).astype(dtype)
    W[0, :35], W[0, 35:70] = 0.0, -0.0                    # both first elements, also for the later blocks' quarters
    for q in range(1, 14):
        W[q * bs // 4, q % 2:70:2] = -0.0
    Wn = W.copy()
    Wn[1::7, 100:] = np.nan                               # NaNs are skipped by both comparisons
    for src in (W, Wn):
        Bq, s, z = oracle.C.quantize(src, 4, bs, symmetric)
        b, sc, zp = quantize_blockwise(dev(src), 4, bs, symmetric)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(sc.cpu().numpy()), _bits(s))
        if not symmetric:
            assert np.array_equal(zp.cpu().numpy(), z)
        if src is W:                                      # (a NaN element itself converts to an unspecified integer)
            assert np.array_equal(b.cpu().numpy(), Bq)
    if symmetric:
        s_bits = _bits(s)[:70, 0]
        sign = np.uint32(1) << np.uint32(8 * s.dtype.itemsize - 1)
        assert np.array_equal((s_bits & sign) != 0, np.arange(70) < 35)   # +0 first -> scale -0


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("bs", [16, 64])
@pytest.mark.parametrize("symmetric", [False, True])
def test_exact_ties_round_away_from_zero(dtype, bits, bs, symmetric):
    """Elements exactly half way between two integers: the device returns the closed-form integers of the reference's
    roundf (x + 0.5 -> x + 1, q4_dq.cpp:558), the same ones tests/test_oracle_quantize.py demands of the oracle."""
    W, scale, zp_want, want = tie_cases.element_ties(bits, bs, dtype, symmetric)
    K, N = W.shape
    b, sc, zp = quantize_blockwise(dev(W), bits, bs, symmetric)
    torch.cuda.synchronize()
    assert np.array_equal(sc.cpu().numpy(), scale)
    if not symmetric:
        assert np.array_equal(np_unpack_zp(zp.cpu().numpy(), N, K, bits, bs), zp_want)
    assert np.array_equal(np_unpack_q(b.cpu().numpy(), N, K, bits, bs), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_zero_point_ties_round_away_from_zero(dtype, bits):
    """-min / scale = z + 0.5 -> zero point z + 1 (roundf, q4_dq.cpp:367), and the elements that become ties with it."""
    W, scale, zp_want, want = tie_cases.zero_point_ties(bits, 32, dtype)
    K, N = W.shape
    b, sc, zp = quantize_blockwise(dev(W), bits, 32, symmetric=False)
    torch.cuda.synchronize()
    assert np.array_equal(sc.cpu().numpy(), scale)
    assert np.array_equal(np_unpack_zp(zp.cpu().numpy(), N, K, bits, 32), zp_want)
    assert np.array_equal(np_unpack_q(b.cpu().numpy(), N, K, bits, 32), want)


def test_strided_source_and_grid_round_trip():
    """Weights that lie exactly on a quantisation grid come back unchanged through quantise -> dequantise."""
    rng = np.random.default_rng(3)
    N, kb, bs, bits = 70, 5, 32, 4
    K = kb * bs
    q = rng.integers(0, 16, size=(N, kb, bs))
    q[:, :, 0], q[:, :, 1] = 0, 15
    zp = rng.integers(1, 15, size=(N, kb))
    scale = np.ldexp(1.0, -rng.integers(2, 9, size=(N, kb)))
    w = ((q - zp[..., None]) * scale[..., None]).reshape(N, K).T.astype(np.float16)     # [K, N], exact
    wide = torch.zeros(K, N + 10, dtype=torch.float16, device="cuda")
    wide[:, :N] = dev(w)
    b, sc, z = quantize_blockwise(wide[:, :N], bits, bs, symmetric=False)                # row stride N + 10
    back = dequantize_blockwise(b, sc, z, N, K, bits, bs)
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy(), w.T)


@pytest.mark.parametrize("symmetric", [False, True])
def test_full_size_properties(symmetric):
    """K=4096, N=14336 (BASELINE configs[1] shape): error bound of the round trip and the op on the result."""
    K, N, bits, bs = 4096, 14336, 4, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    w = torch.randn(K, N, generator=g, device="cuda", dtype=torch.float16) * 0.05
    b, sc, z = quantize_blockwise(w, bits, bs, symmetric)
    back = dequantize_blockwise(b, sc, z, N, K, bits, bs)                               # [N, K]
    step = sc.abs().float().repeat_interleave(bs, dim=1)[:, :K]
    err = (back.float() - w.t().float()).abs()
    # inside the grid the error is half a step; at its ends the rounded zero point can push a value half a step out
    # of range (asymmetric), and the symmetric grid is one step short on one side
    slack = 1.5 if symmetric else 1.0
    assert bool((err <= step * slack * 1.02 + 1e-6).all())
    assert float((err <= step * 0.5 * 1.02 + 1e-6).float().mean()) > 0.97
    # the operator on the quantised weights equals A x dequantised weights
    op = MatMulNBits(K, N, bits, bs, dtype=torch.float16, has_zero_points=z is not None)
    assert op.PrePack(b, sc, z)
    a = torch.randn(4, K, generator=g, device="cuda", dtype=torch.float16)
    y = op.Compute(a)
    ref = a.float() @ back.float().t()
    rel = float((y.float() - ref).norm() / ref.norm())
    assert rel <= 5e-3, rel


def test_quantise_write_model_run_through_plugin(oracle, tmp_path):
    """fp16 weights -> device quantiser -> .onnx file -> the node of that file through the plugin EP."""
    from ep_host import host
    from onnxruntime_amd import onnx_writer as ow
    if not host.available():
        pytest.skip("plugin EP or host shim not built")
    rng = np.random.default_rng(5)
    K, N, bits, bs = 384, 200, 4, 64
    W = (rng.standard_normal((K, N)) * 0.1).astype(np.float16)
    b, sc, zp = quantize_blockwise(dev(W), bits, bs, symmetric=False)
    path = tmp_path / "fc.onnx"
    path.write_bytes(ow.matmul_nbits_model(b.cpu().numpy(), sc.cpu().numpy(), zp.cpu().numpy(), K, N, bits, bs,
                                           prefix="fc"))
    m = ow.read_model(path.read_bytes())
    nd = m["nodes"][0]
    ins = [m["initializers"].get(name) for name in nd["inputs"][1:]]
    A = rng.standard_normal((9, K)).astype(np.float16)
    y, trace = host.run_matmul_nbits(nd["attrs"]["N"], nd["attrs"]["K"], nd["attrs"]["bits"],
                                     nd["attrs"]["block_size"], A, ins[0], ins[1], ins[2])
    assert "prepacked=1,2,3," in trace
    y64, _ = oracle.C.matmul_f64(A, ins[0], ins[1], ins[2], None, N, K, bits, bs)
    rel = np.linalg.norm(y.astype(np.float64) - y64) / np.linalg.norm(y64)
    assert rel <= 5e-3
    # and the quantised model stays close to the original weights: 4-bit, 64-deep blocks of N(0, 0.1)
    y_fp = A.astype(np.float64) @ W.astype(np.float64)
    assert np.linalg.norm(y64 - y_fp) / np.linalg.norm(y_fp) < 0.15
