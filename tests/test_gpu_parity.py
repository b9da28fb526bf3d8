"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle and the golden vectors."""
import numpy as np
import pytest
import torch

from golden_cases import load_js_cases
from gpu_util import check_against_oracle, dev, make_op, run_case, tdtype
from onnxruntime_amd.matmul_nbits import MatMulNBits, dequantize_blockwise
from onnxruntime_amd.synthetic import make_case

pytestmark = pytest.mark.gpu

JS = load_js_cases()


def _bits_view(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


# ----------------------------------------------------------------------------------------------- golden vectors
@pytest.mark.parametrize("prepack", [True, False])
@pytest.mark.parametrize("case", JS, ids=[f"{i}" for i in range(len(JS))])
def test_reference_vectors(case, prepack):
    c = case
    op = MatMulNBits(c["K"], c["N"], c["bits"], c["block_size"], dtype=torch.float32,
                     has_zero_points=c["zero_points"] is not None)
    a, b, s, z = dev(c["A"]), dev(c["B"]), dev(c["scales"]), dev(c["zero_points"])
    if prepack:
        assert op.PrePack(b, s, z)
        y = op.Compute(a)
    else:
        y = op.Compute(a, b, s, z)
    torch.cuda.synchronize()
    assert tuple(y.shape) == c["Y"].shape
    assert np.array_equal(y.cpu().numpy(), c["Y"]), c["name"]


# ----------------------------------------------------------------------------------------------- dequant, bit exact
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("zp", [False, True])
def test_dequant_bit_exact(oracle, dtype, bits, bs, zp):
    for (N, K) in [(8, 64), (33, 93), (300, 260), (5, 1234)]:
        c = make_case(1, N, K, bits, bs, dtype, has_zp=zp, seed=N + K)
        want = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs)
        got = dequantize_blockwise(dev(c.B), dev(c.scales), dev(c.zero_points), N, K, bits, bs).cpu().numpy()
        assert np.array_equal(_bits_view(got), _bits_view(want)), "canonical dequantise"
        op = make_op(c)
        got_p = op.dequantize_packed().cpu().numpy()
        assert np.array_equal(_bits_view(got_p), _bits_view(want)), "packed dequantise"


@pytest.mark.parametrize("bits,bs", [(4, 16), (8, 16), (4, 32)])
def test_dequant_exhaustive_q_zp(bits, bs):
    """All 2^bits x 2^bits (q, zp) pairs against integer arithmetic, for both model types."""
    levels = 1 << bits
    N, K = levels, max(levels, bs) * 2
    kb = K // bs
    q = np.broadcast_to(np.arange(K)[None, :] % levels, (N, K)).copy()
    zpv = (np.arange(N)[:, None] + np.arange(kb)[None, :]) % levels
    per = 8 // bits
    B = np.zeros((N, kb, bs * bits // 8), np.uint8)
    Z = np.zeros((N, (kb * bits + 7) // 8), np.uint8)
    qq = q.reshape(N, kb, bs // per, per)
    for j in range(per):
        B |= (qq[..., j] << (bits * j)).astype(np.uint8)
    zz = np.zeros((N, Z.shape[1] * per), np.int64)
    zz[:, :kb] = zpv
    zz = zz.reshape(N, Z.shape[1], per)
    for j in range(per):
        Z |= (zz[..., j] << (bits * j)).astype(np.uint8)
    scales = (0.5 ** (np.arange(N * kb) % 5)).astype(np.float32).reshape(N, kb) * 3
    want = (q - np.repeat(zpv, bs, axis=1)).astype(np.float64) * np.repeat(scales, bs, axis=1)
    for dt in (np.float32, np.float16):
        s = scales.astype(dt)
        got = dequantize_blockwise(dev(B), dev(s), dev(Z), N, K, bits, bs).cpu().numpy()
        assert np.array_equal(got.astype(np.float64), want)
        op = MatMulNBits(K, N, bits, bs, dtype=tdtype(dt), has_zero_points=True)
        op.PrePack(dev(B), dev(s), dev(Z))
        assert np.array_equal(op.dequantize_packed().cpu().numpy().astype(np.float64), want)


# ----------------------------------------------------------------------------------------------- unit vectors
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits,bs,K,N", [(4, 32, 96, 70), (4, 16, 48, 9), (8, 64, 256, 130), (4, 128, 256, 64),
                                         (8, 16, 40, 11), (4, 64, 93, 17)])
def test_unit_vectors_recover_dequant(oracle, dtype, bits, bs, K, N):
    """A = I pushes every weight through the compute kernels unchanged: Y must equal the dequantised bits.

    M = K rows exercises the large-M kernel; the first rows alone (M <= 16) exercise the GEMV."""
    c = make_case(K, N, K, bits, bs, dtype, has_zp=True, seed=9)
    want = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs).T.copy()  # [K, N]
    eye = np.eye(K, dtype=dtype)
    y = run_case(c, A=eye)
    assert np.array_equal(_bits_view(y), _bits_view(want)), "large-M kernel"
    for m in (1, 3, 16):
        y = run_case(c, A=eye[:m])
        assert np.array_equal(_bits_view(y), _bits_view(want[:m])), f"GEMV M={m}"


# ----------------------------------------------------------------------------------------------- random parity
SHAPES_SMALL_M = [(1, 33, 93), (1, 1031, 1027), (2, 64, 64), (3, 401, 500), (4, 128, 4096), (5, 17, 260),
                  (8, 2131, 527), (11, 1031, 1027), (16, 64, 1234), (16, 256, 2048), (1, 32, 80), (7, 300, 16)]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits,bs,zp,bias", [(4, 32, True, False), (4, 128, False, True), (4, 16, True, True),
                                             (8, 64, True, True), (8, 256, False, False), (4, 64, False, False),
                                             (4, 256, True, True), (8, 16, True, False), (8, 32, False, True),
                                             (8, 128, True, False)])
def test_gemv_parity(oracle, dtype, bits, bs, zp, bias):
    for (M, N, K) in SHAPES_SMALL_M:
        c = make_case(M, N, K, bits, bs, dtype, has_zp=zp, has_bias=bias, seed=M * 7 + N)
        y = run_case(c)
        check_against_oracle(oracle, c, y)


SHAPES_LARGE_M = [(17, 64, 64), (43, 401, 500), (64, 256, 512), (100, 130, 264), (128, 128, 128), (129, 257, 1032),
                  (300, 512, 1024), (33, 1031, 1027), (257, 384, 96)]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("bits,bs,zp,bias", [(4, 32, True, True), (4, 128, False, False), (4, 16, True, False),
                                             (8, 64, True, True), (8, 16, False, True), (4, 64, True, False),
                                             (8, 256, True, False), (4, 256, False, True)])
def test_gemm_parity(oracle, dtype, bits, bs, zp, bias):
    for (M, N, K) in SHAPES_LARGE_M:
        c = make_case(M, N, K, bits, bs, dtype, has_zp=zp, has_bias=bias, seed=M + N + K)
        y = run_case(c)
        check_against_oracle(oracle, c, y)


@pytest.mark.parametrize("bits,bs,zp", [(4, 32, True), (4, 16, False), (8, 64, True), (2, 32, True)])
@pytest.mark.parametrize("M,N,K,offset", [(1500, 2100, 160, 0), (1100, 2100, 100, 0), (700, 4100, 93, 1)])
def test_fp32_matrix_core_gemm_with_128_row_tiles(oracle, bits, bs, zp, M, N, K, offset):
    """fp32 problems whose 64-row tiles no longer fit the chip in one round run 128 x 128 tiles; K that is not a
    multiple of the 32-deep step (tail guarded), A that is not 16-byte aligned (element-wise loads), and unit-vector
    rows that must come back as the fp32 dequantisation, bit for bit, through the fp32 matrix instruction."""
    c = make_case(M, N, K, bits, bs, np.float32, has_zp=zp, has_bias=True, seed=M + K + bits)
    ks = np.arange(K)
    c.A[:K] = 0
    c.A[ks, ks] = 1                                   # rows 0..K-1: unit vectors
    op = make_op(c)
    a = torch.zeros(M * K + 4, dtype=torch.float32, device="cuda:0")
    a_view = a[offset:offset + M * K].view(M, K)
    a_view.copy_(dev(c.A))
    y = op.Compute(a_view, bias=dev(c.bias)).cpu().numpy()
    check_against_oracle(oracle, c, y)
    w = oracle.C.dequantize(c.B, c.scales, c.zero_points, N, K, bits, bs)          # [N, K] fp32
    want = (w.T.astype(np.float32) + c.bias[None, :]).astype(np.float32)            # one fp32 addition per element
    assert np.array_equal(_bits_view(y[:K]), _bits_view(want))


@pytest.mark.parametrize("bits,bs,zp", [(4, 128, False), (4, 128, True), (4, 32, True), (8, 64, True), (8, 16, False)])
@pytest.mark.parametrize("N,K,M", [(8200, 512, 1), (9000, 1024, 5), (12288, 2048, 16), (11008, 4096, 1),
                                   (12281, 640, 3), (9216, 4096, 8), (11008, 4096, 16)])
def test_decode_with_three_tile_slabs(oracle, bits, bs, zp, N, K, M):
    """513..768 column tiles: the decode kernel cuts N into slabs of 48 columns that do not start at multiples of 64
    (tiles addressed one by one); every chunk schedule (one, two, many chunks per wavefront), both dequantisation
    modes, ragged N, eight wavefronts instead of sixteen for raw 4-bit operands from four rows on (the last two
    shapes), and unit vectors that recover W bit for bit across slab boundaries."""
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=True, seed=N + K + bits)
    y = run_case(c)
    check_against_oracle(oracle, c, y)
    if K <= 1024:
        eye = np.zeros((16, K), np.float16)
        ks = np.linspace(0, K - 1, 16).astype(int)
        eye[np.arange(16), ks] = 1
        c0 = make_case(16, N, K, bits, bs, np.float16, has_zp=zp, seed=N + K + bits)
        w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
        assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))


@pytest.mark.parametrize("bits,bs,zp", [(4, 128, True), (4, 32, False), (8, 64, True), (8, 128, False)])
@pytest.mark.parametrize("N,K", [(100, 4096), (6144, 2048), (9000, 1024), (14400, 512), (200, 14336), (5200, 8320),
                                 (300, 4160)])
@pytest.mark.parametrize("M", [5, 8, 9, 16])
def test_decode_with_activations_through_lds(oracle, bits, bs, zp, N, K, M):
    """More than four rows: the decode kernel reads its chunk of A row-contiguously and passes it through LDS in a
    swizzled layout (eight rows of it up to M = 8 on single- and two-tile slabs, sixteen otherwise).  Shapes cover one, two and many chunks per wavefront (also unevenly
    many), slabs of one to four tiles, and long K on 4-bit weights (eight wavefronts); with unit-vector rows the
    product must return columns of W bit for bit, so a wrong piece, row or swizzle cannot hide in a tolerance."""
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=True, seed=N + K + M)
    check_against_oracle(oracle, c, run_case(c))
    if N <= 300:
        rng = np.random.default_rng(M + K)
        ks = rng.choice(K, size=M, replace=False)
        eye = np.zeros((M, K), np.float16)
        eye[np.arange(M), ks] = 1
        c0 = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, seed=N + K + M)
        w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
        assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))


@pytest.mark.parametrize("bits,bs,zp", [(4, 128, True), (4, 32, False), (4, 64, True), (8, 64, True), (8, 128, False),
                                        (2, 128, True), (2, 64, False)])
@pytest.mark.parametrize("N,K", [(100, 1024), (4096, 2048), (4090, 4096), (300, 14336), (200, 11008), (6144, 4096),
                                 (6150, 8192), (5200, 2304), (260, 4352)])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
def test_decode_of_up_to_four_rows_on_narrow_slabs(oracle, bits, bs, zp, N, K, M):
    """Up to four rows on single- and two-tile slabs (N < 12800): one load fetches a chunk of all four rows and LDS hands
    the operands out (rows beyond M repeat row M - 1 and are never stored).  Shapes cover one, two and many chunks per
    wavefront, uneven chunk counts, ragged N, both slab widths, the three weight widths and both dequantisation
    modes; with unit-vector rows the product must return columns of W bit for bit, so a wrong row, piece or swizzle
    cannot hide in a tolerance, and distinct unit vectors per row catch rows that were swapped or repeated."""
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=True, seed=N + K + M)
    check_against_oracle(oracle, c, run_case(c))
    if N <= 300 or K <= 2304:
        ks = np.random.default_rng(M + K + N).choice(K, size=M, replace=False)
        eye = np.zeros((M, K), np.float16)
        eye[np.arange(M), ks] = 1
        c0 = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, seed=N + K + M)
        w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
        assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))


@pytest.mark.parametrize("bits,bs,zp", [(4, 128, True), (4, 32, False), (8, 64, True), (8, 16, False)])
@pytest.mark.parametrize("N,K,M", [(20480, 4096, 1), (20490, 4096, 8), (24576, 4096, 16), (28672, 4096, 1),
                                   (28672, 4096, 9), (33000, 8192, 3), (4096, 8192, 2), (4096, 11008, 8),
                                   (14400, 8192, 9), (16000, 14336, 16), (14336, 8320, 12), (28672, 4096, 13),
                                   (14336, 4096, 1), (13000, 4096, 4), (16384, 4096, 3)])
def test_decode_with_more_slabs_than_compute_units(oracle, bits, bs, zp, N, K, M):
    """More four-tile slabs than compute units (N > 16384 on 256 units) with a K deep enough for sixteen wavefronts:
    the decode kernel runs smaller workgroups instead - two-tile slabs up to 1.6 slabs per unit, four or eight
    wavefronts with the general chunk loop beyond - and 8-bit weights over K >= 8192 run eight wavefronts on
    single-tile slabs.  The last four shapes are four-tile slabs whose 4-bit weights run the straight-line chunk loop in
    eight wavefronts from nine rows on (long K) with the activations through LDS (raw operands), also over an uneven
    number of chunks; the last three are raw 4-bit operands with zero points at K = 4096 and up to four rows, which run
    eight wavefronts as well.  Every row of Y against the oracle; unit-vector rows return columns of W bit for bit."""
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=True, seed=N + K + M)
    check_against_oracle(oracle, c, run_case(c))
    if K == 4096 and M >= 8:
        ks = np.random.default_rng(N).choice(K, size=M, replace=False)
        eye = np.zeros((M, K), np.float16)
        eye[np.arange(M), ks] = 1
        c0 = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, seed=N + K + M)
        w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
        assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))


@pytest.mark.parametrize("bits,bs,zp", [(4, 128, True), (4, 32, False), (4, 16, True), (8, 64, True), (8, 16, False)])
@pytest.mark.parametrize("N,K,M", [(28672, 1024, 64), (21000, 1024, 17), (28672, 2048, 32), (24000, 1024, 33),
                                   (11008, 1024, 100), (14336, 4096, 128), (6144, 1024, 250),
                                   (28672, 1152, 64), (21000, 1408, 40)])   # K: 9 and 11 chunks of 128
def test_streaming_kernel_with_activations_shared_through_lds(oracle, bits, bs, zp, N, K, M):
    """Wide matrices whose 128-column slabs make one well-filled round of workgroups: pairs of wavefronts share each
    chunk of the activations through LDS (fetched straight from the caller's A, no staged copy).  Every row of Y against
    the oracle on sampled rows; unit-vector rows return columns of W bit for bit; a misaligned A takes the staged route
    and gives the same sums up to their order."""
    from onnxruntime_amd import _lib
    lib = _lib.load()
    if lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16) != b"mnb_mid_shared_kernel":
        pytest.skip("this device's compute-unit count does not select the shared-activations variant here")
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, has_bias=True, seed=N + K + M)
    y = run_case(c)
    check_against_oracle(oracle, c, y)
    ks = np.random.default_rng(N).choice(K, size=M, replace=False)
    eye = np.zeros((M, K), np.float16)
    eye[np.arange(M), ks] = 1
    c0 = make_case(M, N, K, bits, bs, np.float16, has_zp=zp, seed=N + K + M)
    w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
    assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))
    # a pitch beyond K that keeps the rows 16-byte aligned: still read in place, the same bits
    op = make_op(c)
    pitched = torch.zeros(M, K + 8, dtype=torch.float16, device="cuda")
    pitched[:, :K] = dev(c.A)
    y1 = op.Compute(pitched[:, :K], bias=dev(c.bias)).cpu().numpy()
    assert np.array_equal(_bits_view(y1), _bits_view(y))
    # rows that are not 16-byte aligned: the staged route
    wide = torch.zeros(M, K + 3, dtype=torch.float16, device="cuda")
    wide[:, :K] = dev(c.A)
    y2 = op.Compute(wide[:, :K], bias=dev(c.bias)).cpu().numpy()
    d = np.abs(y2.astype(np.float64) - y.astype(np.float64))
    assert d.max() <= 2e-3 * np.abs(y).max() + 1e-3


@pytest.mark.parametrize("bits,bs,zp", [(4, 32, True), (4, 128, False), (4, 16, True), (8, 64, True)])
@pytest.mark.parametrize("N,K", [(300, 4096), (4100, 8192), (1000, 14336), (8200, 4096)])
@pytest.mark.parametrize("M", [1, 2, 4])
def test_fp32_few_rows_with_k_split_over_sixteen_wavefronts(oracle, bits, bs, zp, N, K, M):
    """fp32 models, up to four rows, K of 32 chunks and more on grids of up to two workgroups per compute unit: the
    16-column kernel splits K over sixteen wavefronts (eight on larger grids: N = 8200 here).  Against the oracle, and
    unit-vector rows return columns of W bit for bit."""
    c = make_case(M, N, K, bits, bs, np.float32, has_zp=zp, has_bias=True, seed=N + K + M)
    check_against_oracle(oracle, c, run_case(c))
    ks = np.random.default_rng(K + M).choice(K, size=M, replace=False)
    eye = np.zeros((M, K), np.float32)
    eye[np.arange(M), ks] = 1
    c0 = make_case(M, N, K, bits, bs, np.float32, has_zp=zp, seed=N + K + M)
    w = oracle.C.dequantize(c0.B, c0.scales, c0.zero_points, N, K, bits, bs)
    assert np.array_equal(_bits_view(run_case(c0, A=eye)), _bits_view(np.ascontiguousarray(w[:, ks].T)))


def test_unpacked_route_matches_packed_and_the_oracle(oracle):
    for dtype in (np.float16, np.float32):
        for (M, N, K, bits, bs) in [(1, 96, 160, 4, 32), (40, 200, 256, 8, 64), (16, 64, 4096, 4, 128),
                                    (3, 33, 93, 2, 16), (70, 130, 1234, 4, 16)]:
            c = make_case(M, N, K, bits, bs, dtype, has_zp=True, has_bias=True, seed=4)
            y = run_case(c, prepack=False)
            assert np.array_equal(run_case(c, prepack=True), y)
            check_against_oracle(oracle, c, y)


def test_batched_leading_dims_and_strided_a(oracle):
    c = make_case(6, 96, 128, 4, 32, np.float16, has_zp=True, seed=2, a_shape=(2, 3, 128))
    op = make_op(c)
    y = op.Compute(dev(c.A))
    assert tuple(y.shape) == (2, 3, 96)
    check_against_oracle(oracle, c, y.cpu().numpy().reshape(6, 96), A=c.A.reshape(6, 128))
    # rows of A with a pitch larger than K
    big = torch.zeros(6, 160, dtype=torch.float16, device="cuda")
    big[:, :128] = dev(c.A.reshape(6, 128))
    y2 = op.Compute(big[:, :128])
    assert torch.equal(y2, y.view(6, 96))


def test_empty_output():
    c = make_case(1, 64, 64, 4, 32, np.float16, seed=1)
    op = make_op(c)
    y = op.Compute(torch.empty(0, 64, dtype=torch.float16, device="cuda"))
    assert tuple(y.shape) == (0, 64)


def test_deterministic_run_to_run():
    c = make_case(4, 4096, 4096, 4, 64, np.float16, has_zp=True, seed=3)
    op = make_op(c)
    a = dev(c.A)
    y0 = op.Compute(a).clone()
    for _ in range(3):
        assert torch.equal(op.Compute(a), y0)


def test_streaming_kernel_needs_no_workspace_when_a_is_aligned(oracle):
    """16 < M with aligned rows and K a whole number of chunks: the streaming kernel reads A in place, so a call without
    the workspace MnbGemmWorkspaceSize names is served (bit-identical to the call with it); a misaligned A still needs
    the staged copy and is refused without room for it."""
    import ctypes
    from onnxruntime_amd import _lib
    lib = _lib.load()
    M, N, K, bits, bs = 40, 384, 1024, 4, 32
    assert lib.MnbGemmKernelName(M, N, K, bits, bs, _lib.DTYPE_FLOAT16).decode() == "mnb_mid_kernel"
    c = make_case(M, N, K, bits, bs, np.float16, has_zp=True, has_bias=True, seed=5)
    op = make_op(c)
    a, bias = dev(c.A), dev(c.bias)
    ptr = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    need = lib.MnbGemmWorkspaceSize(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ys = []
    for w, nbytes in ((ws, need), (None, 0)):
        y = torch.empty(M, N, dtype=torch.float16, device="cuda")
        _lib.check(lib.MnbGemm(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, ptr(a), K, ptr(op.packed), ptr(bias), ptr(y), N,
                               ptr(w), nbytes, None))
        torch.cuda.synchronize()
        ys.append(y)
    assert torch.equal(ys[0].view(torch.int16), ys[1].view(torch.int16))
    check_against_oracle(oracle, c, ys[1].cpu().numpy())
    flat = torch.zeros(M * K + 1, dtype=torch.float16, device="cuda")
    flat[1:] = a.reshape(-1)
    y = torch.empty(M, N, dtype=torch.float16, device="cuda")
    rc = lib.MnbGemm(M, N, K, bits, bs, 1, _lib.DTYPE_FLOAT16, ptr(flat[1:]), K, ptr(op.packed), ptr(bias), ptr(y), N,
                     None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "workspace of" in _lib.last_error()
