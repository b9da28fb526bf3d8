"""The reference's own operator tests, restated on the HIP path: same shape lists, same data construction, same
tolerances (onnxruntime/test/contrib_ops/matmul_4bits_test.cc:128-260, 300-567, 752-1425; matmul_8bits_test.cc:255-610;
matmul_2bits_test.cc:392-465, 1257-1300).

The reference draws A and W from N(0, 0.25), quantises W blockwise (MlasQuantizeBlockwise), runs the operator and
compares with A x dequantised(W) (+ bias from U(1, 5)) at |err| <= abs + rel |expected|: abs 0.05 (fp32) / 0.065 (fp16)
and rel 0.02 in the typed CPU lists, abs 0.02 ... 0.5 and rel 0.001 in the lists it runs on its GPU providers.  Here W
is quantised by the device quantiser, the operator runs through the C ABI, and the result is held to that tolerance AND
to this build's own gates against the oracle (gpu_util.check_against_oracle), which are two to three orders tighter.
Every option set of the reference's tests runs: symmetric, zero points, a group index (the trivial one the reference
uses, 4-bit only), group index + bias, zero points in the activation type, bias, flattened legacy shapes.
accuracy_level is an attribute the device path ignores, so every list runs at level 0 semantics.  bfloat16 has no CPU
kernel in the reference; its lists are held to the reference's tolerance and to a float64 product."""
import numpy as np
import pytest
import torch

from gpu_util import check_against_oracle
from oracle import oracle as oracle_mod
from onnxruntime_amd.matmul_nbits import MatMulNBits, quantize_blockwise
from onnxruntime_amd.synthetic import MatMulNBitsCase

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (M, N, K, block_size): the union of the reference's lists per bit width
LIST_4B = [(1, 1, 16, 16), (1, 2, 16, 16), (1, 32, 16, 16), (1, 32, 32, 16), (1, 32, 16, 128), (1, 288, 16, 16),
           (1, 288, 1024, 16), (1, 288, 1024, 128), (1, 288, 93, 32), (1, 288, 93, 128), (1, 288, 1234, 16),
           (2, 1, 16, 16), (2, 2, 16, 16), (100, 1, 16, 16), (100, 2, 16, 16), (100, 32, 16, 16), (100, 32, 32, 16),
           (100, 32, 16, 128), (100, 64, 32, 32), (100, 128, 128, 32), (100, 288, 16, 16), (100, 288, 1024, 16),
           (100, 288, 1024, 128), (100, 288, 192, 64), (100, 288, 93, 32), (100, 288, 93, 128), (100, 288, 1234, 16),
           (100, 256, 128, 32), (100, 192, 128, 32), (4, 2, 16, 16)]
LIST_8B = [(1, 1, 16, 16), (1, 8, 16, 16), (1, 2, 16, 16), (1, 32, 16, 16), (1, 4, 32, 16), (2, 4, 32, 16),
           (1, 4, 64, 16), (1, 32, 16, 128), (1, 256, 32, 16), (1, 288, 16, 16), (1, 288, 1024, 16),
           (1, 288, 1024, 128), (2, 288, 1024, 128), (1, 40, 576, 32), (2, 40, 576, 32), (1, 288, 93, 32),
           (1, 288, 93, 128), (1, 288, 1234, 16), (2, 1, 16, 16), (2, 2, 16, 16), (100, 1, 16, 16), (100, 2, 16, 16),
           (100, 32, 16, 16), (100, 32, 32, 16), (100, 32, 16, 128), (100, 288, 16, 16), (100, 288, 1024, 16),
           (100, 288, 1024, 128), (100, 288, 192, 64), (100, 288, 93, 32), (100, 288, 93, 128), (100, 288, 1234, 16),
           (32, 64, 260, 32), (100, 64, 32, 32), (100, 128, 128, 32), (199, 40, 576, 32)]
LIST_2B = [(1, 1, 16, 16), (1, 2, 16, 16), (1, 32, 16, 16), (1, 32, 32, 16), (1, 32, 16, 128), (1, 288, 16, 16),
           (2, 1, 16, 16), (2, 2, 16, 16), (4, 1, 16, 16), (4, 2, 16, 16), (4, 32, 16, 16), (4, 32, 32, 16),
           (4, 32, 16, 128), (4, 288, 16, 16), (100, 1, 16, 16), (100, 2, 16, 16), (100, 32, 16, 16),
           (100, 32, 32, 16), (100, 32, 16, 128), (100, 288, 16, 16),
           # the lookup-table GEMM tests of the same file (M, N, K, block)
           (1, 128, 128, 32), (1, 256, 256, 32), (1, 256, 256, 64), (1, 128, 256, 128), (32, 128, 128, 32),
           (32, 256, 256, 32)]
# two large cases the reference runs with its own tolerances: (M, N, K, block, bits, abs, rel)
LARGE = [(369, 6144, 2048, 32, 4, 0.2, 0.03), (2, 5120, 3072, 32, 8, 0.1, 0.02)]

# option sets: "+"-joined flags -- zp (uint8 zero points), typed (zero points in the activation type), g_idx, bias
OPTIONS = ["", "zp", "g_idx", "g_idx+bias", "typed"]   # the typed test's five runs (matmul_4bits_test.cc:357-399)


def to_type(x32, kind):
    if x32 is None:
        return None
    if kind == "bf16":
        return oracle_mod.narrow_bf16(np.ascontiguousarray(x32, np.float32))   # uint16 bits
    return x32.astype(np.float16 if kind == "f16" else np.float32)


def to_dev(x):
    if x is None:
        return None
    if x.dtype == np.uint16:   # bfloat16 bits
        return torch.from_numpy(np.ascontiguousarray(x).view(np.int16)).view(torch.bfloat16).to(DEV)
    return torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def to_f32(x):
    return oracle_mod.widen(x) if x.dtype == np.uint16 else x.astype(np.float32)


def reference_data(M, N, K, bits, bs, kind, has_zp, has_bias):
    """A, the quantised W and the bias as the reference's RunTest builds them (matmul_4bits_test.cc:143-172): fp32 draws,
    W quantised in fp32, then A, scales and bias narrowed to the model's type."""
    rng = np.random.default_rng(1234)
    a32 = (rng.standard_normal((M, K)) * 0.25).astype(np.float32)
    w32 = (rng.standard_normal((K, N)) * 0.25).astype(np.float32)
    b, scales, zp = quantize_blockwise(torch.from_numpy(w32).to(DEV), bits, bs, symmetric=not has_zp)
    torch.cuda.synchronize()
    bias32 = rng.uniform(1.0, 5.0, N).astype(np.float32) if has_bias else None
    return (to_type(a32, kind), b.cpu().numpy(), to_type(scales.cpu().numpy(), kind),
            None if zp is None else zp.cpu().numpy(), to_type(bias32, kind))


def typed_zero_points(zp, N, kb, bits, kind):
    """uint8-packed zero points -> one value per block in the activation type (matmul_4bits_test.cc:222-241)."""
    per = 8 // bits
    fields = np.stack([(zp >> (bits * i)) & ((1 << bits) - 1) for i in range(per)], axis=-1).reshape(N, -1)
    return to_type(fields[:, :kb].astype(np.float32), kind)


TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def run_one(oracle, M, N, K, bits, bs, kind, option, abs_tol=None, rel_tol=0.02):
    flags = set(option.split("+")) - {""}
    has_zp, typed, has_g, has_bias = bool(flags & {"zp", "typed"}), "typed" in flags, "g_idx" in flags, "bias" in flags
    kb = (K + bs - 1) // bs
    A, B, scales, zp, bias = reference_data(M, N, K, bits, bs, kind, has_zp, has_bias)
    tdt = TORCH[kind]
    zp_in, zp_dtype = (typed_zero_points(zp, N, kb, bits, kind), tdt) if typed else (zp, torch.uint8)
    g = (np.arange(kb * bs) // bs).astype(np.int32) if has_g else None   # (matmul_4bits_test.cc:252-259)
    op = MatMulNBits(K, N, bits, bs, dtype=tdt, has_zero_points=has_zp, has_bias=has_bias, has_g_idx=has_g,
                     zero_points_dtype=zp_dtype)
    assert op.supported
    assert op.PrePack(to_dev(B), to_dev(scales), to_dev(zp_in), to_dev(g))
    y = op.Compute(to_dev(A), bias=to_dev(bias))
    torch.cuda.synchronize()
    y = y.cpu()
    y = oracle_mod.widen(y.view(torch.int16).numpy().view(np.uint16)) if kind == "bf16" else y.numpy()
    # the reference's expectation and tolerance: the product over the dequantised weights
    w = oracle.C.dequantize(B, to_f32(scales), zp, N, K, bits, bs).astype(np.float64)   # [N, K]
    expected = to_f32(A).astype(np.float64) @ w.T + (0.0 if bias is None else to_f32(bias).astype(np.float64))
    if abs_tol is None:
        abs_tol = 0.065 if kind == "f16" else (1e-4 if (has_bias and kind == "f32") else 0.05)
    err = np.abs(y.astype(np.float64) - expected)
    assert np.all(err <= abs_tol + rel_tol * np.abs(expected)), \
        f"[{option}] {(M, N, K, bs)}: max err {err.max():.3e} beyond the reference's tolerance"
    # this build's gates (typed zero points hold the same integers, so the canonical oracle applies)
    if kind == "bf16":   # no CPU kernel in the reference: the float64 product only
        rel = float(np.linalg.norm(err) / max(np.linalg.norm(expected), 1e-30))
        assert rel <= 5e-3, f"[{option}] {(M, N, K, bs)}: relative L2 {rel:.3e}"
        return
    case = MatMulNBitsCase(M, N, K, bits, bs, np.dtype(A.dtype), A, B, scales, zp, bias)
    check_against_oracle(oracle, case, y, nthreads=4)


@pytest.mark.parametrize("option", OPTIONS)
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_four_bit_lists(oracle, dtype, option):
    for (M, N, K, bs) in LIST_4B:
        run_one(oracle, M, N, K, 4, bs, dtype, option)


@pytest.mark.parametrize("option", ["", "zp"])   # (the 8-bit typed test has no other option set)
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_eight_bit_lists(oracle, dtype, option):
    for (M, N, K, bs) in LIST_8B:
        run_one(oracle, M, N, K, 8, bs, dtype, option)


@pytest.mark.parametrize("option", ["", "zp", "typed"])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_two_bit_lists(oracle, dtype, option):
    for (M, N, K, bs) in LIST_2B:
        run_one(oracle, M, N, K, 2, bs, dtype, option)


@pytest.mark.parametrize("M,N,K,bs,bits,abs_tol,rel_tol", LARGE)
@pytest.mark.parametrize("option", ["", "zp"])
def test_large_cases(oracle, M, N, K, bs, bits, abs_tol, rel_tol, option):
    dtype = "f16" if bits == 4 else "f32"   # (Float16_4b_Accuracy4's last case; Float32_8b_AccuracyLevel4's)
    run_one(oracle, M, N, K, bits, bs, dtype, option, abs_tol=abs_tol, rel_tol=rel_tol)


def test_legacy_flattened_shapes(oracle):
    """scales [N * k_blocks] and zero_points [N * zp_row] (LegacyShape_4b, matmul_4bits_test.cc:563-567)."""
    for (M, N, K, bs, kind) in [(4, 2, 16, 16, "f32"), (1, 2, 16, 16, "f16")]:
        A, B, scales, zp, _ = reference_data(M, N, K, 4, bs, kind, True, False)
        op = MatMulNBits(K, N, 4, bs, dtype=TORCH[kind], has_zero_points=True)
        assert op.PrePack(to_dev(B), to_dev(scales.reshape(-1)), to_dev(zp.reshape(-1)))
        y = op.Compute(to_dev(A))
        torch.cuda.synchronize()
        case = MatMulNBitsCase(M, N, K, 4, bs, np.dtype(A.dtype), A, B, scales, zp, None)
        check_against_oracle(oracle, case, y.cpu().numpy())


# ---- the lists the reference runs on its GPU providers (fp16 / bfloat16 only; RunTest overload with rel 0.001,
# matmul_4bits_test.cc:752-776) ----------------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 2, 100])
def test_fp16_comprehensive_grid(oracle, M):
    """Float16_Comprehensive (matmul_4bits_test.cc:804-826; the reference skips it in its own pipeline for its size)."""
    for N in (1, 2, 32, 288):
        for K in (16, 32, 64, 128, 256, 1024, 93, 1234):
            for bs in (16, 32, 64, 128):
                for option in ("", "zp", "typed", "g_idx", "g_idx+zp"):   # (a group index forces uint8 zero points)
                    run_one(oracle, M, N, K, 4, bs, "f16", option, abs_tol=0.02, rel_tol=0.001)


@pytest.mark.parametrize("bs", [16, 32, 64, 128])
def test_fp16_large(oracle, bs):
    """Float16_Large (matmul_4bits_test.cc:828-851)."""
    for option in ("", "zp"):
        for (N, K) in [(4096, 4096), (4096, 11008), (11008, 4096)]:
            run_one(oracle, 1, N, K, 4, bs, "f16", option, abs_tol=0.1, rel_tol=0.001)


@pytest.mark.parametrize("kind,abs_tol", [("f16", 0.1), ("bf16", 0.5)])
def test_gpu_provider_lists(oracle, kind, abs_tol):
    """Fp16_/BFloat16_Int4_Int4ZeroPoint, _Fp16ZeroPoint / _BFloat16ZeroPoint, _NoZeroPoint, _BlockSize32_FpAIntB,
    _NoZeroPoint_Bias (matmul_4bits_test.cc:868-1020) and the 8-bit ones (matmul_8bits_test.cc:520-562)."""
    for bs in (32, 64, 128):
        for option in ("", "zp", "typed", "bias"):
            for (M, N, K) in [(1, 256, 1024), (32, 1024, 2048)]:
                run_one(oracle, M, N, K, 4, bs, kind, option, abs_tol=abs_tol, rel_tol=0.001 if kind == "f16" else 0.02)
    for bs in (32, 64, 128):
        for option in ("", "zp"):
            for (M, N, K) in [(1, 256, 1024), (32, 1024, 2048)]:
                run_one(oracle, M, N, K, 8, bs, kind, option, abs_tol=abs_tol, rel_tol=0.001 if kind == "f16" else 0.02)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_small_m_batched_tiles(oracle, kind):
    """Fp16_/BFloat16_Int4_SmallMBatchedTiles (matmul_4bits_test.cc:1109-1146)."""
    for bs in (32, 128):
        for M in (3, 4, 5, 8, 12, 16):
            for option in ("", "zp"):
                for N in (256, 24):
                    run_one(oracle, M, N, 1024, 4, bs, kind, option, abs_tol=0.1, rel_tol=0.001 if kind == "f16" else 0.02)


def test_router_shape(oracle):
    """Fp16_Int4_GptOssRouterShapeNoZeroPoint (matmul_4bits_test.cc:1148-1186)."""
    for bs in (32, 64):
        for option in ("", "bias"):
            run_one(oracle, 1, 32, 2880, 4, bs, "f16", option, abs_tol=0.1, rel_tol=0.02)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_chunked_lists(oracle, kind):
    """Fp16_/BFloat16_Int4_Chunked_* and Fp16_Int8_Chunked_* (matmul_4bits_test.cc:1215-1400, matmul_8bits_test.cc:
    564-610): the shapes the reference pushes through its chunked dequantise-and-multiply route."""
    rel = 0.001 if kind == "f16" else 0.02
    for bits, options in ((4, ("zp", "typed", "")), (8, ("zp", ""))):
        for option in options:
            for bs in (32, 64, 128):
                for M in (1, 2):
                    run_one(oracle, M, 256, 1024, bits, bs, kind, option, abs_tol=0.1, rel_tol=rel)
            run_one(oracle, 1, 256, 96, bits, 32, kind, option, abs_tol=0.1, rel_tol=rel)


def test_basic_shapes(oracle):
    """Basic_M1_N128_K512(_withZp), Basic_M10_N128_K512(_withZp) (matmul_4bits_test.cc:1407-1425)."""
    for M in (1, 10):
        for option in ("", "zp"):
            for kind in ("f32", "f16"):
                run_one(oracle, M, 128, 512, 4, 32, kind, option)


# ---- the kernel library's own unit-test list (onnxruntime/test/mlas/unittest/test_sqnbitgemm.cpp:467-503) ------------
def mlas_short_list():
    """(M, N, K, with_bias) as SQNBitGemmShortExecuteTest registers them for one block length and symmetry."""
    out = []
    for b in range(1, 16):
        out += [(b, b, b, False), (b, b, b, True)]
    for b in (16, 32, 64, 128, 256):
        out += [(b, b, b, False), (b, b, b, True)]
    for b in range(256, 320, 32):
        out += [(b, b, b, True)]
    for b in range(1, 96):
        out += [(1, b, 32, False), (1, 32, b, True), (1, b, b, False)]
    out += [(43, 500, 401, True), (1, 2, 16, True), (1, 2, 16, False), (1, 1027, 1031, False), (11, 1027, 1031, False),
            (1, 1027, 1031, True), (11, 1027, 1031, True), (1, 527, 2131, False), (11, 527, 2131, False),
            (1, 527, 2131, True), (11, 527, 2131, True)]
    return out


def guard_buffer_pattern(n):
    """The deterministic fill of the unit tests' buffers: 32, 39, 46, ... stepping by 7 and wrapping inside [21, 64)
    (onnxruntime/test/mlas/unittest/test_util.h:123-138)."""
    return (((11 + 7 * np.arange(n, dtype=np.int64)) % 43) + 21).astype(np.float32)


@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
def test_kernel_library_unit_test_list(oracle, bs, symmetric):
    """fp32 activations, 4-bit weights quantised from the unit test's buffers (test_sqnbitgemm.cpp:209-274, 582-586);
    fp16 on the same list for two block sizes, with A and W scaled by 1/64 so that the sums stay finite."""
    kinds = ("f32", "f16") if bs in (32, 128) else ("f32",)
    for (M, N, K, with_bias) in mlas_short_list():
        for kind in kinds:
            unit = np.float32(1.0 if kind == "f32" else 1.0 / 64)
            a32 = guard_buffer_pattern(M * K).reshape(M, K) * unit
            w32 = guard_buffer_pattern(N * K).reshape(K, N) * unit
            bias32 = guard_buffer_pattern(N) * unit if with_bias else None
            b, scales, zp = quantize_blockwise(torch.from_numpy(w32).to(DEV), 4, bs, symmetric=symmetric)
            torch.cuda.synchronize()
            B, Z = b.cpu().numpy(), None if zp is None else zp.cpu().numpy()
            A, sc, bias = to_type(a32, kind), to_type(scales.cpu().numpy(), kind), to_type(bias32, kind)
            op = MatMulNBits(K, N, 4, bs, dtype=TORCH[kind], has_zero_points=not symmetric, has_bias=with_bias)
            assert op.PrePack(to_dev(B), to_dev(sc), to_dev(Z))
            y = op.Compute(to_dev(A), bias=to_dev(bias))
            torch.cuda.synchronize()
            case = MatMulNBitsCase(M, N, K, 4, bs, np.dtype(A.dtype), A, B, sc, Z, bias)
            check_against_oracle(oracle, case, y.cpu().numpy(), nthreads=4)


# ---- 2-bit weights with zero points that are not integers (matmul_2bits_test.cc:579-1255) --------------------------
def run_float_zero_points(M, N, K, bs, kind, zp_of, prepacked=True, uint8_zp=None):
    """W ~ N(0, 0.25) quantised symmetrically to 2 bits, then paired with the zero points the test supplies; the
    expectation is A x ((q - zp) scale) as the reference computes it (abs 0.1, rel 0.02), and this build's gates:
    fp32 max |err| <= 1e-4 sum |a w|, fp16 relative L2 <= 5e-3."""
    rng = np.random.default_rng(1234)
    a32 = (rng.standard_normal((M, K)) * 0.25).astype(np.float32)
    w32 = (rng.standard_normal((K, N)) * 0.25).astype(np.float32)
    b, scales, _ = quantize_blockwise(torch.from_numpy(w32).to(DEV), 2, bs, symmetric=True)
    torch.cuda.synchronize()
    kb = (K + bs - 1) // bs
    B, sc, A = b.cpu().numpy(), to_type(scales.cpu().numpy(), kind), to_type(a32, kind)
    if uint8_zp is not None:
        zp_in, zp_dtype = uint8_zp, torch.uint8
        zp_val = oracle_mod.np_unpack_zp(uint8_zp, N, K, 2, bs).astype(np.float64)
    else:
        zp_in = to_type(np.array([[zp_of(n, blk) for blk in range(kb)] for n in range(N)], np.float32), kind)
        zp_dtype, zp_val = TORCH[kind], to_f32(zp_in).astype(np.float64)
    op = MatMulNBits(K, N, 2, bs, dtype=TORCH[kind], has_zero_points=True, zero_points_dtype=zp_dtype)
    assert op.supported
    if prepacked:
        assert op.PrePack(to_dev(B), to_dev(sc), to_dev(zp_in))
        y = op.Compute(to_dev(A))
    else:   # zero points fed per run (Float32_2b_FloatZP_DynamicZP)
        y = op.Compute(to_dev(A), to_dev(B), to_dev(sc), to_dev(zp_in))
    torch.cuda.synchronize()
    y = y.cpu().numpy().astype(np.float64)
    q = oracle_mod.np_unpack_q(B, N, K, 2, bs).reshape(N, kb, bs).astype(np.float64)
    w = ((q - zp_val[:, :, None]) * to_f32(sc).astype(np.float64)[:, :, None]).reshape(N, kb * bs)[:, :K]
    a64 = to_f32(A).astype(np.float64)
    expected, bound = a64 @ w.T, np.abs(a64) @ np.abs(w).T
    err = np.abs(y - expected)
    assert np.all(err <= 0.1 + 0.02 * np.abs(expected)), (M, N, K, bs, float(err.max()))
    if kind == "f32":
        assert float(np.max(err / (bound + 1e-30))) <= 1e-4, (M, N, K, bs)
    else:
        assert float(np.linalg.norm(err) / np.linalg.norm(expected)) <= 5e-3, (M, N, K, bs)


def test_two_bit_float_zero_points():
    # Float32_2b_FloatZP_QAD: zp = 1.5 maps {0, 1, 2, 3} to {-1, -1/3, 1/3, 1} x scale
    for (M, N, K, bs, zp) in [(1, 128, 128, 32, 1.5), (1, 256, 256, 64, 1.5), (1, 128, 128, 32, 0.0),
                              (1, 128, 128, 32, 2.0), (1, 128, 128, 32, 3.0)]:
        run_float_zero_points(M, N, K, bs, "f32", lambda n, blk, zp=zp: zp)
    # Float32_2b_FloatZP_VaryingPerBlock and _DynamicZP: a different zero point for every (column, block)
    varying = lambda n, blk: 0.25 + 0.5 * blk + 0.01 * (n % 17)
    run_float_zero_points(1, 128, 128, 32, "f32", varying)
    run_float_zero_points(1, 128, 128, 32, "f32", varying, prepacked=False)
    # Float32_2b_FloatZP_Fallback, _Fallback_NonAlignedK, MLFloat16_2b_MLFloat16ZP_Fallback
    run_float_zero_points(1, 32, 32, 16, "f32", lambda n, blk: 1.5)
    run_float_zero_points(1, 32, 48, 32, "f32", lambda n, blk: 1.5)
    run_float_zero_points(1, 32, 32, 16, "f16", lambda n, blk: 1.5)


def test_two_bit_uint8_zero_points_that_vary():
    """MLFloat16_2b_Uint8ZP_Fallback and _Accuracy4 (matmul_2bits_test.cc:1102-1255): packed 2-bit zero points, the
    second test with bytes (hi << 4) | lo, lo = 3 i mod 4, hi = (5 i + 1) mod 4, so that they differ from the default."""
    N, K, bs = 32, 32, 16
    rng = np.random.default_rng(7)
    run_float_zero_points(1, N, K, bs, "f16", None, uint8_zp=rng.integers(0, 256, (N, 1), dtype=np.uint8))
    N, K, bs = 32, 128, 64
    i = np.arange(N)
    zp = ((((5 * i + 1) % 4) << 4) | ((3 * i) % 4)).astype(np.uint8).reshape(N, 1)
    run_float_zero_points(1, N, K, bs, "f16", None, uint8_zp=zp)
    run_float_zero_points(1, N, K, bs, "f32", None, uint8_zp=zp)
