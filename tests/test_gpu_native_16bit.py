"""16-bit models on a matrix packed with fp32 scales and zero points - bfloat16, and fp16 with zero points in the
activation type - on the matrix cores in their own type (weights dequantised in fp32, narrowed, fp32 accumulation): the
decode kernel up to 16 rows, the streaming kernel or the tile GEMM beyond (chosen as for fp16 models: the tile GEMM
takes the large problems), through the C ABI's variant entry points and the host class.

The reference's CPU provider has no bfloat16 kernel; its GPU provider dequantises B into bfloat16 and calls a bfloat16
GEMM (contrib_ops/cuda/quantization/matmul_nbits.cc:844-975), which is the arithmetic here.  Gates: relative L2 <= 5e-3
against a float64 product over the reference dequantiser's W (the operator's 16-bit tolerance), bit-exact recovery of W
from unit-vector activations where no operation rounds, and bit-equal results between activations read in place and
activations that go through the copy (misaligned base, odd pitch)."""
import ctypes

import numpy as np
import pytest
import torch

from onnxruntime_amd import MatMulNBits, _lib
from oracle import oracle
from test_gpu_variants import check, make, run_op, to_dev, to_host32, to_np_type

pytestmark = pytest.mark.gpu
C = oracle.C
TILE = "mnb_gemm256_kernel"
DECODE = "mnb_skinny_kernel"
MID = "mnb_mid_kernel"
BIG = (1024, 4096, 4096)   # M, N, K of a problem the tile GEMM takes


def kernel_name(op, M):
    return op.lib.MnbVariantGemmKernelName(ctypes.byref(op.plan), M).decode()


@pytest.mark.parametrize("bits,bs,zp_kind,g_kind", [
    (4, 32, "none", "none"), (4, 32, "u8", "none"), (4, 32, "typed", "none"), (4, 128, "typed", "none"),
    (4, 16, "u8", "none"), (4, 64, "u8", "act_order"), (4, 32, "typed", "act_order"),
    (8, 32, "none", "none"), (8, 64, "u8", "none"), (8, 16, "u8", "none"), (8, 16, "none", "none"),
    (2, 32, "u8", "none"), (2, 64, "typed", "none"), (2, 128, "none", "none")])
@pytest.mark.parametrize("M", [1, 3, 8, 11, 16, 17, 40, 130, 300, 700])
def test_gemm_against_float64(bits, bs, zp_kind, g_kind, M):
    N, K = 300, 512
    c = make("bf16", N, K, bits, bs, zp_kind, g_kind, M, seed=M + bits + bs, bias=M % 2 == 1)
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == (DECODE if M <= 16 else MID)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (M, N)
    check("bf16", c, y, N, K, bits, bs)


@pytest.mark.parametrize("bits,bs,zp_kind,g_kind", [
    (4, 32, "u8", "none"), (4, 128, "typed", "none"), (4, 16, "none", "none"), (4, 64, "u8", "act_order"),
    (8, 64, "u8", "none"), (8, 16, "u8", "none"), (8, 32, "none", "none"), (2, 32, "typed", "none")])
def test_tile_gemm_against_float64(bits, bs, zp_kind, g_kind):
    M, N, K = BIG
    c = make("bf16", N, K, bits, bs, zp_kind, g_kind, M, seed=bits + bs, bias=True)
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == TILE
    check("bf16", c, y, N, K, bits, bs)


def test_tiles_cut_along_k_and_ragged_tiles():
    """A deep K on few tiles makes the plan cut tiles along K (partial sums travel through the workspace); M and N that
    are not multiples of the tile leave ragged tiles."""
    for (M, N, K, bits, bs) in [(512, 8192, 8192, 4, 64), (1024, 4096, 8192, 8, 64), (1000, 4000, 8192, 4, 32)]:
        c = make("bf16", N, K, bits, bs, "u8", "none", M, seed=M, bias=True)
        y, op = run_op("bf16", c, N, K, bits, bs)
        assert kernel_name(op, M) == TILE
        check("bf16", c, y, N, K, bits, bs)


def unit_rows(M, K, seed):
    ks = np.random.default_rng(seed).choice(K, size=M, replace=False)
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), ks] = 1.0
    return a, ks


@pytest.mark.parametrize("bits,bs,zp_kind,g_kind", [
    (4, 32, "typed", "none"), (4, 64, "u8", "act_order"), (4, 16, "u8", "none"), (8, 16, "u8", "none"),
    (8, 64, "none", "none"), (2, 32, "typed", "none")])
@pytest.mark.parametrize("rows", ["mid", "tile"])
def test_unit_rows_recover_columns_of_w_exactly(bits, bs, zp_kind, g_kind, rows):
    """Power-of-two scales and (half-)integer zero points: q - zp has at most 8 significant bits, so neither the fp32
    dequantisation nor the narrowing to bfloat16 rounds, and a unit-vector row e_k of A must produce column k of the
    reference's W, bit for bit."""
    M, N, K = BIG if rows == "tile" else (200, 200, 256)
    c = make("bf16", N, K, bits, bs, zp_kind, g_kind, M, seed=5, exact=True)
    a, ks = unit_rows(M, K, 1)
    c["A"] = to_np_type(a, "bf16")
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == (TILE if rows == "tile" else MID)
    w = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, bits, bs, honour_u8_zp_with_g_idx=True)
    assert np.array_equal(to_host32(y), w[:, ks].T)


@pytest.mark.parametrize("N,K,bits,bs,zp_kind,g_kind", [
    (14336, 4096, 4, 128, "none", "none"),    # the decode benchmark's shape: everything loaded up front; raw operands
    (4096, 4096, 4, 128, "typed", "none"),    # raw bfloat16 operands (blocks of 128 and more), zero points removed after
    (6144, 4096, 4, 256, "u8", "none"),       # the same on three-tile slabs
    (4096, 14336, 4, 32, "u8", "none"),       # general chunk loop
    (6144, 4096, 8, 64, "u8", "none"),        # three-tile slabs
    (1000, 416, 4, 32, "typed", "none"),      # K that is not a whole number of chunks: activations staged in LDS
    (520, 1000, 8, 16, "u8", "none"),
    (300, 640, 4, 16, "typed", "ragged"),     # gathered columns, blocks of 16
    (300, 640, 2, 32, "typed", "none"),
    (20480, 4096, 4, 128, "typed", "none"),   # more slabs than compute units: two-tile slabs of eight (four) wavefronts
    (28672, 4096, 4, 32, "u8", "none"),       # four-tile slabs of four wavefronts, exact weights
    (28672, 4096, 4, 128, "u8", "none"),      # the same with raw operands
    (28680, 2048, 8, 64, "u8", "none")])      # 8-bit: eight wavefronts
@pytest.mark.parametrize("M", [1, 4, 7, 16])
def test_decode_shapes_against_float64(N, K, bits, bs, zp_kind, g_kind, M):
    c = make("bf16", N, K, bits, bs, zp_kind, g_kind, M, seed=M + N, bias=M % 2 == 0)
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == DECODE
    check("bf16", c, y, N, K, bits, bs)


@pytest.mark.parametrize("bits,bs,zp_kind,g_kind", [
    (4, 32, "typed", "none"), (4, 128, "none", "none"), (4, 64, "u8", "act_order"), (4, 16, "u8", "none"),
    (8, 32, "u8", "none"), (8, 16, "none", "none"), (2, 32, "typed", "none"), (4, 128, "u8", "none"),
    (4, 256, "typed", "none"), (2, 128, "u8", "none")])
def test_decode_unit_rows_recover_columns_of_w_exactly(bits, bs, zp_kind, g_kind):
    """Sixteen unit-vector rows e_k: row m of the product must be column k_m of the reference's W, bit for bit
    (power-of-two scales and (half-)integer zero points: nothing rounds)."""
    N, K, M = 520, 1024, 16
    c = make("bf16", N, K, bits, bs, zp_kind, g_kind, M, seed=6, exact=True)
    a, ks = unit_rows(M, K, 1)
    c["A"] = to_np_type(a, "bf16")
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == DECODE
    w = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, bits, bs, honour_u8_zp_with_g_idx=True)
    assert np.array_equal(to_host32(y), w[:, ks].T)


def test_decode_misaligned_activations_agree_with_aligned():
    N, K, bits, bs, M = 520, 1024, 4, 64, 6
    c = make("bf16", N, K, bits, bs, "u8", "none", M, seed=4, bias=True)
    y, op = run_op("bf16", c, N, K, bits, bs)
    a, bias = to_dev(c["A"]), to_dev(c["bias"])
    flat = torch.zeros(M * (K + 3) + 1, dtype=torch.bfloat16, device=a.device)
    view = flat[1:].view(M, K + 3)[:, :K]    # odd base, odd pitch: the kernel stages the rows itself
    view.copy_(a)
    y2 = op.Compute(view, bias=bias)
    torch.cuda.synchronize()
    # the staged kernel splits K over its wavefronts differently: equal up to the rounding of the fp32 sums
    assert torch.allclose(y.float(), y2.float(), rtol=2e-2, atol=1e-3)
    check("bf16", c, y2, N, K, bits, bs)


def test_tile_gemm_activations_read_in_place_and_through_the_copy_agree():
    (M, N, K), bits, bs = BIG, 4, 32
    c = make("bf16", N, K, bits, bs, "u8", "none", M, seed=9, bias=True)
    y, op = run_op("bf16", c, N, K, bits, bs)
    assert kernel_name(op, M) == TILE
    a = to_dev(c["A"])
    bias = to_dev(c["bias"])
    wide = torch.zeros(M, K + 3, dtype=torch.bfloat16, device=a.device)   # a pitch that is not a multiple of 8
    wide[:, :K] = a
    y2 = op.Compute(wide[:, :K], bias=bias)
    flat = torch.zeros(M * K + 1, dtype=torch.bfloat16, device=a.device)  # a base that is not 16-byte aligned
    flat[1:] = a.reshape(-1)
    y3 = op.Compute(flat[1:].view(M, K), bias=bias)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    assert torch.equal(y.view(torch.int16), y3.view(torch.int16))


def test_route_by_rows_and_k():
    op = MatMulNBits(512, 300, bits=4, block_size=32, dtype=torch.bfloat16)
    c = make("bf16", 300, 512, 4, 32, "none", "none", 4, seed=1)
    d = {k: to_dev(v) for k, v in c.items()}
    assert op.PrePack(d["B"], d["scales"], None, None)
    assert kernel_name(op, 16) == DECODE and kernel_name(op, 17) == MID and kernel_name(op, 700) == MID
    op2 = MatMulNBits(416, 300, bits=4, block_size=32, dtype=torch.bfloat16)
    c2 = make("bf16", 300, 416, 4, 32, "none", "none", 4, seed=1)
    d2 = {k: to_dev(v) for k, v in c2.items()}
    assert op2.PrePack(d2["B"], d2["scales"], None, None)
    assert kernel_name(op2, 16) == DECODE and kernel_name(op2, 300) == MID
    big = MatMulNBits(4096, 4096, bits=4, block_size=32, dtype=torch.bfloat16)
    cb = make("bf16", 4096, 4096, 4, 32, "none", "none", 1, seed=1)
    db = {k: to_dev(v) for k, v in cb.items()}
    assert big.PrePack(db["B"], db["scales"], None, None)
    assert kernel_name(big, 64) == MID and kernel_name(big, 1024) == TILE


# ---- fp16 activations with zero points in the activation type (4- and 2-bit): the same two kernels, fp16 operands
@pytest.mark.parametrize("bits,bs,g_kind", [(4, 32, "none"), (4, 128, "none"), (4, 16, "none"), (4, 64, "act_order"),
                                            (4, 32, "ragged"), (2, 32, "none"), (2, 64, "none")])
@pytest.mark.parametrize("M", [1, 5, 16, 17, 130, 600])
def test_f16_typed_zero_points_against_float64(bits, bs, g_kind, M):
    N, K = 300, 512
    c = make("f16", N, K, bits, bs, "typed", g_kind, M, seed=M + bits + bs, bias=M % 2 == 1)
    y, op = run_op("f16", c, N, K, bits, bs)
    assert kernel_name(op, M) == (DECODE if M <= 16 else MID)
    assert y.dtype == torch.float16 and tuple(y.shape) == (M, N)
    check("f16", c, y, N, K, bits, bs)


@pytest.mark.parametrize("bits,bs", [(4, 32), (4, 16), (2, 64), (4, 128), (2, 256)])
@pytest.mark.parametrize("rows", ["decode", "mid", "tile"])
def test_f16_typed_zero_points_unit_rows_recover_w_exactly(bits, bs, rows):
    M, N, K = {"decode": (16, 200, 256), "mid": (200, 200, 256), "tile": BIG}[rows]
    c = make("f16", N, K, bits, bs, "typed", "none", M, seed=7, exact=True)
    a, ks = unit_rows(M, K, 2)
    c["A"] = to_np_type(a, "f16")
    y, op = run_op("f16", c, N, K, bits, bs)
    assert kernel_name(op, M) == {"decode": DECODE, "mid": MID, "tile": TILE}[rows]
    w = C.variant_dequantize(c["B"], c["scales"], c["zp"], None, N, K, bits, bs)
    assert np.array_equal(to_host32(y), w[:, ks].T)


@pytest.mark.parametrize("N,K,bs", [(20480, 4096, 128), (28672, 4096, 32), (28672, 4096, 256)])
@pytest.mark.parametrize("M", [1, 8, 16])
def test_f16_typed_zero_points_decode_with_more_slabs_than_compute_units(N, K, bs, M):
    c = make("f16", N, K, 4, bs, "typed", "none", M, seed=M + N, bias=True)
    y, op = run_op("f16", c, N, K, 4, bs)
    assert kernel_name(op, M) == DECODE
    check("f16", c, y, N, K, 4, bs)


def test_f16_prefill_shape_with_typed_zero_points():
    (M, N, K), bits, bs = BIG, 4, 32
    c = make("f16", N, K, bits, bs, "typed", "none", M, seed=3, bias=True)
    y, op = run_op("f16", c, N, K, bits, bs)
    assert kernel_name(op, M) == TILE
    check("f16", c, y, N, K, bits, bs)
