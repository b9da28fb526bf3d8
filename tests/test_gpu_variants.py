"""The inputs the reference serves through its dequantise-everything route (zero points in the activation type, a
group index; matmul_nbits.cc:1248-1295, matmul_nbits_impl.cc:19-75) and bfloat16 activations, through the C ABI's
variant entry points and the host class.

Gates: the device dequantiser is bit-exact against the oracle's restatement of the reference formula; the GEMM is
checked against a float64 product over that W with the operator's tolerances (fp32: |err| <= 1e-4 * sum|a*w|; fp16 and
bfloat16: relative L2 <= 5e-3), and bit-exactly on inputs where no operation rounds (unit-vector activations recover
W through the gather, the packing in group order and the kernels).  bfloat16 has no CPU kernel in the reference:
its results are pinned by the float64 product only."""
import numpy as np
import pytest
import torch

import onnxruntime_amd as ort_amd
from onnxruntime_amd import MatMulNBits, MnbError, _lib
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
C = oracle.C
TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def to_np_type(x32, kind):
    if kind == "f32":
        return np.ascontiguousarray(x32, np.float32)
    if kind == "f16":
        return np.ascontiguousarray(x32).astype(np.float16)
    return oracle.narrow_bf16(x32)


def to_dev(x):
    if x is None:
        return None
    if x.dtype == np.uint16:  # bfloat16 bits
        return torch.from_numpy(np.ascontiguousarray(x).view(np.int16)).view(torch.bfloat16).to(DEV)
    return torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def to_host32(t):
    if t.dtype == torch.bfloat16:
        return oracle.widen(t.cpu().view(torch.int16).numpy().view(np.uint16))
    return t.cpu().numpy().astype(np.float32)


def group_index(kind, K, bs, rng):
    kb = (K + bs - 1) // bs
    if kind == "none":
        return None
    if kind == "trivial":
        return (np.arange(K) // bs).astype(np.int32)
    if kind == "act_order":       # GPTQ act-order: a permutation of the trivial index, every group keeps bs members
        return (rng.permutation(kb * bs)[:K] // bs).astype(np.int32)
    return rng.integers(0, kb, size=K).astype(np.int32)   # arbitrary membership, ragged groups, maybe empty ones


def make(kind, N, K, bits, bs, zp_kind, g_kind, M, seed, exact=False, bias=False):
    rng = np.random.default_rng(seed)
    kb = (K + bs - 1) // bs
    B = rng.integers(0, 256, size=(N, kb, bs * bits // 8), dtype=np.uint8)
    if exact:
        scales = 2.0 ** rng.integers(-6, -2, size=(N, kb)).astype(np.float32)
        zt = rng.integers(0, 2 ** (bits + 1), size=(N, kb)).astype(np.float32) / 2.0
    else:
        scales = rng.uniform(0.001, 0.01, size=(N, kb)).astype(np.float32)
        zt = rng.uniform(0, 2 ** bits - 1, size=(N, kb)).astype(np.float32)
    zp = None
    if zp_kind == "u8":
        zp = rng.integers(0, 256, size=(N, (kb * bits + 7) // 8), dtype=np.uint8)
    elif zp_kind == "typed":
        zp = to_np_type(zt, kind)
    A = rng.standard_normal((M, K), dtype=np.float32)
    b = (rng.standard_normal(N, dtype=np.float32) * 0.02) if bias else None
    return dict(A=to_np_type(A, kind), B=B, scales=to_np_type(scales, kind), zp=zp,
                g=group_index(g_kind, K, bs, rng), bias=None if b is None else to_np_type(b, kind))


def run_op(kind, c, N, K, bits, bs, prepack=True):
    zp_dtype = torch.uint8 if (c["zp"] is None or c["zp"].dtype == np.uint8) else TORCH[kind]
    op = MatMulNBits(K, N, bits=bits, block_size=bs, dtype=TORCH[kind], has_zero_points=c["zp"] is not None,
                     has_bias=c["bias"] is not None, has_g_idx=c["g"] is not None, zero_points_dtype=zp_dtype)
    assert op.supported and op.variant
    d = {k: to_dev(v) for k, v in c.items()}
    if prepack:
        assert op.PrePack(d["B"], d["scales"], d["zp"], d["g"])
        y = op.Compute(d["A"], bias=d["bias"])
    else:
        y = op.Compute(d["A"], d["B"], d["scales"], d["zp"], d["bias"], g_idx=d["g"])
    torch.cuda.synchronize()
    return y, op


def check(kind, c, y, N, K, bits, bs):
    w = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, bits, bs, honour_u8_zp_with_g_idx=True)
    y64, bound = oracle.dense_matmul_f64(c["A"], w, c["bias"])
    got = to_host32(y).astype(np.float64)
    if kind == "f32":
        worst = float(np.max(np.abs(got - y64) / (bound + 1e-30)))
        assert worst <= 1e-4, worst
    else:
        rel = float(np.linalg.norm(got - y64) / max(np.linalg.norm(y64), 1e-30))
        assert rel <= 5e-3, rel


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("zp_kind", ["none", "u8", "typed"])
@pytest.mark.parametrize("g_kind", ["none", "trivial", "act_order", "ragged"])
def test_device_dequantiser_is_bit_exact(kind, zp_kind, g_kind):
    N, K, bs = 9, 200, 32
    c = make(kind, N, K, 4, bs, zp_kind, g_kind, 1, seed=len(kind) * 100 + len(zp_kind) * 10 + len(g_kind))
    w = ort_amd.dequantize_blockwise_variant(to_dev(c["B"]), to_dev(c["scales"]), to_dev(c["zp"]), to_dev(c["g"]), N, K,
                                             4, bs)
    want = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, 4, bs, honour_u8_zp_with_g_idx=True)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_device_dequantiser_never_reads_through_a_bad_group_index():
    """The group index of this entry point lives on the device: values outside [0, k_blocks) yield NaN, read nothing."""
    N, K, bs = 9, 200, 32
    c = make("f32", N, K, 4, bs, "typed", "ragged", 1, seed=3)
    want = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, 4, bs)
    g = c["g"].copy()
    g[[7, 150]] = [1 << 30, -5]
    w = ort_amd.dequantize_blockwise_variant(to_dev(c["B"]), to_dev(c["scales"]), to_dev(c["zp"]), to_dev(g), N, K, 4,
                                             bs).cpu().numpy()
    bad = np.zeros(K, bool)
    bad[[7, 150]] = True
    assert np.isnan(w[:, bad]).all()
    assert np.array_equal(w[:, ~bad].view(np.uint32), want[:, ~bad].view(np.uint32))


@pytest.mark.parametrize("kind", ["f32", "f16"])
def test_device_dequantiser_two_bits_typed(kind):
    N, K, bs = 5, 100, 16
    c = make(kind, N, K, 2, bs, "typed", "none", 1, seed=4)
    w = ort_amd.dequantize_blockwise_variant(to_dev(c["B"]), to_dev(c["scales"]), to_dev(c["zp"]), None, N, K, 2, bs)
    want = C.variant_dequantize(c["B"], c["scales"], c["zp"], None, N, K, 2, bs)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), want.view(np.uint32))


# every combination that is a variant: a group index, typed zero points or bfloat16
CASES = [(k, z, g) for k in ("f32", "f16", "bf16") for z in ("none", "u8", "typed")
         for g in ("none", "trivial", "act_order", "ragged") if k == "bf16" or z == "typed" or g != "none"]


@pytest.mark.parametrize("kind,zp_kind,g_kind", CASES)
@pytest.mark.parametrize("M", [1, 5, 40, 300])
def test_gemm_against_float64(kind, zp_kind, g_kind, M):
    N, K, bs = 200, 416, 32
    c = make(kind, N, K, 4, bs, zp_kind, g_kind, M, seed=M + len(zp_kind) * 7 + len(g_kind), bias=M % 2 == 1)
    y, op = run_op(kind, c, N, K, 4, bs)
    assert y.dtype == TORCH[kind] and tuple(y.shape) == (M, N)
    if g_kind in ("none", "trivial"):
        assert not op.plan.has_g_idx
    elif g_kind == "act_order":   # every group keeps block_size members: the packed matrix keeps the block size
        assert op.plan.has_g_idx and op.plan.packed_block_size == bs and op.plan.packed_k == K
    else:
        assert op.plan.has_g_idx and op.plan.packed_block_size == 16
    check(kind, c, y, N, K, 4, bs)


@pytest.mark.parametrize("kind", ["f32", "f16"])
@pytest.mark.parametrize("bs", [16, 64])
def test_two_bit_typed_zero_points(kind, bs):
    N, K = 72, 320
    for M in (1, 33):
        c = make(kind, N, K, 2, bs, "typed", "none", M, seed=bs + M, bias=True)
        y, _ = run_op(kind, c, N, K, 2, bs)
        check(kind, c, y, N, K, 2, bs)


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("zp_kind,g_kind", [("typed", "none"), ("typed", "ragged"), ("u8", "act_order"),
                                            ("none", "ragged")])
def test_unit_vectors_recover_w_exactly(kind, zp_kind, g_kind):
    """Power-of-two scales and half-integer zero points: neither formula rounds, so row k of the product of the
    identity with W must be column k of the reference's W, bit for bit, through gather, packing and kernels."""
    N, K, bs = 40, 96, 32
    c = make(kind, N, K, 4, bs, zp_kind, g_kind, K, seed=11, exact=True)
    c["A"] = to_np_type(np.eye(K, dtype=np.float32), kind)
    y, _ = run_op(kind, c, N, K, 4, bs)
    w = C.variant_dequantize(c["B"], c["scales"], c["zp"], c["g"], N, K, 4, bs)
    assert np.array_equal(to_host32(y), w.T)


@pytest.mark.parametrize("kind,zp_kind,g_kind", [("f16", "typed", "none"), ("f16", "u8", "act_order"),
                                                 ("bf16", "none", "none"), ("f32", "typed", "ragged")])
def test_operands_fed_per_run_match_prepacked(kind, zp_kind, g_kind):
    N, K, bs = 100, 256, 64
    c = make(kind, N, K, 4, bs, zp_kind, g_kind, 6, seed=2, bias=True)
    y1, _ = run_op(kind, c, N, K, 4, bs, prepack=True)
    y2, _ = run_op(kind, c, N, K, 4, bs, prepack=False)
    assert torch.equal(y1.view(torch.int16 if kind != "f32" else torch.int32),
                       y2.view(torch.int16 if kind != "f32" else torch.int32))


def test_batched_activations_strides_and_empty_output():
    N, K, bs = 64, 128, 32
    c = make("f16", N, K, 4, bs, "typed", "act_order", 6, seed=8)
    y, op = run_op("f16", c, N, K, 4, bs)
    a3 = to_dev(c["A"]).reshape(2, 3, K)
    y3 = op.Compute(a3)
    assert tuple(y3.shape) == (2, 3, N) and torch.equal(y3.reshape(6, N), y)
    wide = torch.zeros(6, K + 24, dtype=torch.float16, device=DEV)
    wide[:, :K] = to_dev(c["A"])
    assert torch.equal(op.Compute(wide[:, :K]), y)          # row pitch larger than K
    assert tuple(op.Compute(torch.zeros(0, K, dtype=torch.float16, device=DEV)).shape) == (0, N)


def test_errors():
    N, K, bs = 16, 64, 32
    c = make("f32", N, K, 4, bs, "none", "ragged", 2, seed=1)
    c["g"][5] = 2                                            # k_blocks = 2: valid indices are 0 and 1
    with pytest.raises(MnbError, match=r"group_index value at index 5 is 2, which is out of valid range \[0, 2\)") as e:
        run_op("f32", c, N, K, 4, bs)
    assert e.value.code == _lib.INVALID_ARGUMENT
    op = MatMulNBits(K, N, bits=8, block_size=bs, dtype=torch.float16, has_zero_points=True,
                     zero_points_dtype=torch.float16)
    assert not op.supported                                  # the reference rejects 8-bit typed zero points too
    op = MatMulNBits(K, N, bits=4, block_size=bs, dtype=torch.float16, has_g_idx=True)
    d = {k: to_dev(v) for k, v in make("f16", N, K, 4, bs, "none", "ragged", 2, seed=1).items()}
    with pytest.raises(MnbError, match="group_index"):
        op.PrePack(d["B"], d["scales"], None, d["g"][:-1])
