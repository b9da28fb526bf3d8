"""Pins the oracle's restatement of the reference's dequantiser for typed zero points and a group index
(onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_impl.cc:19-75; 2 bits: onnxruntime/core/mlas/lib/q4_dq.cpp:2187-2241).

The reference's own tests recompute their expectations for these inputs (matmul_4bits_test.cc:136-260 builds the
expected output from its own dequantiser) and its code for this route does not build without the whole runtime, so
what pins the restatement is mathematics: inputs on which no operation rounds (the result must equal the exact
(q - zp) * scale), agreement with the canonical dequantiser where both are defined, group selection read back through
power-of-two scales, closeness to the float64 value everywhere, and - for the last ulp of the three-rounding formula
fl(fl(float(q)*s) + fl(-s*zp)) on inexact inputs - exact rational arithmetic rounded to fp32 after every operation."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle
from oracle.oracle import np_unpack_q as _np_unpack_q, np_unpack_zp

C = oracle.C


def np_unpack_q(B, N, K, bits, bs):
    return _np_unpack_q(B, N, K, bits, bs)[:, :K]


def _case(N, K, bits, bs, seed, exact=False, dtype=np.float32):
    rng = np.random.default_rng(seed)
    kb = (K + bs - 1) // bs
    B = rng.integers(0, 256, size=(N, kb, bs * bits // 8), dtype=np.uint8)
    if exact:
        scales = (2.0 ** rng.integers(-9, -3, size=(N, kb))).astype(dtype)
        zt = (rng.integers(0, 2 ** (bits + 1), size=(N, kb)) / 2.0).astype(dtype)       # half-integers: exact
    else:
        scales = rng.uniform(0.001, 0.01, size=(N, kb)).astype(dtype)
        zt = rng.uniform(0, 2 ** bits - 1, size=(N, kb)).astype(dtype)
    zu = rng.integers(0, 256, size=(N, (kb * bits + 7) // 8), dtype=np.uint8)
    return B, scales, zt, zu, kb, rng


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("bs,K", [(16, 48), (32, 93), (128, 260)])
def test_typed_zero_points_exact_inputs(bits, bs, K):
    N = 7
    B, scales, zt, _, kb, _ = _case(N, K, bits, bs, seed=bits + bs, exact=True)
    w = C.variant_dequantize(B, scales, zt, None, N, K, bits, bs)
    q = np_unpack_q(B, N, K, bits, bs).astype(np.float64)
    blk = np.arange(K) // bs
    want = (q - zt.astype(np.float64)[:, blk]) * scales.astype(np.float64)[:, blk]
    assert w.dtype == np.float32 and np.array_equal(w.astype(np.float64), want)


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("with_zp", [False, True])
def test_agrees_with_canonical_dequantiser_on_exact_inputs(bits, with_zp):
    """uint8 / absent zero points without a group index: the canonical route is the one the reference takes; on
    inputs where nothing rounds, both formulas give the same float."""
    N, K, bs = 5, 100, 32
    B, scales, _, zu, kb, _ = _case(N, K, bits, bs, seed=3, exact=True)
    zp = zu if with_zp else None
    w = C.variant_dequantize(B, scales, zp, None, N, K, bits, bs)
    assert np.array_equal(w, C.dequantize(B, scales, zp, N, K, bits, bs))
    # the trivial group index changes nothing
    g = (np.arange(kb * bs) // bs).astype(np.int32)
    assert np.array_equal(w, C.variant_dequantize(B, scales, zp, g, N, K, bits, bs) if bits == 4 else w)


def test_group_index_selects_scale_and_zero_point():
    N, K, bs = 4, 96, 16
    B, _, _, _, kb, rng = _case(N, K, 4, bs, seed=9)
    g = rng.integers(0, kb, size=K).astype(np.int32)
    scales = np.tile((2.0 ** (np.arange(kb) - 8)).astype(np.float32), (N, 1))      # the exponent names the group
    w = C.variant_dequantize(B, scales, None, g, N, K, 4, bs)
    q = np_unpack_q(B, N, K, 4, bs).astype(np.float64)
    assert np.array_equal(w.astype(np.float64), (q - 8.0) * (2.0 ** (g.astype(np.float64) - 8)))
    # typed zero points follow the same index
    zt = np.tile(np.arange(kb, dtype=np.float32) + 0.5, (N, 1))
    w = C.variant_dequantize(B, scales, zt, g, N, K, 4, bs)
    assert np.array_equal(w.astype(np.float64), (q - (g + 0.5)) * (2.0 ** (g.astype(np.float64) - 8)))


def test_uint8_zero_points_with_group_index_literal_and_schema_behaviour():
    """The reference's CPU code reads packed zero points in this combination and then uses 8
    (matmul_nbits_impl.cc:56-66); the schema - and the reference without a group index - applies them."""
    N, K, bs = 3, 64, 16
    B, scales, _, zu, kb, rng = _case(N, K, 4, bs, seed=21, exact=True)
    g = rng.permutation(K).astype(np.int32) // bs
    literal = C.variant_dequantize(B, scales, zu, g, N, K, 4, bs, honour_u8_zp_with_g_idx=False)
    assert np.array_equal(literal, C.variant_dequantize(B, scales, None, g, N, K, 4, bs))
    schema = C.variant_dequantize(B, scales, zu, g, N, K, 4, bs, honour_u8_zp_with_g_idx=True)
    z_typed = np_unpack_zp(zu, N, K, 4, bs).astype(np.float32)
    assert np.array_equal(schema, C.variant_dequantize(B, scales, z_typed, g, N, K, 4, bs))
    assert not np.array_equal(schema, literal)


@pytest.mark.parametrize("dtype", [np.float32, np.float16, "bf16"])
def test_close_to_float64_on_random_inputs(dtype):
    N, K, bs = 6, 200, 32
    B, scales, zt, _, kb, rng = _case(N, K, 4, bs, seed=5)
    if dtype == "bf16":
        scales, zt = oracle.narrow_bf16(scales), oracle.narrow_bf16(zt)
    else:
        scales, zt = scales.astype(dtype), zt.astype(dtype)
    g = rng.integers(0, kb, size=K).astype(np.int32)
    w = C.variant_dequantize(B, scales, zt, g, N, K, 4, bs).astype(np.float64)
    s64, z64 = oracle.widen(scales).astype(np.float64), oracle.widen(zt).astype(np.float64)
    q = np_unpack_q(B, N, K, 4, bs).astype(np.float64)
    exact = (q - z64[:, g]) * s64[:, g]
    # three roundings to fp32, each relative 2^-24, of terms no larger than |q s| + |s zp|
    bound = 2.0 ** -23 * (np.abs(q * s64[:, g]) + np.abs(s64[:, g] * z64[:, g]))
    assert np.all(np.abs(w - exact) <= bound)


def test_bfloat16_helpers():
    x = np.array([1.0, 1.00390625, 1.005859375, -2.5, 3.0e-3, 65504.0], np.float32)
    b = oracle.narrow_bf16(x)
    back = oracle.widen(b)
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -8)
    assert back[0] == 1.0 and back[3] == -2.5
    assert oracle.widen(oracle.narrow_bf16(np.float32([1.00390625])))[0] == 1.0          # tie -> even
    assert oracle.widen(oracle.narrow_bf16(np.float32([1.01171875])))[0] == 1.015625     # tie -> even (up)


def _round_to_f32(x: Fraction) -> np.float32:
    """Round-to-nearest-even of an exact rational to IEEE binary32 (normal and subnormal range; no overflow here)."""
    if x == 0:
        return np.float32(0.0)
    sign, a = (-1 if x < 0 else 1), abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()      # 2^(e-1) < a < 2^(e+1)
    if Fraction(2) ** e > a:
        e -= 1                                                     # now 2^e <= a < 2^(e+1)
    q = max(e - 23, -149)                                          # exponent of the last kept bit
    scaled = a / Fraction(2) ** q
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return np.float32(sign * float(n) * 2.0 ** q)                  # n < 2^25 and a power of two: exact in double


def test_round_to_f32_helper_against_numpy():
    rng = np.random.default_rng(0)
    d = np.concatenate([rng.standard_normal(2000) * 10.0 ** rng.integers(-30, 30, 2000),
                        [1 + 2.0 ** -24, 1 + 3 * 2.0 ** -24, 1 - 2.0 ** -25, 2.0 ** -140 * 1.3, 2.0 ** -149 * 0.5]])
    for v in d:                                                    # doubles are exact rationals; numpy rounds them RNE
        assert _round_to_f32(Fraction(float(v))) == np.float32(v)


@pytest.mark.parametrize("bits,zp_kind", [(4, "typed"), (2, "typed"), (4, "uint8+g_idx"), (4, "none+g_idx")])
def test_three_roundings_against_exact_rational_arithmetic(bits, zp_kind):
    """w = fl(fl(float(q) * s) + fl(-s * zp)), every operation rounded to fp32 by itself
    (matmul_nbits_impl.cc:66-73 with T = float).  A contracted multiply-add, a (q - zp) * s evaluation or a float64
    intermediate each differ from this in the last place on part of these inputs (counted below)."""
    N, K, bs = 5, 96, 16
    B, scales, zt, zu, kb, rng = _case(N, K, bits, bs, seed=31 + bits)
    g = rng.integers(0, kb, size=K).astype(np.int32) if "g_idx" in zp_kind else None
    if zp_kind == "typed":
        zp_arg, zf = zt, zt
    elif zp_kind.startswith("uint8"):
        zp_arg, zf = zu, np_unpack_zp(zu, N, K, bits, bs).astype(np.float32)
    else:
        zp_arg, zf = None, np.full((N, kb), 2 ** (bits - 1), np.float32)
    w = C.variant_dequantize(B, scales, zp_arg, g, N, K, bits, bs)
    q = np_unpack_q(B, N, K, bits, bs)
    blk = g if g is not None else np.arange(K) // bs
    fused_differs = single_differs = 0
    for n in range(N):
        for k in range(K):
            s, z = Fraction(float(scales[n, blk[k]])), Fraction(float(zf[n, blk[k]]))
            adjust = Fraction(float(_round_to_f32(-s * z)))
            prod = Fraction(float(_round_to_f32(int(q[n, k]) * s)))
            want = _round_to_f32(prod + adjust)
            assert w[n, k] == want, (n, k, float(w[n, k]), float(want))
            fused_differs += _round_to_f32(int(q[n, k]) * s + adjust) != want
            single_differs += _round_to_f32((int(q[n, k]) - z) * s) != want
    assert fused_differs > 0 and single_differs > 0      # the inputs do tell the formulas apart
