"""Pins for the oracle's blockwise quantiser (the producer of the MatMulNBits format; used to synthesise weights).

The compiled reference is not available, so the pins are what the mathematics fixes:
  * grids that the quantiser must reproduce exactly (closed form: scale, zero point and every q are known),
  * the error bound |w - dequant(quant(w))| <= scale / 2 inside the representable range,
  * an independent vectorised numpy statement of the published algorithm
    (onnxruntime/core/mlas/lib/q4_dq.cpp:347-386, 468-574; numpy spec in
    onnxruntime/test/python/quantization/test_quantizeblockwise_4bits.py:25-86), compared away from rounding ties,
  * exact .5 ties, whose expected integers are a closed form of the reference's roundf (tests/tie_cases.py).
"""
import numpy as np
import pytest

import tie_cases
from oracle.oracle import np_unpack_q, np_unpack_zp


def _np_quantize(W, bits, bs, symmetric):
    """Independent numpy statement: W [K, N] -> (q [N, kb*bs], scales [N, kb], zp [N, kb]) as int/float arrays."""
    K, N = W.shape
    kb = (K + bs - 1) // bs
    Wp = np.zeros((kb * bs, N), np.float32)
    Wp[:K] = W
    blk = Wp.T.reshape(N, kb, bs)
    valid = (np.arange(kb * bs) < K).reshape(kb, bs)
    maxq, mid = (1 << bits) - 1, 1 << (bits - 1)
    if symmetric:
        big = np.where(valid, blk, np.float32(0)).astype(np.float32)
        mx = np.where(valid, blk, -np.inf).max(-1).astype(np.float32)
        mn = np.where(valid, blk, np.inf).min(-1).astype(np.float32)
        s = np.where(np.abs(mx) > np.abs(mn), mx, mn)
        scale = (-s / np.float32(mid)).astype(np.float32)
        zp = np.full((N, kb), mid, np.int32)
        del big
    else:
        mx = np.maximum(np.where(valid, blk, 0).max(-1), 0).astype(np.float32)
        mn = np.minimum(np.where(valid, blk, 0).min(-1), 0).astype(np.float32)
        scale = ((mx - mn) / np.float32(maxq)).astype(np.float32)
        with np.errstate(divide="ignore", invalid="ignore"):
            zf = np.where(scale != 0, -mn / scale, mn).astype(np.float32)
        zp = np.floor(np.clip(zf, 0, maxq) + np.float32(0.5)).astype(np.int32)  # zf >= 0: half away = half up
    with np.errstate(divide="ignore"):
        r = np.where(scale != 0, np.float32(1) / scale, np.float32(0)).astype(np.float32)
    t = (blk * r[..., None]).astype(np.float32) + zp[..., None].astype(np.float32)
    t = t.astype(np.float32)
    q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), 0, maxq).astype(np.int32)
    frac = np.abs(t - np.floor(t) - 0.5)
    return q.reshape(N, kb * bs), scale, zp, (frac.reshape(N, kb * bs) < 1e-3)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("bs", [16, 32, 128])
def test_asymmetric_grid_is_reproduced_exactly(oracle, bits, bs):
    """w = (q - zp) * 2^-e with q covering 0 and 2^bits - 1: scale, zp and all q are determined."""
    rng = np.random.default_rng(bits * 100 + bs)
    N, kb, maxq = 7, 3, (1 << bits) - 1
    K = kb * bs
    q = rng.integers(0, maxq + 1, size=(N, kb, bs))
    q[:, :, 0], q[:, :, 1] = 0, maxq
    zp = rng.integers(1, maxq, size=(N, kb))
    scale = np.ldexp(1.0, -rng.integers(2, 9, size=(N, kb))).astype(np.float32)
    w = ((q - zp[..., None]) * scale[..., None]).astype(np.float32)          # exact
    Bq, s, z = oracle.C.quantize(w.reshape(N, K).T.copy(), bits, bs, symmetric=False)
    assert np.array_equal(s, scale)
    assert np.array_equal(np_unpack_zp(z, N, K, bits, bs), zp)
    assert np.array_equal(np_unpack_q(Bq, N, K, bits, bs), q.reshape(N, K))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("negative_extreme", [True, False])
def test_symmetric_grid_and_sign_convention(oracle, bits, negative_extreme):
    """The half with the larger magnitude maps to q = 0 (the reference's minus sign): scale may be negative."""
    rng = np.random.default_rng(bits + int(negative_extreme))
    N, kb, bs = 5, 4, 32
    K, mid, maxq = kb * bs, 1 << (bits - 1), (1 << bits) - 1
    q = rng.integers(1, maxq + 1, size=(N, kb, bs))
    q[:, :, 3] = 0                                                            # the extreme: (0 - mid) * scale
    mag = np.ldexp(1.0, -rng.integers(2, 7, size=(N, kb))).astype(np.float32)
    scale = mag if negative_extreme else -mag                                 # extreme value = -mid * scale
    w = ((q - mid) * scale[..., None]).astype(np.float32)
    Bq, s, z = oracle.C.quantize(w.reshape(N, K).T.copy(), bits, bs, symmetric=True)
    assert z is None
    assert np.array_equal(s, scale)
    assert np.array_equal(np_unpack_q(Bq, N, K, bits, bs), q.reshape(N, K))


@pytest.mark.parametrize("bits,bs,symmetric", [(4, 32, False), (4, 128, True), (8, 64, False), (8, 16, True)])
def test_round_trip_error_bound_and_numpy_agreement(oracle, bits, bs, symmetric):
    rng = np.random.default_rng(7)
    K, N = 200, 37                                                            # ragged last block
    W = rng.standard_normal((K, N)).astype(np.float32)
    Bq, s, z = oracle.C.quantize(W, bits, bs, symmetric)
    deq = oracle.C.dequantize(Bq, s, z, N, K, bits, bs)                        # [N, K]
    kb = (K + bs - 1) // bs
    s_full = np.repeat(s, bs, axis=1)[:, :K]
    err = np.abs(deq - W.T)
    if symmetric:
        # one half of the range has one step less: values beyond (2^(b-1) - 1) steps are clamped
        inside = np.abs(W.T / s_full + 0) <= (1 << (bits - 1)) - 1
        assert np.all(err[inside] <= np.abs(s_full[inside]) * 0.5 * (1 + 1e-5) + 1e-7)
    else:
        assert np.all(err <= np.abs(s_full) * 0.5 * (1 + 1e-4) + 1e-7)
    q_ref, s_ref, zp_ref, near_tie = _np_quantize(W, bits, bs, symmetric)
    assert np.array_equal(s, s_ref)
    if not symmetric:
        assert np.array_equal(np_unpack_zp(z, N, K, bits, bs), zp_ref)
    q = np_unpack_q(Bq, N, K, bits, bs)
    valid = np.broadcast_to(np.arange(kb * bs) < K, q.shape) & ~near_tie
    assert valid.mean() > 0.7
    assert np.array_equal(q[valid], q_ref[valid])


def test_all_zero_block_and_padding(oracle):
    W = np.zeros((40, 3), np.float32)
    W[32:, 1] = 1.0
    Bq, s, z = oracle.C.quantize(W, 4, 32, symmetric=False)
    assert s[0, 0] == 0 and np_unpack_zp(z, 3, 40, 4, 32)[0, 0] == 0
    deq = oracle.C.dequantize(Bq, s, z, 3, 40, 4, 32)
    assert np.array_equal(deq, W.T)                                           # 0 and 1 are both on the grid


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("bs", [16, 64])
@pytest.mark.parametrize("symmetric", [False, True])
def test_element_ties_round_half_away_from_zero(oracle, dtype, bits, bs, symmetric):
    """x + 0.5 -> x + 1 for every x, even ones included (roundf, q4_dq.cpp:558); rint would give x for even x."""
    W, scale, zp, want = tie_cases.element_ties(bits, bs, dtype, symmetric)
    K, N = W.shape
    Bq, s, z = oracle.C.quantize(W, bits, bs, symmetric)
    assert np.array_equal(s, scale)
    if not symmetric:
        assert np.array_equal(np_unpack_zp(z, N, K, bits, bs), zp)
    q = np_unpack_q(Bq, N, K, bits, bs)
    assert np.array_equal(q, want)
    even_ties = (want % 2 == 1) & (want < (1 << bits) - 1)
    assert even_ties.sum() > 50                       # cases where half-to-even would have returned want - 1


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_zero_point_ties_round_half_away_from_zero(oracle, dtype, bits):
    """-min / scale = z + 0.5 -> zero point z + 1 (roundf, q4_dq.cpp:367), for even and odd z."""
    W, scale, zp, want = tie_cases.zero_point_ties(bits, 32, dtype)
    K, N = W.shape
    Bq, s, z = oracle.C.quantize(W, bits, 32, symmetric=False)
    assert np.array_equal(s, scale)
    assert np.array_equal(np_unpack_zp(z, N, K, bits, 32), zp)
    assert ((zp - 1) % 2 == 0).sum() > 4              # even z among them
    assert np.array_equal(np_unpack_q(Bq, N, K, bits, 32), want)
