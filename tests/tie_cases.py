"""Weights whose quantisation lands exactly half way between two integers, with the expected integers in closed form.

The reference rounds with roundf, half away from zero (onnxruntime/core/mlas/lib/q4_dq.cpp:367 for the zero point,
:558 for the elements).  Every value v / scale + zp the quantiser can see is >= 0 (the block minimum maps to 0 or
above), so away from zero means up: x + 0.5 -> x + 1.  A quantiser that rounded half to even (rint, the default of
numpy.round and of a plain float -> int conversion on the GPU) would return x for even x and fail these cases.

All weights are small multiples of a power of two: exact in fp32 and fp16, and scale, its reciprocal, v / scale and
the sum with the zero point are computed without rounding, whatever the order of operations.
"""
import numpy as np


def element_ties(bits, bs, dtype, symmetric, seed=0):
    """Returns (W [K, N], scales [N, kb], zp [N, kb] or None, q [N, K]): the block holds both ends of the grid, which
    fix scale and zero point, and otherwise elements (x + 0.5 - zp) * scale whose expected integer is x + 1."""
    rng = np.random.default_rng(seed + bits * 1000 + bs)
    N, kb = 24, 3
    maxq, mid = (1 << bits) - 1, 1 << (bits - 1)
    scale = np.ldexp(1.0, -rng.integers(2, 7, size=(N, kb)))
    if symmetric:
        zp = np.full((N, kb), mid)
        negative_extreme = rng.integers(0, 2, size=(N, kb)).astype(bool)
    else:
        zp = rng.integers(1, maxq, size=(N, kb))
    # t = x + 0.5; symmetric blocks also hold x = maxq (stays inside the range, clamps to maxq)
    nx = maxq + 1 if symmetric else maxq
    x = rng.integers(0, nx, size=(N, kb, bs))
    x[:, :, 2] = np.arange(N * kb).reshape(N, kb) % nx                # every x occurs, the even ones in particular
    t = x + 0.5
    want = np.minimum(x + 1, maxq)
    t[:, :, 0], want[:, :, 0] = 0, 0                                  # q = 0: the block minimum
    if not symmetric:
        t[:, :, 1], want[:, :, 1] = maxq, maxq                        # q = maxq: the block maximum
    w = (t - zp[..., None]) * scale[..., None]
    if symmetric:
        # the extreme (q = 0) may be the largest or the smallest value of the block: mirrored blocks have scale < 0
        sign = np.where(negative_extreme, 1.0, -1.0)
        w = w * sign[..., None]
        scale = scale * sign
    W = np.ascontiguousarray(w.reshape(N, kb * bs).T).astype(dtype)
    assert np.array_equal(W.astype(np.float64), w.reshape(N, kb * bs).T)  # exact in dtype
    return W, scale.astype(dtype), (None if symmetric else zp), want.reshape(N, kb * bs)


def zero_point_ties(bits, bs, dtype, seed=0):
    """Asymmetric blocks whose -min / scale is exactly z + 0.5: expected zero point z + 1 (not z for even z), and with
    that zero point every element on the half grid is a tie again: (j - z - 0.5) * scale -> j + 0.5 -> j + 1."""
    rng = np.random.default_rng(seed + bits * 77 + bs)
    N, kb = 16, 2
    maxq = (1 << bits) - 1
    scale = np.ldexp(1.0, -rng.integers(2, 7, size=(N, kb)))
    z = (np.arange(N * kb).reshape(N, kb) * 2 + rng.integers(0, 2, size=(N, kb))) % (maxq - 1)   # 0 .. maxq - 2
    j = rng.integers(0, maxq + 1, size=(N, kb, bs))
    j[:, :, 0], j[:, :, 1] = 0, maxq                                   # min = -(z + .5) s, max = (maxq - z - .5) s
    w = (j - z[..., None] - 0.5) * scale[..., None]
    want = np.minimum(j + 1, maxq)
    W = np.ascontiguousarray(w.reshape(N, kb * bs).T).astype(dtype)
    assert np.array_equal(W.astype(np.float64), w.reshape(N, kb * bs).T)
    return W, scale.astype(dtype), z + 1, want.reshape(N, kb * bs)
