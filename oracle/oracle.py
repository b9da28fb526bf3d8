"""TEST INFRASTRUCTURE ONLY -- Python face of the CPU oracle for MatMulNBits.

Two independent restatements of the reference's arithmetic contract live here:

* ``C``: ctypes bindings of ``libmnb_oracle.so`` (``mnb_oracle.c``), used for full-size checks and as the
  ``cpu_baseline`` of ``bench.py``;
* ``np_*``: a vectorised numpy restatement written separately from the C code, so that the two can be
  checked against each other and against the reference's own test vectors.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module.
The product (``onnxruntime_amd``) never does.

Parity status of what is defined here on top of the C functions (whose own status is in the header of mnb_oracle.c):
  ``mlp`` / ``qkv``           compositions of pinned parts (matmul, layer normalisation) with silu(g) * u in float64;
                              the reference ships only WebGPU shaders for these operators and no stored outputs, so
                              beyond that composition their parity is PARITY UNPINNED
  ``variant_dequantize``      wrapper of mnbo_variant_dequantize_f32: pinned by mathematics, the last place of its
                              three roundings included (exact rational arithmetic, tests/test_oracle_variants.py);
                              bfloat16 operands have no CPU kernel in the reference at all: PARITY UNPINNED
  ``dense_matmul_f64``        numpy float64 product over a dequantised W, the checker of the variant route

Reference definitions followed (onnxruntime 1.30.0):
  canonical layout + ``(q - zp) * scale``      onnxruntime/core/mlas/lib/q4_dq.cpp:587-641
  operator contract (shapes, optional inputs)   onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3782-3849
  zero-point packing                            onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_helper.h:33-35
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libmnb_oracle.so"


def build(force: bool = False) -> Path:
    """Compile the C oracle (gcc, a second or two)."""
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "mnb_oracle.c").stat().st_mtime:
        subprocess.check_call(["make", "-C", str(_HERE), "-B" if force else "-s", "libmnb_oracle.so"])
    return _LIB_PATH


_u8p = ctypes.POINTER(ctypes.c_uint8)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i64 = ctypes.c_int64
_int = ctypes.c_int


def _ptr(a, typ):
    if a is None:
        return ctypes.cast(None, typ)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(typ)


class _C:
    """Lazy ctypes handle of the C oracle."""

    def __init__(self):
        self._lib = None

    @property
    def lib(self):
        if self._lib is None:
            if not _LIB_PATH.exists():
                build()
            lib = ctypes.CDLL(str(_LIB_PATH))
            lib.mnbo_f16_to_f32.restype = ctypes.c_float
            lib.mnbo_f16_to_f32.argtypes = [ctypes.c_uint16]
            lib.mnbo_f32_to_f16.restype = ctypes.c_uint16
            lib.mnbo_f32_to_f16.argtypes = [ctypes.c_float]
            lib.mnbo_f16_to_f32_buffer.argtypes = [_u16p, _f32p, ctypes.c_size_t]
            lib.mnbo_f32_to_f16_buffer.argtypes = [_f32p, _u16p, ctypes.c_size_t]
            lib.mnbo_dequantize_f32.argtypes = [_f32p, _u8p, _f32p, _u8p, _i64, _i64, _int, _i64]
            lib.mnbo_dequantize_f16.argtypes = [_u16p, _u8p, _u16p, _u8p, _i64, _i64, _int, _i64]
            lib.mnbo_matmul_f32.argtypes = [_f32p, _u8p, _f32p, _u8p, _f32p, _f32p, _i64, _i64, _i64, _int, _i64, _int]
            lib.mnbo_matmul_f64.argtypes = [_f32p, _u8p, _f32p, _u8p, _f32p, _f64p, _f64p, _i64, _i64, _i64, _int,
                                            _i64, _int]
            lib.mnbo_matmul_f16.argtypes = [_u16p, _u8p, _u16p, _u8p, _u16p, _u16p, _i64, _i64, _i64, _int, _i64, _int]
            lib.mnbo_quantize_f32.argtypes = [_u8p, _f32p, _u8p, _f32p, _i64, _i64, _int, _i64, _int]
            lib.mnbo_quantize_f16.argtypes = [_u8p, _u16p, _u8p, _u16p, _i64, _i64, _int, _i64, _int]
            lib.mnbo_quantize_f16.restype = None
            lib.mnbo_variant_dequantize_f32.argtypes = [_f32p, _u8p, _f32p, _int, ctypes.c_void_p,
                                                        ctypes.POINTER(ctypes.c_int32), _i64, _i64, _int, _i64, _int]
            lib.mnbo_variant_dequantize_f32.restype = None
            lib.mnbo_skip_simplified_layer_norm_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _i64, _f32p, _f32p,
                                                                ctypes.c_float, _i64, _i64]
            lib.mnbo_skip_simplified_layer_norm_f32.restype = None
            lib.mnbo_skip_simplified_layer_norm_f16.argtypes = [_u16p, _u16p, _u16p, _u16p, _i64, _u16p, _u16p,
                                                                ctypes.c_float, _i64, _i64]
            lib.mnbo_skip_simplified_layer_norm_f16.restype = None
            _i8p = ctypes.POINTER(ctypes.c_int8)
            lib.mnbo_quantize_a_int8.argtypes = [_i8p, _f32p, _f32p, _i64, _i64, _i64]
            lib.mnbo_quantize_a_int8.restype = None
            lib.mnbo_matmul_int8_f32.argtypes = [_f32p, _u8p, _f32p, _u8p, _f32p, _f32p, _i64, _i64, _i64, _i64, _int]
            lib.mnbo_matmul_int8_f32.restype = None
            lib.mnbo_matmul_int8_f16.argtypes = [_u16p, _u8p, _u16p, _u8p, _u16p, _u16p, _i64, _i64, _i64, _i64, _int]
            lib.mnbo_matmul_int8_f16.restype = None
            for f in (lib.mnbo_f16_to_f32_buffer, lib.mnbo_f32_to_f16_buffer, lib.mnbo_dequantize_f32,
                      lib.mnbo_dequantize_f16, lib.mnbo_matmul_f32, lib.mnbo_matmul_f64, lib.mnbo_matmul_f16,
                      lib.mnbo_quantize_f32):
                f.restype = None
            self._lib = lib
        return self._lib

    # -- fp16 -----------------------------------------------------------------
    def f16_to_f32(self, h: np.ndarray) -> np.ndarray:
        h = np.ascontiguousarray(h).view(np.uint16)
        out = np.empty(h.shape, np.float32)
        self.lib.mnbo_f16_to_f32_buffer(_ptr(h, _u16p), _ptr(out, _f32p), h.size)
        return out

    def f32_to_f16(self, f: np.ndarray) -> np.ndarray:
        f = np.ascontiguousarray(f, np.float32)
        out = np.empty(f.shape, np.uint16)
        self.lib.mnbo_f32_to_f16_buffer(_ptr(f, _f32p), _ptr(out, _u16p), f.size)
        return out.view(np.float16)

    # -- dequantise -----------------------------------------------------------
    def dequantize(self, B, scales, zp, N, K, bits, bs) -> np.ndarray:
        """Returns W as [N, K] in the dtype of ``scales`` (the reference's column-major output)."""
        B = np.ascontiguousarray(B, np.uint8)
        zp = None if zp is None else np.ascontiguousarray(zp, np.uint8)
        if scales.dtype == np.float16:
            s = np.ascontiguousarray(scales).view(np.uint16)
            out = np.empty((N, K), np.uint16)
            self.lib.mnbo_dequantize_f16(_ptr(out, _u16p), _ptr(B, _u8p), _ptr(s, _u16p), _ptr(zp, _u8p), N, K, bits,
                                         bs)
            return out.view(np.float16)
        s = np.ascontiguousarray(scales, np.float32)
        out = np.empty((N, K), np.float32)
        self.lib.mnbo_dequantize_f32(_ptr(out, _f32p), _ptr(B, _u8p), _ptr(s, _f32p), _ptr(zp, _u8p), N, K, bits, bs)
        return out

    def variant_dequantize(self, B, scales, zp, g_idx, N, K, bits, bs, honour_u8_zp_with_g_idx=True) -> np.ndarray:
        """The reference's dequantiser for typed zero points and / or a group index: W as float32 [N, K].

        ``scales`` float32, float16 or bfloat16-as-uint16 (see ``widen``); ``zp`` None, uint8 (packed) or an array of
        the scales' type (typed, [N, k_blocks])."""
        B = np.ascontiguousarray(B, np.uint8)
        s = np.ascontiguousarray(widen(scales), np.float32)
        if zp is None:
            kind, z = 0, None
        elif zp.dtype == np.uint8 and scales.dtype != np.uint8:
            kind, z = 1, np.ascontiguousarray(zp)
        else:
            kind, z = 2, np.ascontiguousarray(widen(zp), np.float32)
        g = None if g_idx is None else np.ascontiguousarray(g_idx, np.int32)
        out = np.empty((N, K), np.float32)
        self.lib.mnbo_variant_dequantize_f32(_ptr(out, _f32p), _ptr(B, _u8p), _ptr(s, _f32p), kind,
                                             None if z is None else z.ctypes.data,
                                             _ptr(g, ctypes.POINTER(ctypes.c_int32)), N, K, bits, bs,
                                             int(bool(honour_u8_zp_with_g_idx)))
        return out

    # -- matmul ---------------------------------------------------------------
    def matmul(self, A, B, scales, zp, bias, N, K, bits, bs, nthreads=1) -> np.ndarray:
        """Y = A x dequant(B)^T (+ bias) with the reference's CPU semantics for the dtype of A."""
        lead = A.shape[:-1]
        M = int(np.prod(lead)) if lead else 1
        B = np.ascontiguousarray(B, np.uint8)
        zp = None if zp is None else np.ascontiguousarray(zp, np.uint8)
        if A.dtype == np.float16:
            a = np.ascontiguousarray(A).view(np.uint16)
            s = np.ascontiguousarray(scales, np.float16).view(np.uint16)
            b = None if bias is None else np.ascontiguousarray(bias, np.float16).view(np.uint16)
            y = np.empty((M, N), np.uint16)
            self.lib.mnbo_matmul_f16(_ptr(a, _u16p), _ptr(B, _u8p), _ptr(s, _u16p), _ptr(zp, _u8p), _ptr(b, _u16p),
                                     _ptr(y, _u16p), M, N, K, bits, bs, nthreads)
            return y.view(np.float16).reshape(*lead, N)
        a = np.ascontiguousarray(A, np.float32)
        s = np.ascontiguousarray(scales, np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        y = np.empty((M, N), np.float32)
        self.lib.mnbo_matmul_f32(_ptr(a, _f32p), _ptr(B, _u8p), _ptr(s, _f32p), _ptr(zp, _u8p), _ptr(b, _f32p),
                                 _ptr(y, _f32p), M, N, K, bits, bs, nthreads)
        return y.reshape(*lead, N)

    # -- int8 activations (accuracy_level 4) ----------------------------------
    def quantize_a_int8(self, A, bs):
        """Blockwise int8 quantisation of the activations: returns (qa [M, k_blocks*bs] int8, scales [M, k_blocks])."""
        a = np.ascontiguousarray(A.astype(np.float32))
        M, K = a.shape
        kb = -(-K // bs)
        qa = np.empty((M, kb * bs), np.int8)
        sc = np.empty((M, kb), np.float32)
        self.lib.mnbo_quantize_a_int8(_ptr(qa, ctypes.POINTER(ctypes.c_int8)), _ptr(sc, _f32p), _ptr(a, _f32p), M, K, bs)
        return qa, sc

    def matmul_int8(self, A, B, scales, zp, bias, N, K, bs, nthreads=1) -> np.ndarray:
        """Y = A x dequant(B)^T (+ bias) with A quantised blockwise to int8 first (4-bit weights), in the dtype of A."""
        lead = A.shape[:-1]
        M = int(np.prod(lead)) if lead else 1
        B = np.ascontiguousarray(B, np.uint8)
        zp = None if zp is None else np.ascontiguousarray(zp, np.uint8)
        if A.dtype == np.float16:
            a = np.ascontiguousarray(A).view(np.uint16)
            s = np.ascontiguousarray(scales, np.float16).view(np.uint16)
            b = None if bias is None else np.ascontiguousarray(bias, np.float16).view(np.uint16)
            y = np.empty((M, N), np.uint16)
            self.lib.mnbo_matmul_int8_f16(_ptr(a, _u16p), _ptr(B, _u8p), _ptr(s, _u16p), _ptr(zp, _u8p),
                                          _ptr(b, _u16p), _ptr(y, _u16p), M, N, K, bs, nthreads)
            return y.view(np.float16).reshape(*lead, N)
        a = np.ascontiguousarray(A, np.float32)
        s = np.ascontiguousarray(scales, np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        y = np.empty((M, N), np.float32)
        self.lib.mnbo_matmul_int8_f32(_ptr(a, _f32p), _ptr(B, _u8p), _ptr(s, _f32p), _ptr(zp, _u8p), _ptr(b, _f32p),
                                      _ptr(y, _f32p), M, N, K, bs, nthreads)
        return y.reshape(*lead, N)

    def matmul_f64(self, A, B, scales, zp, bias, N, K, bits, bs, nthreads=1):
        """fp64 accumulation of the fp32 products and the row bound sum_k |a*w| (+|bias|).

        fp16 inputs are widened exactly first, as the reference does."""
        lead = A.shape[:-1]
        M = int(np.prod(lead)) if lead else 1
        a = np.ascontiguousarray(A.astype(np.float32))
        s = np.ascontiguousarray(scales.astype(np.float32))
        b = None if bias is None else np.ascontiguousarray(bias.astype(np.float32))
        B = np.ascontiguousarray(B, np.uint8)
        zp = None if zp is None else np.ascontiguousarray(zp, np.uint8)
        y = np.empty((M, N), np.float64)
        bound = np.empty((M, N), np.float64)
        self.lib.mnbo_matmul_f64(_ptr(a, _f32p), _ptr(B, _u8p), _ptr(s, _f32p), _ptr(zp, _u8p), _ptr(b, _f32p),
                                 _ptr(y, _f64p), _ptr(bound, _f64p), M, N, K, bits, bs, nthreads)
        return y.reshape(*lead, N), bound.reshape(*lead, N)

    # -- fused projections ----------------------------------------------------
    def simplified_layer_norm(self, A, skip, gamma, epsilon, bias=None, want_sum=False):
        """(Skip)SimplifiedLayerNormalization over the last axis in the dtype of ``A`` (fp16 or fp32).

        ``skip`` may have fewer leading rows than ``A`` (row m uses skip row m % rows).  Returns out, or
        (out, input + skip [+ bias]) when ``want_sum``."""
        K = A.shape[-1]
        M = A.size // K
        f16 = A.dtype == np.float16
        ptr_t, np_t = (_u16p, np.uint16) if f16 else (_f32p, np.float32)

        def arr(x):
            if x is None:
                return None
            x = np.ascontiguousarray(x, np.float16 if f16 else np.float32)
            return x.view(np_t) if f16 else x

        a, sk, g, b = arr(A), arr(skip), arr(gamma), arr(bias)
        srows = 0 if sk is None else sk.size // K
        out = np.empty((M, K), np_t)
        sm = np.empty((M, K), np_t) if want_sum else None
        fn = self.lib.mnbo_skip_simplified_layer_norm_f16 if f16 else self.lib.mnbo_skip_simplified_layer_norm_f32
        fn(_ptr(out, ptr_t), _ptr(sm, ptr_t), _ptr(a, ptr_t), _ptr(sk, ptr_t), srows, _ptr(g, ptr_t), _ptr(b, ptr_t),
           float(epsilon), M, K)
        view = (lambda x: x.view(np.float16).reshape(A.shape)) if f16 else (lambda x: x.reshape(A.shape))
        return (view(out), view(sm)) if want_sum else view(out)

    def projections_f32(self, A, mats, N_each, K, bits, bs, nthreads=1):
        """fp32 result (before the narrowing of an fp16 model) of A x dequant(B_i)^T + bias_i for every
        (B, scales, bias) in ``mats``: operands widened exactly, fp32 accumulation in k order."""
        outs = []
        a32 = np.ascontiguousarray(A.astype(np.float32))
        for (B, scales, bias), N in zip(mats, N_each):
            b32 = None if bias is None else bias.astype(np.float32)
            outs.append(self.matmul(a32, B, scales.astype(np.float32), None, b32, N, K, bits, bs, nthreads))
        return outs

    def mlp(self, A, gate, up, N, K, bits, bs, norm=None, nthreads=1):
        """com.microsoft::MatMulNBitsMlp (contrib_defs.cc:3851-3975): Y = silu(gate(A')) * up(A'), A' = A or its
        (skip) simplified layer normalisation ``norm = (skip or None, gamma, epsilon)``.  gate / up are
        (B, scales, bias or None).  The projections are the fp32 results of :meth:`projections_f32`; the activation
        and the product are evaluated in fp64 and narrowed once to the dtype of A.
        Returns Y, or (Y, input + skip) when ``norm`` has a skip input."""
        act, sm = A, None
        if norm is not None:
            skip, gamma, eps = norm
            if skip is not None:
                act, sm = self.simplified_layer_norm(A, skip, gamma, eps, want_sum=True)
            else:
                act = self.simplified_layer_norm(A, None, gamma, eps)
        g, u = self.projections_f32(act, (gate, up), (N, N), K, bits, bs, nthreads)
        g = g.astype(np.float64)
        with np.errstate(over="ignore"):
            y = g / (1.0 + np.exp(-g)) * u.astype(np.float64)
        y = self.f32_to_f16(y.astype(np.float32)) if A.dtype == np.float16 else y.astype(np.float32)
        return y if sm is None else (y, sm)

    def qkv(self, A, q, k, v, Nq, Nkv, K, bits, bs, norm=None, nthreads=1):
        """com.microsoft::MatMulNBitsQkv (contrib_defs.cc:3977-4090): the three projections of A' (see :meth:`mlp`).
        Returns (Q, K, V) or (Q, K, V, input + skip)."""
        act, sm = A, None
        if norm is not None:
            skip, gamma, eps = norm
            if skip is not None:
                act, sm = self.simplified_layer_norm(A, skip, gamma, eps, want_sum=True)
            else:
                act = self.simplified_layer_norm(A, None, gamma, eps)
        outs = [self.matmul(act, B, s, None, b, n, K, bits, bs, nthreads) for (B, s, b), n in
                zip((q, k, v), (Nq, Nkv, Nkv))]
        return tuple(outs) if sm is None else tuple(outs) + (sm,)

    # -- quantise -------------------------------------------------------------
    def quantize(self, W, bits, bs, symmetric):
        """W is [K, N] row-major, fp32 or fp16 (the model's type; other types are taken as fp32).
        Returns (B[N,kb,blob], scales[N,kb] in W's type, zp[N,zrow] or None)."""
        K, N = W.shape
        kb = (K + bs - 1) // bs
        Bq = np.empty((N, kb, bs * bits // 8), np.uint8)
        zp = None if symmetric else np.empty((N, (kb * bits + 7) // 8), np.uint8)
        if W.dtype == np.float16:
            W = np.ascontiguousarray(W)
            sc = np.empty((N, kb), np.float16)
            self.lib.mnbo_quantize_f16(_ptr(Bq, _u8p), _ptr(sc, _u16p), _ptr(zp, _u8p), _ptr(W, _u16p), K, N, bits,
                                       bs, 1 if symmetric else 0)
            return Bq, sc, zp
        W = np.ascontiguousarray(W, np.float32)
        sc = np.empty((N, kb), np.float32)
        self.lib.mnbo_quantize_f32(_ptr(Bq, _u8p), _ptr(sc, _f32p), _ptr(zp, _u8p), _ptr(W, _f32p), K, N, bits, bs,
                                   1 if symmetric else 0)
        return Bq, sc, zp


C = _C()


# ----------------------------------------------------------------------------- numpy restatement

def widen(x: np.ndarray) -> np.ndarray:
    """float32 view of a float32 / float16 array, or of bfloat16 values held in a uint16 array (exact)."""
    x = np.asarray(x)
    if x.dtype == np.uint16:
        return (x.astype(np.uint32) << 16).view(np.float32)
    return x.astype(np.float32)


def narrow_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 (as uint16), round to nearest even; finite inputs only."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def dense_matmul_f64(A, W, bias=None):
    """Y = A x W^T (+ bias) in float64 over float32 operands, and the row bound sum_k |a*w| (+ |bias|).
    W is [N, K] as the dequantisers return it."""
    a = widen(A).astype(np.float64)
    a = a.reshape(-1, a.shape[-1])
    w = np.asarray(W, np.float32).astype(np.float64)
    y = a @ w.T
    bound = np.abs(a) @ np.abs(w).T
    if bias is not None:
        b = widen(bias).astype(np.float64)
        y = y + b
        bound = bound + np.abs(b)
    return y, bound


def np_unpack_q(B: np.ndarray, N: int, K: int, bits: int, bs: int) -> np.ndarray:
    """Quantised integers as int32 [N, k_blocks*bs] from canonical B [N, k_blocks, bs*bits/8]."""
    kb = (K + bs - 1) // bs
    b = np.asarray(B, np.uint8).reshape(N, kb, bs * bits // 8).astype(np.int32)
    if bits == 8:
        q = b
    elif bits == 4:
        q = np.stack([b & 0xF, b >> 4], axis=-1).reshape(N, kb, bs)
    elif bits == 2:
        q = np.stack([b & 3, (b >> 2) & 3, (b >> 4) & 3, b >> 6], axis=-1).reshape(N, kb, bs)
    else:
        raise ValueError(bits)
    return q.reshape(N, kb * bs)


def np_unpack_zp(zp, N: int, K: int, bits: int, bs: int) -> np.ndarray:
    """Zero points as int32 [N, k_blocks]; ``None`` means the default 2^(bits-1)."""
    kb = (K + bs - 1) // bs
    if zp is None:
        return np.full((N, kb), 1 << (bits - 1), np.int32)
    row = (kb * bits + 7) // 8
    z = np.asarray(zp, np.uint8).reshape(N, row).astype(np.int32)
    if bits == 8:
        return z[:, :kb]
    if bits == 4:
        return np.stack([z & 0xF, z >> 4], axis=-1).reshape(N, row * 2)[:, :kb]
    return np.stack([z & 3, (z >> 2) & 3, (z >> 4) & 3, z >> 6], axis=-1).reshape(N, row * 4)[:, :kb]


def np_dequantize(B, scales, zp, N, K, bits, bs) -> np.ndarray:
    """W [N, K] in the dtype of ``scales``: fp32 -> one fp32 multiply; fp16 -> RNE of the exact fp32 product."""
    kb = (K + bs - 1) // bs
    q = np_unpack_q(B, N, K, bits, bs).reshape(N, kb, bs)
    z = np_unpack_zp(zp, N, K, bits, bs)[:, :, None]
    s = np.asarray(scales).reshape(N, kb)
    d = (q - z).astype(np.float32)
    w = d * s.astype(np.float32)[:, :, None]
    return w.reshape(N, kb * bs)[:, :K].astype(s.dtype if s.dtype == np.float16 else np.float32)


def np_matmul_f64(A, B, scales, zp, bias, N, K, bits, bs) -> np.ndarray:
    """fp64 matmul over the exactly-widened dequantised weights (kept in fp32 precision, not rounded to fp16)."""
    kb = (K + bs - 1) // bs
    q = np_unpack_q(B, N, K, bits, bs).reshape(N, kb, bs)
    z = np_unpack_zp(zp, N, K, bits, bs)[:, :, None]
    s = np.asarray(scales).reshape(N, kb).astype(np.float32)
    w = ((q - z).astype(np.float32) * s[:, :, None]).reshape(N, kb * bs)[:, :K].astype(np.float64)
    lead = A.shape[:-1]
    y = A.reshape(-1, K).astype(np.float64) @ w.T
    if bias is not None:
        y = y + np.asarray(bias).astype(np.float64)[None, :]
    return y.reshape(*lead, N)
