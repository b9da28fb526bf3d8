"""Seeded synthetic MatMulNBits inputs in the operator's canonical on-disk layout.

Shapes follow the op schema (onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3782-3849):
  A [..., K]; B u8 [N, k_blocks, block_size*bits/8]; scales [N, k_blocks]; zero_points u8
  [N, ceil(k_blocks*bits/8)] (optional); bias [N] (optional).
Draw order is fixed (A, B, scales, zero_points, bias) so a (seed, config) pair names one data set.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np


@dataclass
class MatMulNBitsCase:
    M: int
    N: int
    K: int
    bits: int
    block_size: int
    dtype: np.dtype
    A: np.ndarray
    B: np.ndarray
    scales: np.ndarray
    zero_points: Optional[np.ndarray]
    bias: Optional[np.ndarray]

    @property
    def k_blocks(self) -> int:
        return (self.K + self.block_size - 1) // self.block_size

    def algorithmic_bytes(self) -> int:
        """Bytes one call must move: every operand read once, Y written once."""
        es = np.dtype(self.dtype).itemsize
        n = self.N * self.k_blocks * (self.block_size * self.bits // 8) + self.N * self.k_blocks * es
        if self.zero_points is not None:
            n += self.N * ((self.k_blocks * self.bits + 7) // 8)
        if self.bias is not None:
            n += self.N * es
        return n + self.M * self.K * es + self.M * self.N * es

    def flops(self) -> int:
        return 2 * self.M * self.N * self.K


def make_case(M: int, N: int, K: int, bits: int = 4, block_size: int = 32, dtype=np.float16, has_zp: bool = False,
              has_bias: bool = False, seed: int = 0, a_shape=None) -> MatMulNBitsCase:
    rng = np.random.default_rng(seed)
    dtype = np.dtype(dtype)
    kb = (K + block_size - 1) // block_size
    a_shape = tuple(a_shape) if a_shape is not None else (M, K)
    A = rng.standard_normal(a_shape, dtype=np.float32).astype(dtype)
    B = rng.integers(0, 256, size=(N, kb, block_size * bits // 8), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.01, size=(N, kb)).astype(dtype)
    zp = rng.integers(0, 256, size=(N, (kb * bits + 7) // 8), dtype=np.uint8) if has_zp else None
    bias = (rng.standard_normal(N, dtype=np.float32) * 0.02).astype(dtype) if has_bias else None
    return MatMulNBitsCase(int(np.prod(a_shape[:-1])), N, K, bits, block_size, dtype, A, B, scales, zp, bias)


# The five benchmark configurations (Llama-3-8B projection shapes).
def config_c1(seed=0):
    return make_case(1, 4096, 4096, 4, 32, np.float32, has_zp=True, seed=seed)


def config_c2(seed=0):
    return make_case(1, 14336, 4096, 4, 128, np.float16, seed=seed)


def config_c4(seed=0, M=2048):
    return make_case(M, 14336, 4096, 4, 32, np.float16, has_zp=True, has_bias=True, seed=seed)


C3_SHAPES = {"qkv": (4096, 6144), "o": (4096, 4096), "down": (14336, 4096)}
C5_SHAPES = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}
