"""Host-side mirror of the reference's MatMulNBits kernel class, driving the MI355X library through its C ABI.

The class follows contrib::MatMulNBits<T1> (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc):
  constructor   attribute checks                                  :100-138
  PrePack       shape guards + repack of B / scales / zero points  :252-724 (fp16: :729-859)
  Compute       CheckInputs, output shape, empty-output return,    :1513-1570
                packed or unpacked route
Tensors are torch tensors on a HIP device; torch only provides memory and streams here.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import MnbError, MnbTensorInfo

A, B, SCALES, ZERO_POINTS, G_IDX, BIAS = range(6)  # operator input indices (contrib_defs.cc:3794-3828)

_DTYPES = {torch.float32: _lib.DTYPE_FLOAT, torch.float16: _lib.DTYPE_FLOAT16, torch.uint8: _lib.DTYPE_UINT8,
           torch.int32: _lib.DTYPE_INT32}


def _info(shape: Optional[Sequence[int]], dtype) -> MnbTensorInfo:
    if shape is None:
        return MnbTensorInfo(None, 0, 0)
    arr = (ctypes.c_int64 * max(len(shape), 1))(*shape)
    info = MnbTensorInfo(ctypes.cast(arr, ctypes.POINTER(ctypes.c_int64)), len(shape), _DTYPES.get(dtype, 0))
    info._keep = arr
    return info


def check_inputs(b_shape, scales_shape, zp_shape, g_idx_shape, bias_shape, n, k, block_size, bits,
                 scales_dtype=torch.float16, zp_dtype=torch.uint8) -> None:
    """matmul_nbits_helper::CheckInputs (matmul_nbits_helper.h:38-109) on shapes; raises MnbError(INVALID_ARGUMENT)."""
    lib = _lib.load()
    infos = [_info(b_shape, torch.uint8), _info(scales_shape, scales_dtype), _info(zp_shape, zp_dtype),
             _info(g_idx_shape, torch.int32), _info(bias_shape, scales_dtype)]
    _lib.check(lib.MnbCheckInputs(*[ctypes.byref(i) for i in infos], n, k, block_size, bits))


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream_ptr(device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class MatMulNBits:
    """One MatMulNBits node bound to the MI355X kernels."""

    def __init__(self, K: int, N: int, bits: int = 4, block_size: int = 32, accuracy_level: int = 0,
                 dtype: torch.dtype = torch.float16, has_zero_points: bool = False, has_bias: bool = False,
                 has_g_idx: bool = False, zero_points_dtype: torch.dtype = torch.uint8):
        if bits not in (2, 4, 8):
            raise MnbError(_lib.INVALID_ARGUMENT, "Only 2b, 4b and 8b quantization is supported for MatMulNBits op, "
                                                  "additional bits support is planned.")
        if block_size not in (16, 32, 64, 128, 256):
            raise MnbError(_lib.INVALID_ARGUMENT, "Only block sizes 16, 32, 64, 128, and 256 are supported for "
                                                  f"MatMulNBits op, got: {block_size}")
        self.K, self.N, self.bits, self.block_size = int(K), int(N), int(bits), int(block_size)
        self.accuracy_level = int(accuracy_level)
        self.dtype = dtype
        self.has_zero_points, self.has_bias, self.has_g_idx = has_zero_points, has_bias, has_g_idx
        self.zero_points_dtype = zero_points_dtype
        self.k_blocks = (self.K + self.block_size - 1) // self.block_size
        self.blob_size = self.block_size * self.bits // 8
        self.zp_row = (self.k_blocks * self.bits + 7) // 8
        self.lib = _lib.load()
        # what this device path takes; everything else stays with the CPU provider
        self.supported = (dtype in (torch.float16, torch.float32) and bits in (4, 8) and not has_g_idx
                          and zero_points_dtype == torch.uint8
                          and bool(self.lib.MnbIsAvailable(bits, block_size, _DTYPES[dtype])))
        self.packed: Optional[torch.Tensor] = None
        self._workspace = {}

    # -- PrePack ------------------------------------------------------------------------------------------------
    def _validate_initializer(self, idx: int, t: torch.Tensor) -> None:
        """The PrePack shape guards of matmul_nbits.cc:282-341 with the same messages."""
        n, kb, blob, zb = self.N, self.k_blocks, self.blob_size, self.zp_row
        shape = tuple(t.shape)
        s = "{" + ",".join(str(d) for d in shape) + "}"
        if idx == B and shape != (n, kb, blob):
            raise MnbError(_lib.INVALID_ARGUMENT,
                           f"MatMulNBits PrePack: B initializer shape {s} does not match attribute-derived shape "
                           f"[{n},{kb},{blob}] (N={self.N}, K={self.K}, bits={self.bits}, "
                           f"block_size={self.block_size})")
        if idx == SCALES and shape not in ((n * kb,), (n, kb)):
            raise MnbError(_lib.INVALID_ARGUMENT,
                           f"MatMulNBits PrePack: scales initializer shape {s} does not match attribute-derived "
                           f"shape [{n * kb}] or [{n},{kb}]")
        if idx == ZERO_POINTS:
            if t.dtype == torch.uint8:
                if shape not in ((n * zb,), (n, zb)):
                    raise MnbError(_lib.INVALID_ARGUMENT,
                                   f"MatMulNBits PrePack: zero_points initializer shape {s} does not match "
                                   f"attribute-derived shape [{n * zb}] or [{n},{zb}]")
            elif shape not in ((n * kb,), (n, kb)):
                raise MnbError(_lib.INVALID_ARGUMENT,
                               f"MatMulNBits PrePack: zero_points initializer shape {s} does not match "
                               f"attribute-derived shape [{n * kb}] or [{n},{kb}]")

    def PrePack(self, b: torch.Tensor, scales: torch.Tensor, zero_points: Optional[torch.Tensor] = None) -> bool:
        """Repacks constant B / scales / zero_points (device tensors, canonical layout) into the tiled layout.

        Returns True when the weights were packed (the caller may then drop the originals), False when this
        configuration is left to the unpacked route."""
        self._validate_initializer(B, b)
        self._validate_initializer(SCALES, scales)
        if zero_points is not None:
            self._validate_initializer(ZERO_POINTS, zero_points)
        if not self.supported:
            return False
        if (zero_points is not None) != self.has_zero_points:
            raise MnbError(_lib.INVALID_ARGUMENT, "MatMulNBits PrePack: zero_points presence differs from the node")
        dt = _DTYPES[self.dtype]
        size = self.lib.MnbPackQuantBDataSize(self.N, self.K, self.bits, self.block_size,
                                              int(self.has_zero_points), dt)
        packed = torch.empty(size, dtype=torch.uint8, device=b.device)
        _lib.check(self.lib.MnbPackQuantBData(self.N, self.K, self.bits, self.block_size, dt, _ptr(b.contiguous()),
                                              _ptr(scales.contiguous()),
                                              _ptr(None if zero_points is None else zero_points.contiguous()),
                                              _ptr(packed), _stream_ptr(b.device)))
        self.packed = packed
        return True

    # -- Compute ------------------------------------------------------------------------------------------------
    def _get_workspace(self, device, nbytes: int) -> Optional[torch.Tensor]:
        if nbytes == 0:
            return None
        key = (device, torch.cuda.current_stream(device).cuda_stream)
        ws = self._workspace.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)  # tickets start at zero
            self._workspace[key] = ws
        return ws

    def Compute(self, a: torch.Tensor, b: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None,
                zero_points: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Y = A x dequant(B)^T (+ bias). b/scales/zero_points are only needed when PrePack did not run."""
        if not self.supported:
            raise MnbError(_lib.NOT_IMPLEMENTED, "this MatMulNBits configuration has no MI355X kernel")
        check_inputs(None if b is None else tuple(b.shape), None if scales is None else tuple(scales.shape),
                     None if zero_points is None else tuple(zero_points.shape), None,
                     None if bias is None else tuple(bias.shape), self.N, self.K, self.block_size, self.bits,
                     scales_dtype=self.dtype)
        if a.dtype != self.dtype:
            raise MnbError(_lib.INVALID_ARGUMENT, f"A has dtype {a.dtype}, the node was built for {self.dtype}")
        if a.shape[-1] != self.K:
            raise MnbError(_lib.INVALID_ARGUMENT,
                           f"MatMulNBits: the last dimension of A ({a.shape[-1]}) must equal K ({self.K})")
        lead = tuple(a.shape[:-1])
        a2 = a.reshape(-1, self.K)
        if a2.stride(-1) != 1:
            a2 = a2.contiguous()
        M = a2.shape[0]
        y = out if out is not None else torch.empty(*lead, self.N, dtype=self.dtype, device=a.device)
        if y.numel() == 0:
            return y  # empty output: nothing to compute (matmul_nbits.cc:1533-1536)
        y2 = y.view(-1, self.N)
        dt = _DTYPES[self.dtype]
        lda = a2.stride(0) if M > 1 else self.K
        stream = _stream_ptr(a.device)
        if self.packed is not None:
            wsz = self.lib.MnbGemmWorkspaceSize(M, self.N, self.K, self.bits, self.block_size,
                                                int(self.has_zero_points), dt)
            ws = self._get_workspace(a.device, wsz)
            _lib.check(self.lib.MnbGemm(M, self.N, self.K, self.bits, self.block_size, int(self.has_zero_points), dt,
                                        _ptr(a2), lda, _ptr(self.packed), _ptr(bias), _ptr(y2), self.N, _ptr(ws),
                                        wsz, stream))
        else:
            if b is None or scales is None:
                raise MnbError(_lib.INVALID_ARGUMENT, "MatMulNBits: B and scales are required when B was not prepacked")
            has_zp = int(zero_points is not None)
            wsz = self.lib.MnbGemmUnpackedWorkspaceSize(M, self.N, self.K, self.bits, self.block_size, has_zp, dt)
            ws = self._get_workspace(a.device, wsz)
            _lib.check(self.lib.MnbGemmUnpacked(M, self.N, self.K, self.bits, self.block_size, dt, _ptr(a2), lda,
                                                _ptr(b.contiguous()), _ptr(scales.contiguous()),
                                                _ptr(None if zero_points is None else zero_points.contiguous()),
                                                _ptr(bias), _ptr(y2), self.N, _ptr(ws), wsz, stream))
        return y

    # -- test hooks ---------------------------------------------------------------------------------------------
    def dequantize_packed(self) -> torch.Tensor:
        """W [N, K] read back from the packed buffer through the kernels' own unpack code."""
        assert self.packed is not None
        w = torch.empty(self.N, self.K, dtype=self.dtype, device=self.packed.device)
        _lib.check(self.lib.MnbDequantizePacked(_ptr(w), _ptr(self.packed), self.N, self.K, self.bits, self.block_size,
                                                int(self.has_zero_points), _DTYPES[self.dtype],
                                                _stream_ptr(w.device)))
        return w


def dequantize_blockwise(b: torch.Tensor, scales: torch.Tensor, zero_points: Optional[torch.Tensor], N: int, K: int,
                         bits: int, block_size: int) -> torch.Tensor:
    """MlasDequantizeBlockwise on the device: W [N, K] in the dtype of scales."""
    lib = _lib.load()
    w = torch.empty(N, K, dtype=scales.dtype, device=b.device)
    _lib.check(lib.MnbDequantizeBlockwise(_ptr(w), _ptr(b.contiguous()), _ptr(scales.contiguous()),
                                          _ptr(None if zero_points is None else zero_points.contiguous()), block_size,
                                          bits, K, N, _DTYPES[scales.dtype], _stream_ptr(b.device)))
    return w


def quantize_blockwise(w: torch.Tensor, bits: int, block_size: int, symmetric: bool):
    """MlasQuantizeBlockwise on the device (column-wise blocks): w is the [K, N] weight matrix of a MatMul in fp16 or
    fp32 (row stride >= N allowed). Returns the operator's inputs (B u8 [N, k_blocks, block_size*bits/8],
    scales [N, k_blocks] in w's dtype, zero_points u8 [N, ceil(k_blocks*bits/8)] or None when symmetric)."""
    lib = _lib.load()
    if w.dim() != 2 or w.dtype not in (torch.float16, torch.float32):
        raise MnbError(_lib.INVALID_ARGUMENT, "quantize_blockwise: w must be a 2-D fp16 or fp32 tensor")
    if w.stride(1) != 1:
        w = w.contiguous()
    K, N = w.shape
    kb = (K + block_size - 1) // block_size
    b = torch.empty(N, kb, block_size * bits // 8, dtype=torch.uint8, device=w.device)
    scales = torch.empty(N, kb, dtype=w.dtype, device=w.device)
    zp = None if symmetric else torch.empty(N, (kb * bits + 7) // 8, dtype=torch.uint8, device=w.device)
    _lib.check(lib.MnbQuantizeBlockwise(_ptr(b), _ptr(scales), _ptr(zp), _ptr(w), block_size, bits, K, N,
                                        w.stride(0) if K > 1 else N, _DTYPES[w.dtype], _stream_ptr(w.device)))
    return b, scales, zp
