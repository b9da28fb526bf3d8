"""Host-side mirror of the reference's MatMulNBits kernel class, driving the MI355X library through its C ABI.

The class follows contrib::MatMulNBits<T1> (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc):
  constructor   attribute checks                                  :100-138
  PrePack       shape guards + repack of B / scales / zero points  :252-724 (fp16: :729-859)
  Compute       CheckInputs, output shape, empty-output return,    :1513-1570
                packed or unpacked route
The inputs the reference serves through its dequantise-everything route (:1248-1295: zero points in the activation
type, a group index) and bfloat16 activations go through the library's variant entry points.
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
           torch.int32: _lib.DTYPE_INT32, torch.bfloat16: _lib.DTYPE_BFLOAT16}


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
                 has_g_idx: bool = False, zero_points_dtype: torch.dtype = torch.uint8,
                 int8_activations: bool = False):
        """``int8_activations``: take the permission that accuracy_level = 4 grants and quantise A blockwise to int8
        (MnbGemmInt8) where that route exists; off by default, because the full-accuracy route is the faster one."""
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
        # typed zero points, a group index, bfloat16: the variant entry points
        self.variant = has_g_idx or zero_points_dtype != torch.uint8 or dtype == torch.bfloat16
        # what this device path takes; everything else stays with the CPU provider
        if self.variant:
            self.supported = (dtype in (torch.float16, torch.float32, torch.bfloat16)
                              and zero_points_dtype in (torch.uint8, dtype)
                              and (zero_points_dtype == torch.uint8 or bits in (2, 4))   # matmul_nbits.cc:1251-1252
                              and (not has_g_idx or bits == 4))
        else:
            self.supported = (dtype in (torch.float16, torch.float32) and bits in (2, 4, 8)
                              and bool(self.lib.MnbIsAvailable(bits, block_size, _DTYPES[dtype])))
        self.packed: Optional[torch.Tensor] = None
        self.plan: Optional[_lib.MnbVariantPlan] = None
        self._workspace = {}
        self.int8_activations = bool(int8_activations) and self.accuracy_level == 4 and not self.variant

    @property
    def zp_kind(self) -> int:
        if not self.has_zero_points:
            return _lib.ZP_NONE
        return _lib.ZP_UINT8 if self.zero_points_dtype == torch.uint8 else _lib.ZP_TYPED

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

    def _pack_variant(self, b, scales, zero_points, g_idx):
        """(plan, packed buffer) for the variant route; g_idx is copied to the host, where the k order is planned."""
        if (g_idx is not None) != self.has_g_idx:
            raise MnbError(_lib.INVALID_ARGUMENT, "MatMulNBits PrePack: g_idx presence differs from the node")
        if scales.dtype != self.dtype or (zero_points is not None and zero_points.dtype != self.zero_points_dtype):
            raise MnbError(_lib.INVALID_ARGUMENT, "MatMulNBits PrePack: scales / zero_points types differ from the node")
        g_host, g_ptr, g_len = None, None, 0
        if g_idx is not None:
            g_host = g_idx.to(device="cpu", dtype=torch.int32).contiguous().numpy()
            g_ptr, g_len = g_host.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), g_host.size
        plan = _lib.MnbVariantPlan()
        _lib.check(self.lib.MnbVariantMakePlan(self.N, self.K, self.bits, self.block_size, _DTYPES[self.dtype],
                                               self.zp_kind, g_ptr, g_len, ctypes.byref(plan)))
        packed = torch.empty(plan.packed_bytes, dtype=torch.uint8, device=b.device)
        _lib.check(self.lib.MnbVariantPack(ctypes.byref(plan), _ptr(b.contiguous()), _ptr(scales.contiguous()),
                                           _ptr(None if zero_points is None else zero_points.contiguous()), g_ptr,
                                           g_len, _ptr(packed), _stream_ptr(b.device)))
        return plan, packed

    def PrePack(self, b: torch.Tensor, scales: torch.Tensor, zero_points: Optional[torch.Tensor] = None,
                g_idx: Optional[torch.Tensor] = None) -> bool:
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
        if self.variant:
            self.plan, self.packed = self._pack_variant(b, scales, zero_points, g_idx)
            return True
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
                out: Optional[torch.Tensor] = None, g_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Y = A x dequant(B)^T (+ bias). b/scales/zero_points/g_idx are only needed when PrePack did not run."""
        if not self.supported:
            raise MnbError(_lib.NOT_IMPLEMENTED, "this MatMulNBits configuration has no MI355X kernel")
        check_inputs(None if b is None else tuple(b.shape), None if scales is None else tuple(scales.shape),
                     None if zero_points is None else tuple(zero_points.shape),
                     None if g_idx is None else tuple(g_idx.shape),
                     None if bias is None else tuple(bias.shape), self.N, self.K, self.block_size, self.bits,
                     scales_dtype=self.dtype, zp_dtype=self.zero_points_dtype)
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
        if self.variant:
            plan, packed = self.plan, self.packed
            if packed is None:  # operands fed per run: plan and pack per call, like the reference's unpacked route
                if b is None or scales is None:
                    raise MnbError(_lib.INVALID_ARGUMENT,
                                   "MatMulNBits: B and scales are required when B was not prepacked")
                plan, packed = self._pack_variant(b, scales, zero_points, g_idx)
            wsz = self.lib.MnbVariantGemmWorkspaceSize(ctypes.byref(plan), M)
            ws = self._get_workspace(a.device, wsz)
            _lib.check(self.lib.MnbVariantGemm(ctypes.byref(plan), M, _ptr(a2), lda, _ptr(packed), _ptr(bias),
                                               _ptr(y2), self.N, _ptr(ws), wsz, stream))
            return y
        if self.packed is not None and self.int8_activations:
            wsz = self.lib.MnbGemmInt8WorkspaceSize(M, self.N, self.K, self.bits, self.block_size,
                                                    int(self.has_zero_points), dt)
            if wsz:  # 0: no int8 route for this configuration, the full-accuracy one below takes it
                ws = self._get_workspace(a.device, wsz)
                _lib.check(self.lib.MnbGemmInt8(M, self.N, self.K, self.bits, self.block_size,
                                                int(self.has_zero_points), dt, _ptr(a2), lda, _ptr(self.packed),
                                                _ptr(bias), _ptr(y2), self.N, _ptr(ws), wsz, stream))
                return y
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


class _FusedProjections:
    """Shared host side of MatMulNBitsMlp / MatMulNBitsQkv: attribute checks, the optional
    (Skip)SimplifiedLayerNormalization prologue and the workspace."""

    OP = ""

    def __init__(self, K: int, bits: int, block_size: int, accuracy_level: int, epsilon: float, dtype: torch.dtype):
        if bits not in (2, 4, 8):
            raise MnbError(_lib.INVALID_ARGUMENT, "Only 2b, 4b and 8b quantization is supported for MatMulNBits op, "
                                                  "additional bits support is planned.")
        if block_size not in (16, 32, 64, 128, 256):
            raise MnbError(_lib.INVALID_ARGUMENT, "Only block sizes 16, 32, 64, 128, and 256 are supported for "
                                                  f"MatMulNBits op, got: {block_size}")
        self.K, self.bits, self.block_size = int(K), int(bits), int(block_size)
        self.accuracy_level, self.epsilon, self.dtype = int(accuracy_level), float(epsilon), dtype
        self.k_blocks = (self.K + self.block_size - 1) // self.block_size
        self.blob_size = self.block_size * self.bits // 8
        self.lib = _lib.load()
        self.supported = (dtype in (torch.float16, torch.float32) and bits in (2, 4, 8)
                          and bool(self.lib.MnbIsAvailable(bits, block_size, _DTYPES[dtype])))
        self.packed: Optional[torch.Tensor] = None
        self._workspace = {}

    def _check_projection(self, name: str, n: int, b, scales, bias) -> None:
        kb, blob = self.k_blocks, self.blob_size
        check_inputs(tuple(b.shape), tuple(scales.shape), None, None, None if bias is None else tuple(bias.shape),
                     n, self.K, self.block_size, self.bits, scales_dtype=self.dtype)
        if scales.dtype != self.dtype or (bias is not None and bias.dtype != self.dtype):
            raise MnbError(_lib.INVALID_ARGUMENT, f"{self.OP}: {name} scales and bias must have the type of A")

    _get_workspace = MatMulNBits._get_workspace

    def _prologue(self, a2: torch.Tensor, skip, norm_scale, want_sum: bool):
        """Returns (MnbNormPrologue or None, skip-sum tensor or None, tensors to keep alive)."""
        if norm_scale is None:
            if skip is not None:
                raise MnbError(_lib.INVALID_ARGUMENT, "norm_scale input must be present when skip input is provided")
            return None, None, ()
        if tuple(norm_scale.shape) != (self.K,):
            raise MnbError(_lib.INVALID_ARGUMENT, f"norm_scale shape must be [K] where K = {self.K}")
        M = a2.shape[0]
        n = _lib.MnbNormPrologue()
        n.norm_scale_dev = norm_scale.contiguous().data_ptr()
        n.epsilon = self.epsilon
        keep = [norm_scale]
        sm = None
        if skip is not None:
            if skip.shape[-1] != self.K or skip.numel() == 0 or a2.numel() % skip.numel() != 0:
                raise MnbError(_lib.INVALID_ARGUMENT, f"{self.OP}: skip must broadcast over the rows of A")
            s2 = skip.reshape(-1, self.K).contiguous()
            n.skip_dev, n.ld_skip, n.skip_rows = s2.data_ptr(), self.K, s2.shape[0]
            keep.append(s2)
            if want_sum:
                sm = torch.empty(M, self.K, dtype=self.dtype, device=a2.device)
                n.skip_sum_dev, n.ld_skip_sum = sm.data_ptr(), self.K
        elif want_sum:
            raise MnbError(_lib.INVALID_ARGUMENT,
                           "skip input must be present when input_skip_bias_sum output is requested")
        return n, sm, tuple(keep)

    def _rows(self, a: torch.Tensor) -> torch.Tensor:
        if not self.supported:
            raise MnbError(_lib.NOT_IMPLEMENTED, f"this {self.OP} configuration has no MI355X kernel")
        if self.packed is None:
            raise MnbError(_lib.INVALID_ARGUMENT, f"{self.OP}: PrePack has not run")
        if a.dtype != self.dtype:
            raise MnbError(_lib.INVALID_ARGUMENT, f"A has dtype {a.dtype}, the node was built for {self.dtype}")
        if a.shape[-1] != self.K:
            raise MnbError(_lib.INVALID_ARGUMENT,
                           f"{self.OP}: the last dimension of A ({a.shape[-1]}) must equal K ({self.K})")
        a2 = a.reshape(-1, self.K)
        return a2 if a2.stride(-1) == 1 else a2.contiguous()


class MatMulNBitsMlp(_FusedProjections):
    """com.microsoft::MatMulNBitsMlp (contrib_defs.cc:3851-3975) bound to the MI355X kernels:
    Y = silu(A' gate^T + gate_bias) * (A' up^T + up_bias), A' = A or its (skip) simplified layer normalisation."""

    OP = "MatMulNBitsMlp"

    def __init__(self, K: int, N: int, bits: int = 4, block_size: int = 32, accuracy_level: int = 0,
                 activation: str = "silu", epsilon: float = 1e-5, dtype: torch.dtype = torch.float16):
        super().__init__(K, bits, block_size, accuracy_level, epsilon, dtype)
        if activation != "silu":  # matmul_nbits_mlp.cc:24-31
            raise MnbError(_lib.INVALID_ARGUMENT, f"MatMulNBitsMlp: activation '{activation}' is not supported.")
        self.N = int(N)

    def PrePack(self, gate_b, gate_scales, gate_bias, up_b, up_scales, up_bias) -> bool:
        self._check_projection("gate", self.N, gate_b, gate_scales, gate_bias)
        self._check_projection("up", self.N, up_b, up_scales, up_bias)
        if not self.supported:
            return False
        dt = _DTYPES[self.dtype]
        size = self.lib.MnbMlpPackSize(self.N, self.K, self.bits, self.block_size, dt)
        packed = torch.empty(size, dtype=torch.uint8, device=gate_b.device)
        c = lambda t: None if t is None else t.contiguous()  # noqa: E731
        ts = [c(gate_b), c(gate_scales), c(gate_bias), c(up_b), c(up_scales), c(up_bias)]
        _lib.check(self.lib.MnbMlpPack(self.N, self.K, self.bits, self.block_size, dt, *[_ptr(t) for t in ts],
                                       _ptr(packed), _stream_ptr(gate_b.device)))
        self.packed = packed
        return True

    def Compute(self, a: torch.Tensor, skip: Optional[torch.Tensor] = None, norm_scale: Optional[torch.Tensor] = None,
                want_skip_sum: bool = False):
        """Returns Y, or (Y, input_skip_bias_sum) when ``want_skip_sum``."""
        a2 = self._rows(a)
        lead, M = tuple(a.shape[:-1]), a2.shape[0]
        y = torch.empty(*lead, self.N, dtype=self.dtype, device=a.device)
        norm, sm, keep = self._prologue(a2, skip, norm_scale, want_skip_sum)
        if y.numel():
            dt = _DTYPES[self.dtype]
            wsz = self.lib.MnbMlpWorkspaceSize(M, self.N, self.K, self.bits, self.block_size, dt, int(norm is not None))
            ws = self._get_workspace(a.device, wsz)
            _lib.check(self.lib.MnbMlpGemm(M, self.N, self.K, self.bits, self.block_size, dt, _ptr(a2),
                                           a2.stride(0) if M > 1 else self.K,
                                           None if norm is None else ctypes.byref(norm), _ptr(self.packed), 0,
                                           _ptr(y), self.N, _ptr(ws), wsz, _stream_ptr(a.device)))
        del keep
        return (y, sm.view(*lead, self.K)) if want_skip_sum else y


class MatMulNBitsQkv(_FusedProjections):
    """com.microsoft::MatMulNBitsQkv (contrib_defs.cc:3977-4090): Q, K, V = A' x {q, k, v}^T + bias."""

    OP = "MatMulNBitsQkv"

    def __init__(self, K: int, Nq: int, Nkv: int, bits: int = 4, block_size: int = 32, accuracy_level: int = 0,
                 epsilon: float = 1e-6, dtype: torch.dtype = torch.float16):
        super().__init__(K, bits, block_size, accuracy_level, epsilon, dtype)
        self.Nq, self.Nkv = int(Nq), int(Nkv)

    def PrePack(self, q_b, q_scales, q_bias, k_b, k_scales, k_bias, v_b, v_scales, v_bias) -> bool:
        self._check_projection("q", self.Nq, q_b, q_scales, q_bias)
        self._check_projection("k", self.Nkv, k_b, k_scales, k_bias)
        self._check_projection("v", self.Nkv, v_b, v_scales, v_bias)
        if not self.supported:
            return False
        dt = _DTYPES[self.dtype]
        size = self.lib.MnbQkvPackSize(self.Nq, self.Nkv, self.K, self.bits, self.block_size, dt)
        packed = torch.empty(size, dtype=torch.uint8, device=q_b.device)
        ts = [None if t is None else t.contiguous()
              for t in (q_b, q_scales, q_bias, k_b, k_scales, k_bias, v_b, v_scales, v_bias)]
        _lib.check(self.lib.MnbQkvPack(self.Nq, self.Nkv, self.K, self.bits, self.block_size, dt,
                                       *[_ptr(t) for t in ts], _ptr(packed), _stream_ptr(q_b.device)))
        self.packed = packed
        return True

    def Compute(self, a: torch.Tensor, skip: Optional[torch.Tensor] = None, norm_scale: Optional[torch.Tensor] = None,
                want_skip_sum: bool = False):
        """Returns (Q, K, V) or (Q, K, V, input_skip_bias_sum).  The operator requires norm_scale; it is optional
        here so that the projections can be used on their own."""
        a2 = self._rows(a)
        lead, M = tuple(a.shape[:-1]), a2.shape[0]
        outs = [torch.empty(*lead, n, dtype=self.dtype, device=a.device) for n in (self.Nq, self.Nkv, self.Nkv)]
        norm, sm, keep = self._prologue(a2, skip, norm_scale, want_skip_sum)
        if M:
            dt = _DTYPES[self.dtype]
            wsz = self.lib.MnbQkvWorkspaceSize(M, self.Nq, self.Nkv, self.K, self.bits, self.block_size, dt,
                                               int(norm is not None))
            ws = self._get_workspace(a.device, wsz)
            _lib.check(self.lib.MnbQkvGemm(M, self.Nq, self.Nkv, self.K, self.bits, self.block_size, dt, _ptr(a2),
                                           a2.stride(0) if M > 1 else self.K,
                                           None if norm is None else ctypes.byref(norm), _ptr(self.packed),
                                           _ptr(outs[0]), self.Nq, _ptr(outs[1]), self.Nkv, _ptr(outs[2]), self.Nkv,
                                           _ptr(ws), wsz, _stream_ptr(a.device)))
        del keep
        return tuple(outs) + ((sm.view(*lead, self.K),) if want_skip_sum else ())


def simplified_layer_norm(a: torch.Tensor, norm_scale: torch.Tensor, epsilon: float,
                          skip: Optional[torch.Tensor] = None, want_skip_sum: bool = False):
    """(Skip)SimplifiedLayerNormalization over the last axis on the device (the prologue of the fused operators)."""
    lib = _lib.load()
    K = a.shape[-1]
    a2 = a.reshape(-1, K)
    a2 = a2 if a2.stride(-1) == 1 else a2.contiguous()
    M = a2.shape[0]
    out = torch.empty(M, K, dtype=a.dtype, device=a.device)
    n = _lib.MnbNormPrologue()
    g = norm_scale.contiguous()
    n.norm_scale_dev, n.epsilon = g.data_ptr(), float(epsilon)
    sm = None
    if skip is not None:
        s2 = skip.reshape(-1, K).contiguous()
        n.skip_dev, n.ld_skip, n.skip_rows = s2.data_ptr(), K, s2.shape[0]
        if want_skip_sum:
            sm = torch.empty(M, K, dtype=a.dtype, device=a.device)
            n.skip_sum_dev, n.ld_skip_sum = sm.data_ptr(), K
    _lib.check(lib.MnbSimplifiedLayerNorm(M, K, _DTYPES[a.dtype], _ptr(a2), a2.stride(0) if M > 1 else K,
                                          ctypes.byref(n), _ptr(out), _stream_ptr(a.device)))
    out = out.view(a.shape)
    return (out, sm.view(a.shape)) if want_skip_sum else out


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


def dequantize_blockwise_variant(b: torch.Tensor, scales: torch.Tensor, zero_points: Optional[torch.Tensor],
                                 g_idx: Optional[torch.Tensor], N: int, K: int, bits: int,
                                 block_size: int) -> torch.Tensor:
    """The reference's dequantiser for typed zero points and / or a group index on the device
    (matmul_nbits_impl.cc:19-75): W float32 [N, K] = float(q) * scale + (-scale * zp), whatever the scales' type."""
    lib = _lib.load()
    w = torch.empty(N, K, dtype=torch.float32, device=b.device)
    if zero_points is None:
        kind = _lib.ZP_NONE
    else:
        kind = _lib.ZP_UINT8 if zero_points.dtype == torch.uint8 else _lib.ZP_TYPED
    g = None if g_idx is None else g_idx.to(torch.int32).contiguous()
    _lib.check(lib.MnbVariantDequantize(_ptr(w), _ptr(b.contiguous()), _ptr(scales.contiguous()),
                                        _ptr(None if zero_points is None else zero_points.contiguous()), kind,
                                        _ptr(g), N, K, bits, block_size, _DTYPES[scales.dtype],
                                        _stream_ptr(b.device)))
    return w
