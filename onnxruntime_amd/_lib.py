"""ctypes binding of libmnb_mi355x.so -- the only way this package reaches the device kernels.

There is no fallback: if the shared library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_int64, c_size_t, c_void_p, c_char_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libmnb_mi355x.so"

DTYPE_FLOAT = 1
DTYPE_UINT8 = 2
DTYPE_INT32 = 6
DTYPE_FLOAT16 = 10
DTYPE_BFLOAT16 = 16

OK, FAIL, INVALID_ARGUMENT, NOT_IMPLEMENTED, EP_FAIL = 0, 1, 2, 9, 11


class MnbError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


class MnbTensorInfo(ctypes.Structure):
    _fields_ = [("dims", ctypes.POINTER(c_int64)), ("rank", c_size_t), ("dtype", c_int)]


class MnbNormPrologue(ctypes.Structure):
    _fields_ = [("norm_scale_dev", c_void_p), ("skip_dev", c_void_p), ("ld_skip", c_size_t), ("skip_rows", c_size_t),
                ("skip_sum_dev", c_void_p), ("ld_skip_sum", c_size_t), ("epsilon", ctypes.c_float)]


_NORM_P = ctypes.POINTER(MnbNormPrologue)

ZP_NONE, ZP_UINT8, ZP_TYPED = 0, 1, 2


class MnbVariantPlan(ctypes.Structure):
    _fields_ = [("N", c_int64), ("K", c_int64), ("bits", c_int), ("block_size", c_int), ("a_dtype", c_int),
                ("zp_kind", c_int), ("has_g_idx", c_int), ("compute_dtype", c_int), ("packed_k", c_int64),
                ("packed_block_size", c_int), ("reserved", c_int), ("gather_offset", ctypes.c_uint64),
                ("packed_bytes", ctypes.c_uint64)]


_PLAN_P = ctypes.POINTER(MnbVariantPlan)
_I32_P = ctypes.POINTER(ctypes.c_int32)

# name -> (restype, argtypes); every symbol include/mnb_mi355x.h declares
SIGNATURES = {
    "MnbGetLastErrorMessage": (c_char_p, []),
    "MnbGetVersion": (c_int, []),
    "MnbGetDeviceCount": (c_int, []),
    "MnbIsAvailable": (c_int, [c_int, c_int, c_int]),
    "MnbCheckInputs": (c_int, [ctypes.POINTER(MnbTensorInfo)] * 5 + [c_int64] * 4),
    "MnbPackQuantBDataSize": (c_size_t, [c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbPackQuantBData": (c_int, [c_size_t, c_size_t, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p]),
    "MnbGemmWorkspaceSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbGemm": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p,
                        c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "MnbGemmWorkspaceStatus": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                       c_void_p, ctypes.POINTER(c_int)]),
    "MnbGemmStaticScratchCapacity": (c_size_t, []),
    "MnbGemmStaticScratch": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p,
                                     c_void_p, c_void_p, c_size_t, c_void_p]),
    "MnbGemmUnpackedWorkspaceSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbGemmUnpacked": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p,
                                c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "MnbQuantizeBlockwise": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_size_t, c_size_t, c_size_t,
                                     c_int, c_void_p]),
    "MnbDequantizeBlockwise": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_size_t, c_size_t,
                                       c_int, c_void_p]),
    "MnbDequantizePacked": (c_int, [c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_void_p]),
    "MnbMlpPackSize": (c_size_t, [c_size_t, c_size_t, c_int, c_int, c_int]),
    "MnbMlpPack": (c_int, [c_size_t, c_size_t, c_int, c_int, c_int] + [c_void_p] * 8),
    "MnbMlpWorkspaceSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbMlpGemm": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_void_p, c_size_t, _NORM_P, c_void_p,
                           c_int, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "MnbQkvPackSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int]),
    "MnbQkvPack": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int] + [c_void_p] * 11),
    "MnbQkvWorkspaceSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbQkvGemm": (c_int, [c_size_t, c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_void_p, c_size_t, _NORM_P,
                           c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t,
                           c_void_p]),
    "MnbSimplifiedLayerNorm": (c_int, [c_size_t, c_size_t, c_int, c_void_p, c_size_t, _NORM_P, c_void_p, c_void_p]),
    "MnbVariantMakePlan": (c_int, [c_size_t, c_size_t, c_int, c_int, c_int, c_int, _I32_P, c_size_t, _PLAN_P]),
    "MnbVariantPack": (c_int, [_PLAN_P, c_void_p, c_void_p, c_void_p, _I32_P, c_size_t, c_void_p, c_void_p]),
    "MnbVariantGemmWorkspaceSize": (c_size_t, [_PLAN_P, c_size_t]),
    "MnbVariantGemmKernelName": (c_char_p, [_PLAN_P, c_size_t]),
    "MnbVariantGemm": (c_int, [_PLAN_P, c_size_t, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p,
                               c_size_t, c_void_p]),
    "MnbVariantDequantize": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_size_t,
                                     c_int, c_int, c_int, c_void_p]),
    "MnbGemmInt8WorkspaceSize": (c_size_t, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int]),
    "MnbGemmInt8": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p,
                            c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "MnbGemmKernelName": (c_char_p, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int]),
    "MnbGemmKernelNameStrided": (c_char_p, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_size_t]),
    "MnbGemmTilePlan": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, c_int, c_int, ctypes.POINTER(c_int),
                                ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the shared library (once). Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m onnxruntime_amd.build` "
                               "(there is no CPU fallback)")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().MnbGetLastErrorMessage().decode()


def check(code: int) -> None:
    if code != OK:
        raise MnbError(code, last_error())
