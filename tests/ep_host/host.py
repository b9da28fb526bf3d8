"""ctypes front end of the ONNX Runtime host test double (ort_host_shim.cc)."""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
SHIM = HERE / "libort_host_shim.so"
PLUGIN = HERE.parent.parent / "onnxruntime_amd" / "libonnxruntime_mi355x_ep.so"

NOT_CLAIMED, LOAD_FAILED, NO_DEVICE, PROTOCOL = -1, -2, -3, -4
_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int32): 6, np.dtype(np.float16): 10}


class EpHostTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dims", ctypes.POINTER(ctypes.c_int64)), ("rank", ctypes.c_size_t),
                ("dtype", ctypes.c_int)]


class EpHostError(RuntimeError):
    def __init__(self, code, message, trace=""):
        super().__init__(f"[{code}] {message}")
        self.code, self.message, self.trace = code, message, trace


def available() -> bool:
    return SHIM.exists() and PLUGIN.exists()


def _load():
    lib = ctypes.CDLL(str(SHIM))
    lib.EpHostProbeFactory.restype = ctypes.c_int
    lib.EpHostProbeFactory.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p,
                                       ctypes.c_size_t]
    lib.EpHostRunMatMulNBits.restype = ctypes.c_int
    lib.EpHostRunMatMulNBits.argtypes = [
        ctypes.c_char_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
        ctypes.POINTER(EpHostTensor), ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int64),
        ctypes.POINTER(ctypes.c_size_t), ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p,
        ctypes.c_size_t]
    return lib


def probe_factory(offer_amd_gpu: bool = True) -> dict:
    lib = _load()
    out, err = ctypes.create_string_buffer(512), ctypes.create_string_buffer(1024)
    rc = lib.EpHostProbeFactory(str(PLUGIN).encode(), int(offer_amd_gpu), out, len(out), err, len(err))
    if rc != 0:
        raise EpHostError(rc, err.value.decode())
    name, vendor, vendor_id, version, ndev, stream_aware = out.value.decode().split("|")
    return dict(name=name, vendor=vendor, vendor_id=int(vendor_id, 16), version=version, num_ep_devices=int(ndev),
                stream_aware=bool(int(stream_aware)))


def run_matmul_nbits(N, K, bits, block_size, A, B, scales, zero_points=None, g_idx=None, bias=None,
                     constant=("B", "scales", "zero_points", "bias"), accuracy_level=0, repeat=1):
    """One MatMulNBits node through the plugin EP. Returns (Y, trace). Raises EpHostError on any failure."""
    lib = _load()
    names = ["A", "B", "scales", "zero_points", "g_idx", "bias"]
    arrays = [A, B, scales, zero_points, g_idx, bias]
    tensors = (EpHostTensor * 6)()
    keep = []
    mask = 0
    for i, (nm, arr) in enumerate(zip(names, arrays)):
        if arr is None:
            tensors[i] = EpHostTensor(None, None, 0, 0)
            continue
        arr = np.ascontiguousarray(arr)
        dims = (ctypes.c_int64 * max(arr.ndim, 1))(*arr.shape)
        keep += [arr, dims]
        # an empty array still needs a non-NULL data pointer to count as present
        ptr = arr.ctypes.data if arr.size else ctypes.addressof(dims)
        tensors[i] = EpHostTensor(ptr, ctypes.cast(dims, ctypes.POINTER(ctypes.c_int64)), arr.ndim,
                                  _ONNX_TYPE[arr.dtype])
        if nm in constant and i > 0:
            mask |= 1 << i
    lead = A.shape[:-1]
    y = np.empty(lead + (N,), dtype=A.dtype)
    y_dims = (ctypes.c_int64 * 8)()
    y_rank = ctypes.c_size_t(0)
    trace, err = ctypes.create_string_buffer(512), ctypes.create_string_buffer(2048)
    rc = lib.EpHostRunMatMulNBits(str(PLUGIN).encode(), N, K, bits, block_size, accuracy_level, tensors, mask,
                                  y.ctypes.data if y.size else None, y.nbytes, y_dims, ctypes.byref(y_rank), repeat,
                                  trace, len(trace), err, len(err))
    if rc != 0:
        raise EpHostError(rc, err.value.decode(), trace.value.decode())
    shape = tuple(y_dims[i] for i in range(y_rank.value))
    assert shape == y.shape, (shape, y.shape)
    return y, trace.value.decode()
