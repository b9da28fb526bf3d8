"""ctypes front end of the ONNX Runtime host test double (ort_host_shim.cc)."""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
SHIM = HERE / "libort_host_shim.so"
PLUGIN = HERE.parent.parent / "onnxruntime_amd" / "libonnxruntime_mi355x_ep.so"

NOT_CLAIMED, LOAD_FAILED, NO_DEVICE, PROTOCOL, NOT_FUSED = -1, -2, -3, -4, -5
# bfloat16 tensors travel as uint16 arrays of their bit patterns
_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int32): 6, np.dtype(np.float16): 10,
              np.dtype(np.uint16): 16}


class EpHostTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dims", ctypes.POINTER(ctypes.c_int64)), ("rank", ctypes.c_size_t),
                ("dtype", ctypes.c_int)]


class EpHostAttr(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("kind", ctypes.c_int), ("i", ctypes.c_int64), ("f", ctypes.c_float),
                ("s", ctypes.c_char_p)]


class EpHostNodeSpec(ctypes.Structure):
    _fields_ = [("op_type", ctypes.c_char_p), ("attrs", ctypes.POINTER(EpHostAttr)), ("num_attrs", ctypes.c_size_t),
                ("schema_attrs", ctypes.POINTER(ctypes.c_char_p)), ("num_schema_attrs", ctypes.c_size_t),
                ("input_names", ctypes.POINTER(ctypes.c_char_p)), ("input_types", ctypes.POINTER(ctypes.c_char_p)),
                ("num_inputs", ctypes.c_size_t), ("num_outputs", ctypes.c_size_t),
                ("skipped_output_mask", ctypes.c_int)]


class EpHostAddSpec(ctypes.Structure):
    _fields_ = [("operand", EpHostTensor), ("operand_is_constant", ctypes.c_int),
                ("product_input_index", ctypes.c_int), ("product_is_graph_output", ctypes.c_int),
                ("extra_consumer", ctypes.c_int)]


class EpHostOutput(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("capacity", ctypes.c_size_t), ("dims", ctypes.c_int64 * 8),
                ("rank", ctypes.c_size_t), ("produced", ctypes.c_int)]


class EpHostError(RuntimeError):
    def __init__(self, code, message, trace=""):
        super().__init__(f"[{code}] {message}")
        self.code, self.message, self.trace = code, message, trace


class profiled:
    """Context manager: the next run_* call inside it is followed by the plugin's profiler; ``events`` then holds
    dicts with category, name, timestamp_us, duration_us and the event's arguments."""

    def __enter__(self):
        self._buf = ctypes.create_string_buffer(8192)
        lib = _load()
        lib.EpHostProfileNextRun.restype = None
        lib.EpHostProfileNextRun.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
        lib.EpHostProfileNextRun(self._buf, len(self._buf))
        self.events = []
        return self

    def __exit__(self, *exc):
        for line in self._buf.value.decode().splitlines():
            cat, name, ts, dur, *args = line.split("|")
            self.events.append(dict(category=int(cat), name=name, timestamp_us=int(ts), duration_us=int(dur),
                                    **dict(a.split("=", 1) for a in args)))
        _load().EpHostProfileNextRun(None, 0)
        return False


class EpHostRunStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in ("scratch_requests", "scratch_served", "scratch_bytes_max",
                                                "allocator_requests", "allocators_released", "scratch_freed",
                                                "ep_allocs", "arena_allocs")] + \
               [(n, ctypes.c_double) for n in ("host_us_per_compute", "wall_us_per_compute",
                                               "device_us_per_compute")] + [("timed_computes", ctypes.c_uint64)]


def last_run_stats() -> dict:
    """Allocator / scratch statistics (and timing figures, when asked for) of the last run_* call on this thread."""
    lib = _load()
    lib.EpHostLastRunStats.restype = None
    lib.EpHostLastRunStats.argtypes = [ctypes.POINTER(EpHostRunStats)]
    st = EpHostRunStats()
    lib.EpHostLastRunStats(ctypes.byref(st))
    return {n: getattr(st, n) for n, _ in EpHostRunStats._fields_}


class scratch_mode:
    """Context manager: how the host answers KernelContext_GetScratchBuffer inside it (0 serve, 1 fail with a status,
    2 succeed with NULL, 3 return a buffer that is only 64-byte aligned)."""

    def __init__(self, mode: int):
        self.mode = mode

    def __enter__(self):
        lib = _load()
        lib.EpHostSetScratchMode.restype = None
        lib.EpHostSetScratchMode.argtypes = [ctypes.c_int]
        lib.EpHostSetScratchMode(self.mode)
        return self

    def __exit__(self, *exc):
        _load().EpHostSetScratchMode(0)
        return False


def time_next_run(warmup: int, iters: int) -> None:
    """The next run_* call on this thread ends with ``warmup`` untimed and ``iters`` timed Compute calls on
    device-resident inputs; ``last_run_stats()`` then reports host / wall / device microseconds per call."""
    lib = _load()
    lib.EpHostTimeNextRun.restype = None
    lib.EpHostTimeNextRun.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.EpHostTimeNextRun(warmup, iters)


def available() -> bool:
    return SHIM.exists() and PLUGIN.exists()


def _load():
    lib = ctypes.CDLL(str(SHIM))
    lib.EpHostProbeFactory.restype = ctypes.c_int
    lib.EpHostProbeFactory.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p,
                                       ctypes.c_size_t]
    lib.EpHostSetSessionConfig.restype = None
    lib.EpHostSetSessionConfig.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    lib.EpHostRunMatMulNBits.restype = ctypes.c_int
    lib.EpHostRunMatMulNBits.argtypes = [
        ctypes.c_char_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
        ctypes.POINTER(EpHostTensor), ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int64),
        ctypes.POINTER(ctypes.c_size_t), ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p,
        ctypes.c_size_t]
    lib.EpHostRunMatMulNBitsAdd.restype = ctypes.c_int
    lib.EpHostRunMatMulNBitsAdd.argtypes = [
        ctypes.c_char_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
        ctypes.POINTER(EpHostTensor), ctypes.c_int, ctypes.POINTER(EpHostAddSpec), ctypes.c_void_p, ctypes.c_size_t,
        ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_size_t), ctypes.c_int, ctypes.c_char_p,
        ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t]
    lib.EpHostRunNode.restype = ctypes.c_int
    lib.EpHostRunNode.argtypes = [ctypes.c_char_p, ctypes.POINTER(EpHostNodeSpec), ctypes.POINTER(EpHostTensor),
                                  ctypes.c_int, ctypes.POINTER(EpHostOutput), ctypes.c_int, ctypes.c_char_p,
                                  ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t]
    return lib


def _tensors(arrays, names, constant):
    tensors = (EpHostTensor * len(arrays))()
    keep, mask = [], 0
    for i, (nm, arr) in enumerate(zip(names, arrays)):
        if arr is None:
            tensors[i] = EpHostTensor(None, None, 0, 0)
            continue
        arr = np.ascontiguousarray(arr)
        dims = (ctypes.c_int64 * max(arr.ndim, 1))(*arr.shape)
        keep += [arr, dims]
        ptr = arr.ctypes.data if arr.size else ctypes.addressof(dims)
        tensors[i] = EpHostTensor(ptr, ctypes.cast(dims, ctypes.POINTER(ctypes.c_int64)), arr.ndim,
                                  _ONNX_TYPE[arr.dtype])
        if nm in constant and i > 0:
            mask |= 1 << i
    return tensors, mask, keep


def run_node(op_type, attrs, schema_attrs, input_names, input_types, arrays, constant, out_shapes, skipped=(),
             repeat=1):
    """One node of the com.microsoft domain through the plugin EP.

    ``attrs``: dict name -> int | float | str.  ``arrays``: inputs in operator order (None = omitted).
    ``out_shapes``: expected shape of every schema output; outputs whose index is in ``skipped`` are optional outputs
    the graph does not use.  Returns ([outputs or None], trace)."""
    lib = _load()
    cattrs = (EpHostAttr * len(attrs))()
    for j, (k, v) in enumerate(attrs.items()):
        if isinstance(v, str):
            cattrs[j] = EpHostAttr(k.encode(), 2, 0, 0.0, v.encode())
        elif isinstance(v, float):
            cattrs[j] = EpHostAttr(k.encode(), 1, 0, v, None)
        else:
            cattrs[j] = EpHostAttr(k.encode(), 0, int(v), 0.0, None)
    sa = (ctypes.c_char_p * len(schema_attrs))(*[x.encode() for x in schema_attrs])
    inn = (ctypes.c_char_p * len(input_names))(*[x.encode() for x in input_names])
    itt = (ctypes.c_char_p * len(input_types))(*[x.encode() for x in input_types])
    tensors, mask, keep = _tensors(arrays, input_names, constant)
    dtype = arrays[0].dtype
    outs = (EpHostOutput * len(out_shapes))()
    bufs = []
    skip_mask = 0
    for o, shape in enumerate(out_shapes):
        if o in skipped:
            skip_mask |= 1 << o
            bufs.append(None)
            continue
        buf = np.empty(shape, dtype)
        bufs.append(buf)
        outs[o].data = buf.ctypes.data if buf.size else None
        outs[o].capacity = buf.nbytes
    spec = EpHostNodeSpec(op_type.encode(), cattrs, len(attrs), sa, len(schema_attrs), inn, itt, len(input_names),
                          len(out_shapes), skip_mask)
    trace, err = ctypes.create_string_buffer(512), ctypes.create_string_buffer(2048)
    rc = lib.EpHostRunNode(str(PLUGIN).encode(), ctypes.byref(spec), tensors, mask, outs, repeat, trace, len(trace),
                           err, len(err))
    if rc != 0:
        raise EpHostError(rc, err.value.decode(), trace.value.decode())
    for o, buf in enumerate(bufs):
        if buf is None:
            assert not outs[o].produced
            continue
        assert outs[o].produced
        assert tuple(outs[o].dims[i] for i in range(outs[o].rank)) == buf.shape
    del keep
    return bufs, trace.value.decode()


_MLP_INPUTS = ["A", "skip", "norm_scale", "gate_B", "gate_scales", "gate_bias", "up_B", "up_scales", "up_bias"]
_MLP_TYPES = ["T1", "T1", "T1", "T2", "T1", "T1", "T2", "T1", "T1"]
_QKV_INPUTS = ["A", "skip", "norm_scale", "q_B", "q_scales", "q_bias", "k_B", "k_scales", "k_bias", "v_B", "v_scales",
               "v_bias"]
_QKV_TYPES = ["T1", "T1", "T1", "T2", "T1", "T1", "T2", "T1", "T1", "T2", "T1", "T1"]


def run_mlp(N, K, bits, block_size, A, gate, up, skip=None, norm_scale=None, want_sum=False, activation="silu",
            epsilon=None, constant=None, repeat=1):
    """One MatMulNBitsMlp node; gate / up are (B, scales, bias or None).  Returns (Y, sum or None, trace)."""
    attrs = {"K": K, "N": N, "bits": bits, "block_size": block_size, "accuracy_level": 0, "activation": activation}
    if epsilon is not None:
        attrs["epsilon"] = float(epsilon)
    arrays = [A, skip, norm_scale, *gate, *up]
    constant = _MLP_INPUTS[2:] if constant is None else constant
    outs, trace = run_node("MatMulNBitsMlp", attrs, ["K", "N", "bits", "block_size", "accuracy_level", "activation",
                                                     "epsilon"], _MLP_INPUTS, _MLP_TYPES, arrays, constant,
                           [A.shape[:-1] + (N,), A.shape], skipped=() if want_sum else (1,), repeat=repeat)
    return outs[0], outs[1], trace


def run_qkv(Nq, Nkv, K, bits, block_size, A, q, k, v, skip=None, norm_scale=None, want_sum=False, epsilon=None,
            constant=None, repeat=1):
    """One MatMulNBitsQkv node.  Returns (Q, K, V, sum or None, trace)."""
    attrs = {"K": K, "Nq": Nq, "Nkv": Nkv, "bits": bits, "block_size": block_size, "accuracy_level": 0}
    if epsilon is not None:
        attrs["epsilon"] = float(epsilon)
    arrays = [A, skip, norm_scale, *q, *k, *v]
    constant = _QKV_INPUTS[2:] if constant is None else constant
    lead = A.shape[:-1]
    outs, trace = run_node("MatMulNBitsQkv", attrs, ["K", "Nq", "Nkv", "bits", "block_size", "accuracy_level",
                                                     "epsilon"], _QKV_INPUTS, _QKV_TYPES, arrays, constant,
                           [lead + (Nq,), lead + (Nkv,), lead + (Nkv,), A.shape], skipped=() if want_sum else (3,),
                           repeat=repeat)
    return outs[0], outs[1], outs[2], outs[3], trace


class session_config:
    """Context manager: session configuration entries (what OrtSessionOptions::AddConfigEntry sets) for the runs
    inside the block."""

    def __init__(self, **entries):
        self.entries = {k.replace("__", "."): str(v) for k, v in entries.items()}

    def __enter__(self):
        lib = _load()
        for k, v in self.entries.items():
            lib.EpHostSetSessionConfig(k.encode(), v.encode())
        return self

    def __exit__(self, *exc):
        lib = _load()
        for k in self.entries:
            lib.EpHostSetSessionConfig(k.encode(), None)
        return False


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


def run_matmul_nbits_add(N, K, bits, block_size, A, B, scales, operand, zero_points=None, bias=None,
                         constant=("B", "scales", "zero_points", "bias"), operand_is_constant=True,
                         product_input_index=0, product_is_graph_output=False, extra_consumer=False, repeat=1):
    """MatMulNBits followed by Add(product, operand) through the plugin EP's compile path.  Returns (sum, trace);
    raises EpHostError with code NOT_FUSED when the plugin leaves the pair un-fused."""
    lib = _load()
    names = ["A", "B", "scales", "zero_points", "g_idx", "bias"]
    tensors, mask, keep = _tensors([A, B, scales, zero_points, None, bias], names, constant)
    op_t, _, keep2 = _tensors([operand], ["operand"], ())
    add = EpHostAddSpec(op_t[0], int(operand_is_constant), int(product_input_index), int(product_is_graph_output),
                        int(extra_consumer))
    y = np.empty(A.shape[:-1] + (N,), dtype=A.dtype)
    y_dims = (ctypes.c_int64 * 8)()
    y_rank = ctypes.c_size_t(0)
    trace, err = ctypes.create_string_buffer(512), ctypes.create_string_buffer(2048)
    rc = lib.EpHostRunMatMulNBitsAdd(str(PLUGIN).encode(), N, K, bits, block_size, tensors, mask, ctypes.byref(add),
                                     y.ctypes.data if y.size else None, y.nbytes, y_dims, ctypes.byref(y_rank),
                                     repeat, trace, len(trace), err, len(err))
    del keep, keep2
    if rc != 0:
        raise EpHostError(rc, err.value.decode(), trace.value.decode())
    assert tuple(y_dims[i] for i in range(y_rank.value)) == y.shape
    return y, trace.value.decode()
