"""Minimal ONNX (protobuf) writer and reader for graphs made of com.microsoft::MatMulNBits nodes.

The reference produces such models with its Python quantisation tool (MatMulNBitsQuantizer.quantize_matmul,
onnxruntime/python/tools/quantization/matmul_nbits_quantizer.py:1034-1130: a MatMul with a constant weight becomes a
MatMulNBits node with initializers <name>_Q4 / _scales / _zero_points and attributes K, N, bits, block_size). That
tool needs the `onnx` package; this module writes the same wire format directly: protobuf wire types 0 (varint) and 2
(length-delimited) with the field numbers of onnx.proto (ModelProto, GraphProto, NodeProto, AttributeProto,
TensorProto, ValueInfoProto, TypeProto, TensorShapeProto, OperatorSetIdProto). Fields are emitted in field-number
order and repeated int64 dims unpacked, which is what the protobuf runtime emits for these proto2 messages, so a
model written here is byte-identical to the one `onnx.helper` produces from the same content.
"""
from __future__ import annotations

from typing import Iterable, Optional, Sequence, Union

import numpy as np

FLOAT, UINT8, INT32, INT64, FLOAT16 = 1, 2, 6, 7, 10  # TensorProto.DataType
_NP_TO_ONNX = {np.dtype(np.float32): FLOAT, np.dtype(np.uint8): UINT8, np.dtype(np.int32): INT32,
               np.dtype(np.int64): INT64, np.dtype(np.float16): FLOAT16}
_ATTR_INT = 2  # AttributeProto.AttributeType.INT


# ---------------------------------------------------------------------------------------------- wire format
def _varint(n: int) -> bytes:
    if n < 0:
        n += 1 << 64  # two's complement, as protobuf encodes negative int64
    out = bytearray()
    while True:
        b = n & 0x7F
        n >>= 7
        if n:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _int(field: int, value: int) -> bytes:
    return _varint(field << 3) + _varint(value)


def _bytes(field: int, payload: bytes) -> bytes:
    return _varint((field << 3) | 2) + _varint(len(payload)) + payload


def _str(field: int, s: str) -> bytes:
    return _bytes(field, s.encode("utf-8"))


# ---------------------------------------------------------------------------------------------- messages
def tensor(name: str, array: np.ndarray) -> bytes:
    """TensorProto with raw_data (little endian), as numpy_helper.from_array writes it."""
    a = np.ascontiguousarray(array)
    if a.dtype not in _NP_TO_ONNX:
        raise TypeError(f"unsupported tensor dtype {a.dtype}")
    out = b"".join(_int(1, d) for d in a.shape)           # dims
    out += _int(2, _NP_TO_ONNX[a.dtype])                  # data_type
    out += _str(8, name)                                  # name
    out += _bytes(9, a.astype(a.dtype.newbyteorder("<"), copy=False).tobytes())  # raw_data
    return out


def attribute_int(name: str, value: int) -> bytes:
    return _str(1, name) + _int(3, value) + _int(20, _ATTR_INT)


def node(op_type: str, inputs: Sequence[str], outputs: Sequence[str], name: str = "", domain: str = "",
         int_attrs: Sequence[tuple] = ()) -> bytes:
    out = b"".join(_str(1, i) for i in inputs)            # omitted optional inputs are empty strings
    out += b"".join(_str(2, o) for o in outputs)
    if name:
        out += _str(3, name)
    out += _str(4, op_type)
    out += b"".join(_bytes(5, attribute_int(k, v)) for k, v in int_attrs)
    if domain:
        out += _str(7, domain)
    return out


def value_info(name: str, elem_type: int, shape: Sequence[Union[int, str]]) -> bytes:
    dims = b""
    for d in shape:
        dims += _bytes(1, _str(2, d) if isinstance(d, str) else _int(1, d))   # dim_param | dim_value
    tensor_type = _int(1, elem_type) + _bytes(2, dims)
    return _str(1, name) + _bytes(2, _bytes(1, tensor_type))


def graph(name: str, nodes: Iterable[bytes], initializers: Iterable[bytes], inputs: Iterable[bytes],
          outputs: Iterable[bytes]) -> bytes:
    out = b"".join(_bytes(1, n) for n in nodes)
    out += _str(2, name)
    out += b"".join(_bytes(5, t) for t in initializers)
    out += b"".join(_bytes(11, v) for v in inputs)
    out += b"".join(_bytes(12, v) for v in outputs)
    return out


def model(graph_bytes: bytes, opsets: Sequence[tuple], ir_version: int = 10, producer_name: str = "") -> bytes:
    out = _int(1, ir_version)
    if producer_name:
        out += _str(2, producer_name)
    out += _bytes(7, graph_bytes)
    for domain, version in opsets:
        out += _bytes(8, (_str(1, domain) if domain else b"") + _int(2, version))
    return out


# ---------------------------------------------------------------------------------------------- MatMulNBits
def matmul_nbits_node(a: str, y: str, prefix: str, K: int, N: int, bits: int, block_size: int,
                      has_zero_points: bool, bias: Optional[str] = None, accuracy_level: Optional[int] = None,
                      name: str = "") -> bytes:
    """The node the reference's quantiser emits for one MatMul: inputs A, <prefix>_Q<bits>, <prefix>_scales,
    [<prefix>_zero_points], ['' for g_idx, bias]."""
    inputs = [a, f"{prefix}_Q{bits}", f"{prefix}_scales"]
    if has_zero_points or bias:
        inputs.append(f"{prefix}_zero_points" if has_zero_points else "")
    if bias:
        inputs += ["", bias]
    attrs = [("K", K), ("N", N), ("bits", bits), ("block_size", block_size)]
    if accuracy_level is not None:
        attrs.append(("accuracy_level", accuracy_level))
    return node("MatMulNBits", inputs, [y], name=name, domain="com.microsoft", int_attrs=attrs)


def matmul_nbits_model(B: np.ndarray, scales: np.ndarray, zero_points: Optional[np.ndarray], K: int, N: int,
                       bits: int, block_size: int, bias: Optional[np.ndarray] = None, prefix: str = "W",
                       graph_name: str = "matmul_nbits", onnx_opset: int = 21,
                       accuracy_level: Optional[int] = None) -> bytes:
    """A one-node model  Y[M, N] = MatMulNBits(A[M, K])  over the given quantised operands (canonical layout)."""
    elem = _NP_TO_ONNX[np.dtype(scales.dtype)]
    inits = [tensor(f"{prefix}_Q{bits}", np.asarray(B, np.uint8)), tensor(f"{prefix}_scales", scales)]
    if zero_points is not None:
        inits.append(tensor(f"{prefix}_zero_points", np.asarray(zero_points, np.uint8)))
    if bias is not None:
        inits.append(tensor(f"{prefix}_bias", np.asarray(bias, scales.dtype)))
    n = matmul_nbits_node("A", "Y", prefix, K, N, bits, block_size, zero_points is not None,
                          bias=f"{prefix}_bias" if bias is not None else None, accuracy_level=accuracy_level,
                          name=f"{prefix}_MatMulNBits")
    g = graph(graph_name, [n], inits, [value_info("A", elem, ["M", K])], [value_info("Y", elem, ["M", N])])
    return model(g, [("", onnx_opset), ("com.microsoft", 1)], producer_name="onnxruntime_amd")


# ---------------------------------------------------------------------------------------------- reader
def parse(data: bytes) -> list:
    """Schema-less decode of one message: [(field, wire_type, value)], value = int or bytes."""
    out, i = [], 0
    while i < len(data):
        key, i = _read_varint(data, i)
        field, wt = key >> 3, key & 7
        if wt == 0:
            v, i = _read_varint(data, i)
        elif wt == 2:
            ln, i = _read_varint(data, i)
            v = data[i:i + ln]
            i += ln
        elif wt == 5:
            v = data[i:i + 4]
            i += 4
        elif wt == 1:
            v = data[i:i + 8]
            i += 8
        else:
            raise ValueError(f"unsupported wire type {wt}")
        out.append((field, wt, v))
    return out


def _read_varint(data: bytes, i: int):
    r = s = 0
    while True:
        c = data[i]
        i += 1
        r |= (c & 0x7F) << s
        s += 7
        if not c & 0x80:
            return r, i


def read_model(data: bytes) -> dict:
    """Decodes the parts of a model this module writes: nodes (with int attributes), initializers, opsets."""
    m = {"ir_version": None, "opsets": [], "nodes": [], "initializers": {}, "inputs": [], "outputs": []}
    for f, _, v in parse(data):
        if f == 1:
            m["ir_version"] = v
        elif f == 8:
            d = {ff: vv for ff, _, vv in parse(v)}
            m["opsets"].append((d.get(1, b"").decode(), d.get(2, 0)))
        elif f == 7:
            for gf, _, gv in parse(v):
                if gf == 1:
                    nd = {"inputs": [], "outputs": [], "attrs": {}, "name": "", "domain": "", "op_type": ""}
                    for nf, _, nv in parse(gv):
                        if nf == 1:
                            nd["inputs"].append(nv.decode())
                        elif nf == 2:
                            nd["outputs"].append(nv.decode())
                        elif nf == 3:
                            nd["name"] = nv.decode()
                        elif nf == 4:
                            nd["op_type"] = nv.decode()
                        elif nf == 7:
                            nd["domain"] = nv.decode()
                        elif nf == 5:
                            a = {af: av for af, _, av in parse(nv)}
                            nd["attrs"][a[1].decode()] = a.get(3)
                    m["nodes"].append(nd)
                elif gf == 5:
                    dims, dt, name, raw = [], None, "", b""
                    for tf, _, tv in parse(gv):
                        if tf == 1:
                            dims.append(tv)
                        elif tf == 2:
                            dt = tv
                        elif tf == 8:
                            name = tv.decode()
                        elif tf == 9:
                            raw = tv
                    np_dt = {v2: k for k, v2 in _NP_TO_ONNX.items()}[dt]
                    m["initializers"][name] = np.frombuffer(raw, dtype=np_dt).reshape(dims)
                elif gf in (11, 12):
                    d = {ff: vv for ff, _, vv in parse(gv)}
                    m["inputs" if gf == 11 else "outputs"].append(d[1].decode())
    return m
