"""In-memory form and on-disk writer/reader of the sparse-convolution ONNX dialect.

The dialect is the one the reference's exporters emit and its loader reads:
`libraries/3DSparseConvolution/src/onnx-parser.cpp:101-231` (consumer) and
`CUDA-CenterPoint/qat/onnx_export/exptool.py:115-138,178-205,223-256` (producer).  Neither the
`onnx` package nor libprotobuf is needed: the few message types involved are written and parsed
directly in protobuf wire format, with the field numbers of
`libraries/3DSparseConvolution/src/onnx/onnx-ml.proto:116-176,181-215,342-382,441-462,486-587`.

Op types: SparseConvolution, Add / QuantAdd, Relu, ScatterDense, Reshape, Transpose.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import Dict, List, Sequence, Union

import numpy as np

AttrValue = Union[int, float, str, Sequence[int], Sequence[float]]

ONNX_FLOAT16 = 10


@dataclass
class Node:
    op_type: str
    name: str
    inputs: List[str]
    outputs: List[str]
    attrs: Dict[str, AttrValue] = field(default_factory=dict)


@dataclass
class Graph:
    """One `scn` graph: tensor names are strings, weights/biases are fp16 initializers."""
    inputs: List[str]
    outputs: List[str]
    nodes: List[Node]
    initializers: Dict[str, np.ndarray]
    name: str = "scn"


# --------------------------------------------------------------------------- wire-format writer
def _varint(v: int) -> bytes:
    if v < 0:
        v += 1 << 64
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _tag(fieldno: int, wt: int) -> bytes:
    return _varint((fieldno << 3) | wt)


def _ld(fieldno: int, payload: bytes) -> bytes:
    return _tag(fieldno, 2) + _varint(len(payload)) + payload


def _vi(fieldno: int, v: int) -> bytes:
    return _tag(fieldno, 0) + _varint(int(v))


def _attr(name: str, value: AttrValue) -> bytes:
    out = _ld(1, name.encode())
    if isinstance(value, (bool, np.bool_)):
        value = int(value)
    if isinstance(value, (int, np.integer)):
        out += _vi(3, int(value)) + _vi(20, 2)
    elif isinstance(value, (float, np.floating)):
        out += _tag(2, 5) + struct.pack("<f", float(value)) + _vi(20, 1)
    elif isinstance(value, (str, bytes)):
        out += _ld(4, value.encode() if isinstance(value, str) else value) + _vi(20, 3)
    else:
        seq = list(value)
        if len(seq) and all(isinstance(x, (float, np.floating)) for x in seq):
            out += _ld(7, b"".join(struct.pack("<f", float(x)) for x in seq)) + _vi(20, 6)
        else:
            out += _ld(8, b"".join(_varint(int(x)) for x in seq)) + _vi(20, 7)
    return out


def _tensor(name: str, arr: np.ndarray) -> bytes:
    arr = np.ascontiguousarray(arr, dtype=np.float16)
    out = b"".join(_vi(1, d) for d in arr.shape)
    out += _vi(2, ONNX_FLOAT16) + _ld(8, name.encode()) + _ld(9, arr.tobytes())
    return out


def serialize(graph: Graph, float_lists_attr: Sequence[str] = ("weight_dynamic_ranges",)) -> bytes:
    """Graph -> ModelProto bytes (ir_version 6, opset 11, producer "pytorch", graph name "scn")."""
    g = b""
    for n in graph.nodes:
        nb = b"".join(_ld(1, i.encode()) for i in n.inputs)
        nb += b"".join(_ld(2, o.encode()) for o in n.outputs)
        nb += _ld(3, n.name.encode()) + _ld(4, n.op_type.encode())
        for k, v in n.attrs.items():
            if k in float_lists_attr:
                v = [float(x) for x in v]
            nb += _ld(5, _attr(k, v))
        g += _ld(1, nb)
    g += _ld(2, graph.name.encode())
    for name, arr in graph.initializers.items():
        g += _ld(5, _tensor(name, arr))
    for name in graph.inputs:
        g += _ld(11, _ld(1, name.encode()))
    for name in graph.outputs:
        g += _ld(12, _ld(1, name.encode()))
    model = _vi(1, 6) + _ld(2, b"pytorch") + _ld(7, g) + _ld(8, _ld(1, b"") + _vi(2, 11))
    return model


def save(graph: Graph, path: str) -> None:
    with open(path, "wb") as f:
        f.write(serialize(graph))


# --------------------------------------------------------------------------- wire-format reader
def _read_varint(buf: bytes, pos: int):
    v = 0
    shift = 0
    while True:
        b = buf[pos]
        pos += 1
        v |= (b & 0x7F) << shift
        if not b & 0x80:
            break
        shift += 7
    return v, pos


def _fields(buf: bytes):
    pos = 0
    n = len(buf)
    while pos < n:
        key, pos = _read_varint(buf, pos)
        fno, wt = key >> 3, key & 7
        if wt == 0:
            v, pos = _read_varint(buf, pos)
        elif wt == 1:
            v = buf[pos:pos + 8]
            pos += 8
        elif wt == 2:
            ln, pos = _read_varint(buf, pos)
            v = buf[pos:pos + ln]
            pos += ln
        elif wt == 5:
            v = buf[pos:pos + 4]
            pos += 4
        else:
            raise ValueError(f"unsupported wire type {wt}")
        yield fno, wt, v


def _s64(v: int) -> int:
    return v - (1 << 64) if v >= (1 << 63) else v


def _parse_attr(buf: bytes):
    name, atype = "", 0
    f = i = s = None
    floats: List[float] = []
    ints: List[int] = []
    for fno, wt, v in _fields(buf):
        if fno == 1:
            name = v.decode()
        elif fno == 2:
            f = struct.unpack("<f", v)[0]
        elif fno == 3:
            i = _s64(v)
        elif fno == 4:
            s = v.decode()
        elif fno == 7:
            if wt == 2:
                floats += list(struct.unpack(f"<{len(v) // 4}f", v))
            else:
                floats.append(struct.unpack("<f", v)[0])
        elif fno == 8:
            if wt == 2:
                p = 0
                while p < len(v):
                    x, p = _read_varint(v, p)
                    ints.append(_s64(x))
            else:
                ints.append(_s64(v))
        elif fno == 20:
            atype = v
    if atype == 1 or (atype == 0 and f is not None):
        return name, f
    if atype == 2 or (atype == 0 and i is not None):
        return name, i
    if atype == 3 or (atype == 0 and s is not None):
        return name, s
    if atype == 6 or (atype == 0 and floats):
        return name, floats
    return name, ints


def parse(data: bytes) -> Graph:
    graph_bytes = b""
    for fno, _, v in _fields(data):
        if fno == 7:
            graph_bytes = v
    g = Graph([], [], [], {})
    for fno, _, v in _fields(graph_bytes):
        if fno == 1:
            node = Node("", "", [], [])
            for nf, _, nv in _fields(v):
                if nf == 1:
                    node.inputs.append(nv.decode())
                elif nf == 2:
                    node.outputs.append(nv.decode())
                elif nf == 3:
                    node.name = nv.decode()
                elif nf == 4:
                    node.op_type = nv.decode()
                elif nf == 5:
                    k, val = _parse_attr(nv)
                    node.attrs[k] = val
            g.nodes.append(node)
        elif fno == 2:
            g.name = v.decode()
        elif fno == 5:
            dims: List[int] = []
            dtype, name, raw = 0, "", b""
            for tf, twt, tv in _fields(v):
                if tf == 1:
                    if twt == 2:
                        p = 0
                        while p < len(tv):
                            x, p = _read_varint(tv, p)
                            dims.append(x)
                    else:
                        dims.append(tv)
                elif tf == 2:
                    dtype = tv
                elif tf == 8:
                    name = tv.decode()
                elif tf == 9:
                    raw = tv
            if dtype != ONNX_FLOAT16:
                raise ValueError(f"initializer {name}: only FLOAT16 raw_data is part of the dialect")
            g.initializers[name] = np.frombuffer(raw, dtype=np.float16).reshape(dims).copy()
        elif fno in (11, 12):
            for vf, _, vv in _fields(v):
                if vf == 1:
                    (g.inputs if fno == 11 else g.outputs).append(vv.decode())
    return g


def load(path: str) -> Graph:
    with open(path, "rb") as f:
        return parse(f.read())
