"""TEST INFRASTRUCTURE (see oracle/__init__.py): a pure-Python reader of ONNX protobuf files.

An independent restatement of what the reference's importer extracts from a ModelProto
(schema/src/onnx_import/transform.rs:76-260; field numbers from
schema/src/onnx/protos/onnx.proto), used to cross-check the native reader and to hand a loaded
`.onnx` graph, with its initializers as numpy arrays, to the graph walker of this package.
Pinned by: files exported by PyTorch's own ONNX serialiser (tests/golden/*.onnx) whose outputs
PyTorch computed, and round trips through the independent writer of rmlk_amd.onnx_io.
"""
from __future__ import annotations

import os
import struct
from dataclasses import dataclass, field
from typing import Dict, List

import numpy as np

DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32,
          7: np.int64, 9: np.bool_, 10: np.float16, 11: np.float64, 12: np.uint32, 13: np.uint64}


def _varint(b, i):
    v = 0
    shift = 0
    while True:
        c = b[i]
        i += 1
        v |= (c & 0x7F) << shift
        shift += 7
        if c < 0x80:
            return v, i


def _fields(b):
    """[(field number, wire type, int | bytes)] of one message."""
    out = []
    i = 0
    n = len(b)
    while i < n:
        key, i = _varint(b, i)
        num, wire = key >> 3, key & 7
        if wire == 0:
            v, i = _varint(b, i)
        elif wire == 1:
            v = b[i:i + 8]
            i += 8
        elif wire == 2:
            ln, i = _varint(b, i)
            v = b[i:i + ln]
            i += ln
        elif wire == 5:
            v = b[i:i + 4]
            i += 4
        else:
            raise ValueError(f"wire type {wire}")
        out.append((num, wire, v))
    return out


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _varints(wire, v):
    if wire == 0:
        return [_signed(v)]
    out = []
    i = 0
    while i < len(v):
        x, i = _varint(v, i)
        out.append(_signed(x))
    return out


def _fixed(wire, v, fmt, size):
    if wire == 2:
        return list(struct.unpack("<%d%s" % (len(v) // size, fmt), v))
    return [struct.unpack("<" + fmt, v)[0]]


def _tensor(b, base_dir):
    dims, dtype, name, raw = [], 0, "", None
    f32, i32, i64, f64, u64 = [], [], [], [], []
    ext, external = {}, False
    for num, wire, v in _fields(b):
        if num == 1:
            dims += _varints(wire, v)
        elif num == 2:
            dtype = v
        elif num == 4:
            f32 += _fixed(wire, v, "f", 4)
        elif num == 5:
            i32 += _varints(wire, v)
        elif num == 7:
            i64 += _varints(wire, v)
        elif num == 8:
            name = bytes(v).decode()
        elif num == 9:
            raw = bytes(v)
        elif num == 10:
            f64 += _fixed(wire, v, "d", 8)
        elif num == 11:
            u64 += _varints(wire, v)
        elif num == 13:
            kv = {n: bytes(x).decode() for n, _, x in _fields(v)}
            ext[kv.get(1)] = kv.get(2)
        elif num == 14:
            external = v == 1
    dt = np.dtype(DTYPES[dtype])
    if external:
        path = os.path.join(base_dir or "", ext["location"])
        with open(path, "rb") as f:
            f.seek(int(ext.get("offset", 0)))
            raw = f.read(int(ext["length"])) if "length" in ext else f.read()
    if raw is not None:
        arr = np.frombuffer(raw, dtype=dt.newbyteorder("<")).astype(dt)
    elif dtype == 1:
        arr = np.array(f32, dtype=dt)
    elif dtype == 11:
        arr = np.array(f64, dtype=dt)
    elif dtype == 7:
        arr = np.array(i64, dtype=dt)
    elif dtype in (12, 13):
        arr = np.array([x & ((1 << 64) - 1) for x in u64], dtype=np.uint64).astype(dt)
    elif dtype == 10:
        arr = np.array(i32, dtype=np.int64).astype(np.uint16).view(np.float16)
    else:
        arr = np.array(i32, dtype=np.int64).astype(dt)
    return name, arr.reshape(dims)


def _value_info(b):
    name, dtype, dims = "", 0, []
    for num, _, v in _fields(b):
        if num == 1:
            name = bytes(v).decode()
        elif num == 2:
            for n2, _, t in _fields(v):
                if n2 != 1:
                    continue
                for n3, _, x in _fields(t):
                    if n3 == 1:
                        dtype = x
                    elif n3 == 2:
                        for n4, _, d in _fields(x):
                            if n4 == 1:
                                val = 0
                                for n5, _, y in _fields(d):
                                    if n5 == 1:
                                        val = y
                                dims.append(val)
    return name, dtype, dims


def _attribute(b, base_dir):
    name, typ = "", 0
    got = {}
    floats, ints = [], []
    for num, wire, v in _fields(b):
        if num == 1:
            name = bytes(v).decode()
        elif num == 2:
            got[1] = struct.unpack("<f", v)[0]
        elif num == 3:
            got[2] = _signed(v)
        elif num == 4:
            got[3] = bytes(v).decode()
        elif num == 5:
            got[4] = _tensor(v, base_dir)[1]
        elif num == 7:
            floats += _fixed(wire, v, "f", 4)
            got.setdefault(6, floats)
        elif num == 8:
            ints += _varints(wire, v)
            got.setdefault(7, ints)
        elif num == 20:
            typ = v
    if typ == 0 and got:
        typ = sorted(got)[0]
    if typ == 6:
        return name, [float(x) for x in floats]
    if typ == 7:
        return name, [int(x) for x in ints]
    return name, got.get(typ)


@dataclass
class Node:
    op: str
    inputs: List[str]
    outputs: List[str]
    attrs: Dict[str, object] = field(default_factory=dict)


@dataclass
class LoadedGraph:
    """The fields oracle.graph.run_graph reads."""
    nodes: List[Node]
    inputs: Dict[str, tuple]
    initializers: Dict[str, np.ndarray]
    outputs: List[str]


def read_onnx(path_or_bytes, base_dir=None) -> LoadedGraph:
    if isinstance(path_or_bytes, (bytes, bytearray, memoryview)):
        data = bytes(path_or_bytes)
    else:
        base_dir = os.path.dirname(os.fspath(path_or_bytes)) if base_dir is None else base_dir
        with open(path_or_bytes, "rb") as f:
            data = f.read()
    graph = None
    for num, wire, v in _fields(memoryview(data)):
        if num == 7 and wire == 2:
            graph = v
    if graph is None:
        raise ValueError("the model does not have a graph")
    nodes, inits, inputs, outputs = [], {}, {}, []
    raw_nodes, raw_inputs = [], []
    for num, wire, v in _fields(graph):
        if num == 1:
            raw_nodes.append(v)
        elif num == 5:
            name, arr = _tensor(v, base_dir)
            inits[name] = arr
        elif num == 11:
            raw_inputs.append(v)
        elif num == 12:
            outputs.append(_value_info(v)[0])
    for v in raw_inputs:
        name, dtype, dims = _value_info(v)
        if name not in inits:
            inputs[name] = (dtype, dims)
    for v in raw_nodes:
        ins, outs, op, attrs = [], [], "", {}
        for num, _, x in _fields(v):
            if num == 1:
                ins.append(bytes(x).decode())
            elif num == 2:
                outs.append(bytes(x).decode())
            elif num == 4:
                op = bytes(x).decode()
            elif num == 5:
                k, val = _attribute(x, base_dir)
                attrs[k] = val
        nodes.append(Node(op, ins, outs, attrs))
    return LoadedGraph(nodes, inputs, inits, outputs)
