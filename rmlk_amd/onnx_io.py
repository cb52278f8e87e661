"""ONNX files in and out.

Reading is native (`rmlk_graph_load_onnx*` in librmlk_hip.so, the counterpart of the reference's
`Builder::from_onnx_path`, runtime/src/core/instance.rs:187-196). Writing is a small protobuf
encoder for the graphs this package builds, so that benchmark and fixture graphs can be stored as
`.onnx` without the `onnx` package; field numbers follow schema/src/onnx/protos/onnx.proto of the
reference (ModelProto.graph = 7, GraphProto node = 1 / initializer = 5 / input = 11 / output = 12,
NodeProto input = 1 / output = 2 / name = 3 / op_type = 4 / attribute = 5, AttributeProto name = 1 /
f = 2 / i = 3 / s = 4 / t = 5 / floats = 7 / ints = 8 / type = 20, TensorProto dims = 1 /
data_type = 2 / name = 8 / raw_data = 9 / external_data = 13 / data_location = 14).
"""
from __future__ import annotations

import ctypes
import json
import os
import struct
from typing import Optional

import numpy as np

from ._lib import lib
from .runtime import Graph, NodeDesc, ONNX_DTYPES, _check, onnx_dtype


# ---- protobuf encoding ---------------------------------------------------------------------------

def _varint(v: int) -> bytes:
    v &= (1 << 64) - 1          # negative int64 as two's complement, 10 bytes
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field: int, wire: int) -> bytes:
    return _varint((field << 3) | wire)


def _f_varint(field: int, v: int) -> bytes:
    return _key(field, 0) + _varint(v)


def _f_bytes(field: int, payload: bytes) -> bytes:
    return _key(field, 2) + _varint(len(payload)) + payload


def _f_string(field: int, s: str) -> bytes:
    return _f_bytes(field, s.encode())


def _tensor(name: Optional[str], arr: np.ndarray, external=None) -> bytes:
    arr = np.asarray(arr, order="C")
    out = b"".join(_f_varint(1, int(d)) for d in arr.shape)
    out += _f_varint(2, onnx_dtype(arr.dtype))
    if name is not None:
        out += _f_string(8, name)
    raw = arr.astype(arr.dtype.newbyteorder("<"), copy=False).tobytes()
    if external is not None:
        location, fh = external
        offset = fh.tell()
        fh.write(raw)
        for k, v in (("location", location), ("offset", str(offset)), ("length", str(len(raw)))):
            out += _f_bytes(13, _f_string(1, k) + _f_string(2, v))
        out += _f_varint(14, 1)          # DataLocation.EXTERNAL
    else:
        out += _f_bytes(9, raw)
    return out


def _attribute(name: str, value) -> bytes:
    out = _f_string(1, name)
    if isinstance(value, (bool, int, np.integer)):
        out += _f_varint(3, int(value)) + _f_varint(20, 2)
    elif isinstance(value, float):
        out += _key(2, 5) + struct.pack("<f", value) + _f_varint(20, 1)
    elif isinstance(value, str):
        out += _f_bytes(4, value.encode()) + _f_varint(20, 3)
    elif isinstance(value, np.ndarray):
        out += _f_bytes(5, _tensor(None, value)) + _f_varint(20, 4)
    elif isinstance(value, (list, tuple)) and any(isinstance(v, float) for v in value):
        out += b"".join(_key(7, 5) + struct.pack("<f", float(v)) for v in value) + _f_varint(20, 6)
    elif isinstance(value, (list, tuple)):
        out += b"".join(_f_varint(8, int(v)) for v in value) + _f_varint(20, 7)
    else:
        raise TypeError(f"unsupported attribute type for {name}: {type(value)}")
    return out


def _value_info(name: str, dtype: int, dims) -> bytes:
    shape = b""
    for i, d in enumerate(dims):
        # 0 is this package's spelling of a dynamic dim: written as a symbolic dim_param
        dim = _f_varint(1, int(d)) if int(d) > 0 else _f_string(2, f"{name}_dim{i}")
        shape += _f_bytes(1, dim)
    tensor_type = _f_varint(1, dtype) + _f_bytes(2, shape)
    return _f_string(1, name) + _f_bytes(2, _f_bytes(1, tensor_type))


def graph_to_onnx_bytes(graph: Graph, external=None, external_threshold: int = 1024,
                        opset: int = 14, ir_version: int = 10) -> bytes:
    """Serialise a built Graph as an ONNX ModelProto. With `external = (file name, open binary
    file)` initializers of at least `external_threshold` bytes go to that file."""
    g = b""
    for i, node in enumerate(graph.nodes):
        n = b"".join(_f_string(1, x) for x in node.inputs)
        n += b"".join(_f_string(2, x) for x in node.outputs)
        n += _f_string(3, f"node_{i}") + _f_string(4, node.op)
        for k in sorted(node.attrs):
            n += _f_bytes(5, _attribute(k, node.attrs[k]))
        g += _f_bytes(1, n)
    g += _f_string(2, "rmlk_amd_graph")
    for name, arr in graph.initializers.items():
        ext = external if external is not None and np.asarray(arr).nbytes >= external_threshold else None
        g += _f_bytes(5, _tensor(name, arr, ext))
    for name, (dtype, dims) in graph.inputs.items():
        g += _f_bytes(11, _value_info(name, dtype, dims))
    for name in graph.outputs:
        # element type and shape of outputs are inferred at run time; the value info carries the
        # name and an untyped tensor type only when nothing is known
        g += _f_bytes(12, _f_string(1, name))
    model = _f_varint(1, ir_version) + _f_string(2, "rmlk_amd") + _f_bytes(7, g)
    model += _f_bytes(8, _f_string(1, "") + _f_varint(2, opset))
    return model


def save_onnx(graph: Graph, path: str, external_data: bool = False,
              external_threshold: int = 1024) -> None:
    """Write `path` (and `path + ".data"` holding the large initializers when external_data)."""
    if external_data:
        location = os.path.basename(path) + ".data"
        with open(os.path.join(os.path.dirname(path) or ".", location), "wb") as fh:
            data = graph_to_onnx_bytes(graph, (location, fh), external_threshold)
    else:
        data = graph_to_onnx_bytes(graph)
    with open(path, "wb") as f:
        f.write(data)


# ---- loading (native reader) -------------------------------------------------------------------

def describe(handle) -> dict:
    """The native graph as a dict (inputs, initializers with byte hashes, nodes, outputs)."""
    need = lib().rmlk_graph_describe(handle, None, 0)
    buf = ctypes.create_string_buffer(int(need))
    lib().rmlk_graph_describe(handle, buf, need)
    return json.loads(buf.value.decode())


def _graph_from_handle(handle) -> Graph:
    d = describe(handle)
    nodes = [NodeDesc(n["op"], list(n["inputs"]), list(n["outputs"]), dict(n["attrs"]))
             for n in d["nodes"]]
    inputs = {i["name"]: (i["dtype"], list(i["dims"])) for i in d["inputs"]}
    # initializer payloads stay on the native side; a CPU checker reads the file itself
    return Graph(handle, nodes, inputs, {}, list(d["outputs"]))


def load_onnx(path: str) -> Graph:
    """ref: Builder::from_onnx_path (runtime/src/core/instance.rs:187-196)."""
    h = ctypes.c_void_p()
    _check(lib().rmlk_graph_load_onnx_file(os.fspath(path).encode(), ctypes.byref(h)),
           f"load_onnx({path})", True)
    return _graph_from_handle(h)


def load_onnx_bytes(data: bytes, base_dir: Optional[str] = None) -> Graph:
    """ref: graph_from_onnx_bytes (schema/src/onnx_import/transform.rs:249-258)."""
    h = ctypes.c_void_p()
    buf = ctypes.create_string_buffer(data, len(data))
    _check(lib().rmlk_graph_load_onnx(buf, len(data), base_dir.encode() if base_dir else None,
                                      ctypes.byref(h)), "load_onnx_bytes", True)
    return _graph_from_handle(h)


__all__ = ["graph_to_onnx_bytes", "save_onnx", "load_onnx", "load_onnx_bytes", "describe",
           "ONNX_DTYPES"]
