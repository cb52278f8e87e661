"""Graph builder and sessions over the C ABI of include/rmlk_runtime.h.

Python mirror of the reference's public surface on this path:
  GraphBuilder   <-> schema::GraphBuilder          (schema/src/builder.rs:49-260)
  Builder        <-> runtime::core::Builder        (runtime/src/core/instance.rs:131-222)
  ModelInstance  <-> runtime::core::ModelInstance  (runtime/src/core/instance.rs:89-119)

The executor, the operator dispatch and the kernels are native (librmlk_hip.so); this module only
marshals numpy arrays in and out. `Graph` also keeps a plain-Python description of its nodes so
that a test can hand the same graph to a CPU checker.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np

from ._lib import RmlkError, lib

ONNX_DTYPES = {
    1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32, 7: np.int64,
    9: np.bool_, 10: np.float16, 11: np.float64, 12: np.uint32, 13: np.uint64,
}
NP_TO_ONNX = {np.dtype(v): k for k, v in ONNX_DTYPES.items()}


class InferenceError(RmlkError):
    """ref: runtime/src/core/error.rs:12-14"""


class GraphBuildError(RmlkError):
    """ref: schema/src/builder.rs:11-22"""


def _check(status: int, where: str, graph: bool = False) -> int:
    if status < 0 or (status > 0 and not graph):
        msg = lib().rmlk_last_error()
        cls = GraphBuildError if graph else InferenceError
        raise cls(status, msg.decode() if msg else "unknown error", where)
    return status


def _dims(shape):
    shape = [int(d) for d in shape]
    return (ctypes.c_int64 * max(len(shape), 1))(*shape), len(shape)


def onnx_dtype(dt) -> int:
    if isinstance(dt, int):
        return dt
    return NP_TO_ONNX[np.dtype(dt)]


@dataclass
class NodeDesc:
    op: str
    inputs: List[str]
    outputs: List[str]
    attrs: Dict[str, object] = field(default_factory=dict)


@dataclass
class Graph:
    """A built graph: the native handle plus a description a CPU checker can walk."""
    handle: ctypes.c_void_p
    nodes: List[NodeDesc]
    inputs: Dict[str, tuple]            # name -> (onnx dtype, dims)
    initializers: Dict[str, np.ndarray]
    outputs: List[str]

    def __del__(self):
        try:
            if self.handle:
                lib().rmlk_graph_destroy(self.handle)
        except Exception:
            pass


class OpBuilder:
    """Returned by GraphBuilder.op so attributes can be chained (ref: builder.rs:216-232)."""

    def __init__(self, gb: "GraphBuilder", index: int, desc: NodeDesc):
        self._gb, self._index, self._desc = gb, index, desc

    def attr(self, name: str, value) -> "OpBuilder":
        g, i, key = self._gb._handle, self._index, name.encode()
        if isinstance(value, (bool, int, np.integer)):
            _check(lib().rmlk_graph_attr_int(g, i, key, int(value)), "attr", True)
        elif isinstance(value, float):
            _check(lib().rmlk_graph_attr_float(g, i, key, value), "attr", True)
        elif isinstance(value, str):
            _check(lib().rmlk_graph_attr_string(g, i, key, value.encode()), "attr", True)
        elif isinstance(value, np.ndarray):
            arr = np.asarray(value, order="C")
            d, r = _dims(arr.shape)
            _check(lib().rmlk_graph_attr_tensor(g, i, key, onnx_dtype(arr.dtype), d, r,
                                                arr.ctypes.data_as(ctypes.c_void_p)), "attr", True)
        elif isinstance(value, (list, tuple)) and any(isinstance(v, float) for v in value):
            vals = [float(v) for v in value]
            arr = (ctypes.c_float * max(len(vals), 1))(*vals)
            _check(lib().rmlk_graph_attr_floats(g, i, key, arr, len(vals)), "attr", True)
        elif isinstance(value, (list, tuple)):
            vals = [int(v) for v in value]
            arr = (ctypes.c_int64 * max(len(vals), 1))(*vals)
            _check(lib().rmlk_graph_attr_ints(g, i, key, arr, len(vals)), "attr", True)
        else:
            raise TypeError(f"unsupported attribute type for {name}: {type(value)}")
        self._desc.attrs[name] = value
        return self


class GraphBuilder:
    """Name-based builder. Values (inputs, constants) must exist before an op reads them; op
    outputs are declared by the op (ref: schema/src/builder.rs:44-260)."""

    def __init__(self):
        h = ctypes.c_void_p()
        _check(lib().rmlk_graph_create(ctypes.byref(h)), "rmlk_graph_create", True)
        self._handle = h
        self._nodes: List[NodeDesc] = []
        self._inputs: Dict[str, tuple] = {}
        self._inits: Dict[str, np.ndarray] = {}
        self._outputs: List[str] = []
        self._built = False

    def input(self, name: str, dtype, dims: Sequence[int]) -> "GraphBuilder":
        d, r = _dims(dims)
        _check(lib().rmlk_graph_input(self._handle, name.encode(), onnx_dtype(dtype), d, r),
               "GraphBuilder.input", True)
        self._inputs[name] = (onnx_dtype(dtype), [int(x) for x in dims])
        return self

    def constant(self, name: str, tensor) -> "GraphBuilder":
        arr = np.asarray(tensor, order="C")
        d, r = _dims(arr.shape)
        _check(lib().rmlk_graph_constant(self._handle, name.encode(), onnx_dtype(arr.dtype), d, r,
                                         arr.ctypes.data_as(ctypes.c_void_p)),
               "GraphBuilder.constant", True)
        self._inits[name] = arr
        return self

    def value(self, name: str, dtype=None, dims=None) -> "GraphBuilder":
        """Kept for parity with the reference builder; op outputs need no declaration here."""
        return self

    def op(self, op: str, inputs: Sequence[Optional[str]], outputs: Sequence[str]) -> OpBuilder:
        ins = [(i or "") for i in inputs]
        in_arr = (ctypes.c_char_p * max(len(ins), 1))(*[s.encode() for s in ins])
        out_arr = (ctypes.c_char_p * max(len(outputs), 1))(*[s.encode() for s in outputs])
        idx = _check(lib().rmlk_graph_op(self._handle, op.encode(), in_arr, len(ins), out_arr,
                                         len(outputs)), "GraphBuilder.op", True)
        desc = NodeDesc(op, list(ins), list(outputs))
        self._nodes.append(desc)
        return OpBuilder(self, idx, desc)

    def output(self, name: str) -> "GraphBuilder":
        _check(lib().rmlk_graph_output(self._handle, name.encode()), "GraphBuilder.output", True)
        self._outputs.append(name)
        return self

    def build(self) -> Graph:
        if not self._outputs:
            raise GraphBuildError(-20, "graph has no outputs", "GraphBuilder.build")
        self._built = True
        g = Graph(self._handle, self._nodes, self._inputs, self._inits, self._outputs)
        self._handle = None
        return g

    def __del__(self):
        try:
            if self._handle and not self._built:
                lib().rmlk_graph_destroy(self._handle)
        except Exception:
            pass


class ModelInstance:
    """ref: runtime/src/core/instance.rs:20-119"""

    def __init__(self, graph: Graph, device: int = 0, fuse: bool = True, weights: str = "auto",
                 bf16_pieces: bool = False):
        self.graph = graph
        h = ctypes.c_void_p()
        flags = (0 if fuse else 1) | {"auto": 0, "f16": 2, "bf16": 4, "f32": 8}[weights] | (16 if bf16_pieces else 0)
        _check(lib().rmlk_session_create_ex(graph.handle, device, flags, ctypes.byref(h)),
               "Builder.build")
        self._h = h

    @property
    def weights_16bit(self) -> int:
        """Constant weight matrices the session holds as 16-bit values."""
        return int(lib().rmlk_session_weights_16bit(self._h))

    @property
    def products_bf16_pieces(self) -> int:
        """Products of the last run that went to the bf16 matrix cores (bf16_pieces=True)."""
        return int(lib().rmlk_session_products_bf16_pieces(self._h))

    @property
    def fused_nodes(self) -> int:
        """Fused nodes formed while building (0 with fuse=False)."""
        return int(lib().rmlk_session_fused_nodes(self._h))

    # -- inputs -------------------------------------------------------------------------------
    def set_input(self, name: str, array) -> None:
        arr = np.asarray(array, order="C")
        d, r = _dims(arr.shape)
        _check(lib().rmlk_session_set_input(self._h, name.encode(), onnx_dtype(arr.dtype), d, r,
                                            arr.ctypes.data_as(ctypes.c_void_p)),
               f"set_input({name})")

    def bind_input(self, name: str, dtype, dims, device_ptr: int, donate: bool = False) -> None:
        d, r = _dims(dims)
        _check(lib().rmlk_session_bind_input(self._h, name.encode(), onnx_dtype(dtype), d, r,
                                             ctypes.c_void_p(device_ptr), int(donate)),
               f"bind_input({name})")

    def feed_output(self, out_name: str, in_name: str) -> None:
        _check(lib().rmlk_session_feed_output(self._h, out_name.encode(), in_name.encode()),
               f"feed_output({out_name}->{in_name})")

    # -- execution ------------------------------------------------------------------------------
    def execute(self) -> None:
        _check(lib().rmlk_session_run(self._h), "ModelInstance.run")

    def capture(self) -> None:
        _check(lib().rmlk_session_capture(self._h), "ModelInstance.capture")

    def replay(self) -> None:
        _check(lib().rmlk_session_replay(self._h), "ModelInstance.replay")

    def replay_enqueue(self) -> None:
        """Launch the recorded graph without waiting for it (several may be enqueued back to back)."""
        _check(lib().rmlk_session_replay_enqueue(self._h), "ModelInstance.replay_enqueue")

    def check(self) -> None:
        """Wait for the session's stream; raises if a kernel of any run or replay since the last
        report failed (an index out of range)."""
        _check(lib().rmlk_session_check(self._h), "ModelInstance.check")

    def sync(self) -> None:
        _check(lib().rmlk_session_sync(self._h), "ModelInstance.sync")

    @property
    def stream(self) -> int:
        return lib().rmlk_session_stream(self._h) or 0

    def output_info(self, name: str):
        dt = ctypes.c_int32()
        rank = ctypes.c_int32()
        dims = (ctypes.c_int64 * 8)()
        ptr = ctypes.c_void_p()
        _check(lib().rmlk_session_output_info(self._h, name.encode(), ctypes.byref(dt), dims,
                                              ctypes.byref(rank), ctypes.byref(ptr)),
               f"output_info({name})")
        return dt.value, [dims[i] for i in range(rank.value)], ptr.value or 0

    def output(self, name: str) -> np.ndarray:
        dt, shape, _ = self.output_info(name)
        out = np.empty(shape, dtype=ONNX_DTYPES[dt])
        _check(lib().rmlk_session_read_output(self._h, name.encode(),
                                              out.ctypes.data_as(ctypes.c_void_p), out.nbytes),
               f"read_output({name})")
        return out

    def run(self, inputs: Dict[str, np.ndarray]) -> Dict[str, np.ndarray]:
        """Feed, execute all nodes in stored order, read every graph output back.
        ref: ModelInstance::run, instance.rs:89-119"""
        for name, arr in inputs.items():
            self.set_input(name, arr)
        self.execute()
        return {name: self.output(name) for name in self.graph.outputs}

    # -- introspection --------------------------------------------------------------------------
    def set_profiling(self, enabled: bool) -> None:
        _check(lib().rmlk_session_set_profiling(self._h, int(enabled)), "set_profiling")

    def node_stats(self):
        n = lib().rmlk_session_node_count(self._h)
        out = []
        for i in range(n):
            op = ctypes.c_char_p()
            us, by, fl = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
            _check(lib().rmlk_session_node_info(self._h, i, ctypes.byref(op), ctypes.byref(us),
                                                ctypes.byref(by), ctypes.byref(fl)), "node_info")
            out.append({"node": i, "op": op.value.decode(), "micros": us.value,
                        "bytes": by.value, "flops": fl.value})
        return out

    def memory_stats(self):
        a, b, c = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        _check(lib().rmlk_session_memory_stats(self._h, ctypes.byref(a), ctypes.byref(b),
                                               ctypes.byref(c)), "memory_stats")
        return {"pool_bytes": a.value, "hip_mallocs": b.value, "device_syncs": c.value}

    def close(self) -> None:
        if self._h:
            lib().rmlk_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Builder:
    """ref: runtime/src/core/instance.rs:131-222"""

    def __init__(self, graph: Graph):
        self._graph = graph

    @staticmethod
    def from_graph(graph: Graph) -> "Builder":
        return Builder(graph)

    @staticmethod
    def from_onnx_path(path) -> "Builder":
        """ref: Builder::from_onnx_path (runtime/src/core/instance.rs:187-196); external tensor
        data is looked up next to the file."""
        from .onnx_io import load_onnx
        return Builder(load_onnx(path))

    @staticmethod
    def from_onnx_bytes(data: bytes, base_dir=None) -> "Builder":
        """ref: graph_from_onnx_bytes (schema/src/onnx_import/transform.rs:249-258)."""
        from .onnx_io import load_onnx_bytes
        return Builder(load_onnx_bytes(data, base_dir))

    def build(self, device: int = 0, fuse: bool = True, weights: str = "auto",
              bf16_pieces: bool = False) -> ModelInstance:
        """fuse=False keeps one kernel per node, as the reference executes a graph. weights: how the
        constant weights of fused MatMuls are stored (the arithmetic is fp32 in every case): "auto"
        as floats, or as 16-bit values where every float of a matrix is a bfloat16 / half value
        already (nothing is lost); "f32" as floats regardless; "f16" / "bf16" rounded to that type
        (half the bytes to stream per token). bf16_pieces: products of 64 and more rows over
        weights held as bfloat16 values split their fp32 operand into three bfloat16 pieces (exactly)
        and run on the bf16 matrix cores - fp32 results, sums in another order, about 2.5x the rate."""
        return ModelInstance(self._graph, device, fuse, weights, bf16_pieces)
