"""ONNX wire format, CPU only: the native reader (librmlk_hip.so), the independent pure-Python
reader of the oracle package and the writer of rmlk_amd.onnx_io against each other and against
files PyTorch's own exporter serialised (tests/golden/torch_*.onnx, made by
tests/golden/export_torch_onnx.py; expected outputs computed by PyTorch)."""
import os
import struct

import numpy as np
import pytest

from rmlk_amd import graphs, onnx_io
from rmlk_amd.runtime import GraphBuildError, GraphBuilder
from oracle import graph as og
from oracle import onnx_read

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TORCH_FILES = ["torch_norm_proj_softmax", "torch_decoder_block"]


def fnv1a(data: bytes) -> str:
    h = 1469598103934665603
    for b in data:
        h = ((h ^ b) * 1099511628211) & ((1 << 64) - 1)
    return format(h, "x")


def norm_attr(v):
    if isinstance(v, np.ndarray):
        return {"dtype": onnx_io.onnx_dtype(v.dtype), "dims": list(v.shape),
                "fnv1a": fnv1a(np.ascontiguousarray(v).tobytes())}
    if isinstance(v, float):
        return float(np.float32(v))
    if isinstance(v, (list, tuple)):
        return [norm_attr(x) for x in v]
    return v


def assert_same_graph(native: dict, py):
    """native: rmlk_graph_describe JSON; py: a description with nodes / inputs / initializers."""
    assert [n["op"] for n in native["nodes"]] == [n.op for n in py.nodes]
    for a, b in zip(native["nodes"], py.nodes):
        ins = list(b.inputs)
        while ins and not ins[-1]:
            ins.pop()
        assert a["inputs"] == ins and a["outputs"] == list(b.outputs)
        want = {k: norm_attr(v) for k, v in b.attrs.items()}
        got = {k: (float(np.float32(v)) if isinstance(v, float) else v) for k, v in a["attrs"].items()}
        assert got == want, (a["op"], got, want)
    assert {i["name"]: (i["dtype"], i["dims"]) for i in native["inputs"]} == \
        {k: (v[0], list(v[1])) for k, v in py.inputs.items()}
    assert native["outputs"] == list(py.outputs)
    inits = {i["name"]: i for i in native["initializers"]}
    assert set(inits) == set(py.initializers)
    for name, arr in py.initializers.items():
        arr = np.asarray(arr)
        assert inits[name]["dims"] == list(arr.shape)
        assert inits[name]["dtype"] == onnx_io.onnx_dtype(arr.dtype)
        assert inits[name]["fnv1a"] == fnv1a(np.ascontiguousarray(arr).tobytes()), name


@pytest.mark.parametrize("name", TORCH_FILES)
def test_native_and_python_readers_agree_on_pytorch_exports(name):
    path = os.path.join(GOLDEN, name + ".onnx")
    g = onnx_io.load_onnx(path)
    assert_same_graph(onnx_io.describe(g.handle), onnx_read.read_onnx(path))


@pytest.mark.parametrize("name", TORCH_FILES)
def test_oracle_reproduces_pytorch_on_its_exports(name):
    """Whole-graph pin of the oracle: the graph PyTorch exported, walked by the numpy oracle,
    gives PyTorch's own fp32 result."""
    lg = onnx_read.read_onnx(os.path.join(GOLDEN, name + ".onnx"))
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    out = og.run_graph(lg, {k: z[k] for k in lg.inputs})
    np.testing.assert_allclose(out["y"], z["y"], rtol=1e-5, atol=2e-6)


def test_dynamic_dim_of_a_pytorch_export_reads_as_zero():
    g = onnx_io.load_onnx(os.path.join(GOLDEN, "torch_norm_proj_softmax.onnx"))
    assert g.inputs == {"x": (1, [2, 0, 64])}


def small_graphs():
    cfg = graphs.LlamaConfig.tiny()
    yield "config1", graphs.rmsnorm_matmul_graph(seed=1, seq=4, hidden=64, n_out=32)[0]
    yield "llama_concat", graphs.llama_graph(cfg, seed=4, style="concat")
    yield "llama_scatter", graphs.llama_graph(cfg, seed=4, style="scatter", max_len=16)
    yield "kv_stress", graphs.kv_stress_graph(seed=5, heads=2, length=16, head_dim=8, vocab=50,
                                              hidden=16, n_gather=7, mask_n=12)[0]


@pytest.mark.parametrize("name,graph", list(small_graphs()))
def test_written_graphs_read_back_identically(name, graph):
    data = onnx_io.graph_to_onnx_bytes(graph)
    loaded = onnx_io.load_onnx_bytes(data)
    assert_same_graph(onnx_io.describe(loaded.handle), graph)
    again = onnx_read.read_onnx(data)
    assert [n.op for n in again.nodes] == [n.op for n in graph.nodes]
    for k, v in graph.initializers.items():
        assert np.array_equal(again.initializers[k], v) and again.initializers[k].dtype == v.dtype


def test_external_data_round_trip(tmp_path):
    graph = graphs.llama_graph(graphs.LlamaConfig.tiny(), seed=4, style="concat")
    path = str(tmp_path / "model.onnx")
    onnx_io.save_onnx(graph, path, external_data=True, external_threshold=256)
    assert os.path.getsize(path + ".data") > 10000
    assert os.path.getsize(path) < os.path.getsize(path + ".data")
    loaded = onnx_io.load_onnx(path)
    assert_same_graph(onnx_io.describe(loaded.handle), graph)
    again = onnx_read.read_onnx(path)
    for k, v in graph.initializers.items():
        assert np.array_equal(again.initializers[k], v)


# ---- hand-encoded messages: the encodings a writer may choose -----------------------------------

def key(field, wire):
    return onnx_io._varint((field << 3) | wire)


def ld(field, payload):
    return key(field, 2) + onnx_io._varint(len(payload)) + payload


def model_of(graph_bytes):
    return onnx_io._f_varint(1, 8) + ld(7, graph_bytes)


def tensor_msg(name, dims, dtype, body, packed_dims=False):
    if packed_dims:
        t = ld(1, b"".join(onnx_io._varint(d) for d in dims))
    else:
        t = b"".join(onnx_io._f_varint(1, d) for d in dims)
    return t + onnx_io._f_varint(2, dtype) + onnx_io._f_string(8, name) + body


def identity_graph(init_msg, extra=b""):
    node = onnx_io._f_string(1, "c") + onnx_io._f_string(2, "y") + onnx_io._f_string(4, "Neg")
    return model_of(ld(1, node) + ld(5, init_msg) + ld(12, onnx_io._f_string(1, "y")) + extra)


@pytest.mark.parametrize("case", ["float_packed", "float_unpacked", "int64_packed", "int64_unpacked",
                                  "int32_negative", "bool_in_int32", "double_packed", "uint64",
                                  "float16_bits", "raw_with_packed_dims", "scalar"])
def test_typed_tensor_fields(case):
    if case == "float_packed":
        want = np.array([1.5, -2.0, 3.25], np.float32)
        msg = tensor_msg("c", [3], 1, ld(4, want.tobytes()))
    elif case == "float_unpacked":
        want = np.array([1.5, -2.0], np.float32)
        msg = tensor_msg("c", [2], 1, b"".join(key(4, 5) + struct.pack("<f", v) for v in want))
    elif case == "int64_packed":
        want = np.array([[7, -1], [2 ** 40, 0]], np.int64)
        msg = tensor_msg("c", [2, 2], 7, ld(7, b"".join(onnx_io._varint(int(v)) for v in want.ravel())))
    elif case == "int64_unpacked":
        want = np.array([-9, 5], np.int64)
        msg = tensor_msg("c", [2], 7, b"".join(onnx_io._f_varint(7, int(v)) for v in want))
    elif case == "int32_negative":
        want = np.array([-3, 4, -2 ** 31], np.int32)
        msg = tensor_msg("c", [3], 6, ld(5, b"".join(onnx_io._varint(int(v)) for v in want)))
    elif case == "bool_in_int32":
        want = np.array([True, False, True], np.bool_)
        msg = tensor_msg("c", [3], 9, ld(5, bytes([1, 0, 1])))
    elif case == "double_packed":
        want = np.array([0.1, -1e300], np.float64)
        msg = tensor_msg("c", [2], 11, ld(10, want.tobytes()))
    elif case == "uint64":
        want = np.array([2 ** 63 + 5, 1], np.uint64)
        msg = tensor_msg("c", [2], 13, ld(11, b"".join(onnx_io._varint(int(v)) for v in want)))
    elif case == "float16_bits":
        want = np.array([1.0, -0.5], np.float16)
        msg = tensor_msg("c", [2], 10, ld(5, b"".join(onnx_io._varint(int(v)) for v in want.view(np.uint16))))
    elif case == "raw_with_packed_dims":
        want = np.arange(6, dtype=np.float32).reshape(2, 3)
        msg = tensor_msg("c", [2, 3], 1, ld(9, want.tobytes()), packed_dims=True)
    else:
        want = np.array(4.5, np.float32)
        msg = tensor_msg("c", [], 1, ld(9, want.tobytes()))
    data = identity_graph(msg)
    g = onnx_io.load_onnx_bytes(data)          # keeps the native graph alive
    native = onnx_io.describe(g.handle)
    (init,) = native["initializers"]
    assert init["dims"] == list(want.shape) and init["dtype"] == onnx_io.onnx_dtype(want.dtype)
    assert init["fnv1a"] == fnv1a(want.tobytes())
    py = onnx_read.read_onnx(data).initializers["c"]
    assert py.dtype == want.dtype and np.array_equal(py, want)


def test_input_that_shadows_an_initializer_keeps_the_constant():
    c = tensor_msg("c", [2], 1, ld(9, np.ones(2, np.float32).tobytes()))
    data = identity_graph(c, extra=ld(11, onnx_io._value_info("c", 1, [2])) +
                          ld(11, onnx_io._value_info("real", 7, [0, 3])))
    g = onnx_io.load_onnx_bytes(data)
    assert g.inputs == {"real": (7, [0, 3])}
    assert onnx_read.read_onnx(data).inputs == {"real": (7, [0, 3])}


def test_attribute_without_type_field_is_inferred_from_the_populated_field():
    attr = onnx_io._f_string(1, "axis") + onnx_io._f_varint(3, -1)          # no field 20
    node = onnx_io._f_string(1, "x") + onnx_io._f_string(2, "y") + onnx_io._f_string(4, "Softmax") + ld(5, attr)
    data = model_of(ld(1, node) + ld(11, onnx_io._value_info("x", 1, [2, 3])) +
                    ld(12, onnx_io._f_string(1, "y")))
    g = onnx_io.load_onnx_bytes(data)
    d = onnx_io.describe(g.handle)
    assert d["nodes"][0]["attrs"] == {"axis": -1}
    assert onnx_read.read_onnx(data).nodes[0].attrs == {"axis": -1}


@pytest.mark.parametrize("data,text", [
    (b"", "does not have a graph"),
    (onnx_io._f_varint(1, 8), "does not have a graph"),
    (b"\x3a\x7f\x01", "failed to parse ONNX model"),                  # graph length past the end
    (b"\xff\xff\xff\xff\xff\xff\xff\xff\xff\xff\xff", "failed to parse ONNX model"),
])
def test_malformed_models_are_rejected(data, text):
    with pytest.raises(GraphBuildError, match=text):
        onnx_io.load_onnx_bytes(data)


def test_unsupported_content_is_rejected():
    sub = ld(6, b"")     # attribute with a subgraph
    attr = onnx_io._f_string(1, "body") + sub
    node = onnx_io._f_string(1, "x") + onnx_io._f_string(2, "y") + onnx_io._f_string(4, "Neg") + ld(5, attr)
    data = model_of(ld(1, node) + ld(11, onnx_io._value_info("x", 1, [2])) + ld(12, onnx_io._f_string(1, "y")))
    with pytest.raises(GraphBuildError, match="subgraphs are not supported"):
        onnx_io.load_onnx_bytes(data)
    s = tensor_msg("c", [1], 8, ld(6, b"abc"))        # string tensor
    with pytest.raises(GraphBuildError):
        onnx_io.load_onnx_bytes(identity_graph(s))
    short = tensor_msg("c", [3], 1, ld(9, b"\0" * 8))  # 8 bytes for 3 floats
    with pytest.raises(GraphBuildError, match="raw_data of 8 bytes for 12"):
        onnx_io.load_onnx_bytes(identity_graph(short))
    node = onnx_io._f_string(1, "x") + onnx_io._f_string(2, "y") + onnx_io._f_string(4, "Foo") + \
        onnx_io._f_string(7, "com.example")
    data = model_of(ld(1, node) + ld(11, onnx_io._value_info("x", 1, [2])) + ld(12, onnx_io._f_string(1, "y")))
    with pytest.raises(GraphBuildError, match="com.example::Foo"):
        onnx_io.load_onnx_bytes(data)


def test_missing_file():
    with pytest.raises(GraphBuildError, match="cannot open"):
        onnx_io.load_onnx("/nonexistent/model.onnx")


def test_builder_from_onnx_path_mirrors_the_reference_entry_point():
    from rmlk_amd.runtime import Builder
    b = Builder.from_onnx_path(os.path.join(GOLDEN, "torch_norm_proj_softmax.onnx"))
    assert isinstance(b, Builder)
    g = GraphBuilder()      # and the plain builder still works next to it
    g.input("a", np.float32, [1])
    g.op("Neg", ["a"], ["b"])
    g.output("b")
    assert len(g.build().nodes) == 1
