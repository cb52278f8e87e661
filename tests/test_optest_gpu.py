"""Operator-level parity through the production dispatch (GraphBuilder -> Builder -> run), the
counterpart of the reference's provider tests (runtime/src/providers/cuda/backend/*.rs, via
runtime/src/testing.rs). Every known-answer vector extracted from those tests is replayed, then
each result is compared with the CPU oracle on the same inputs."""
import json
import os

import numpy as np
import pytest

from helpers import assert_close, assert_exact
from optest import OpTest, decode

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_cases.json")))["provider_cases"]


def build(case):
    t = OpTest(case["op"])
    for f in case["feeds"]:
        arr = decode(f["data"], f["dtype"]).reshape(f["dims"])
        (t.input if f["kind"] == "input" else t.constant)(f["dims"], arr, arr.dtype)
    for k, v in case["attrs"].items():
        if isinstance(v, dict) and "tensor" in v:
            tt = v["tensor"]
            v = decode(tt["data"], tt["dtype"] or "float32").reshape(tt["dims"])
        elif isinstance(v, dict) and "floats" in v:
            v = [float(x) for x in v["floats"]]
        t.attr(k, v)
    return t


# Element types the reference lists in a dispatch arm that this build rejects, or the reverse.
KNOWN_DTYPE_DIFFERENCES = {
    # the reference dispatches Float16 arithmetic but cannot run it (providers/cuda/data.rs:109-126)
}


@pytest.mark.parametrize("case", CASES, ids=[f"{c['op']}-{c['test']}" for c in CASES])
def test_reference_provider_case(device, case):
    t = build(case)
    if case.get("expect_error"):
        err = t.run_err()
        for frag in case.get("error_contains", []):
            assert frag in str(err).lower(), (frag, str(err))
        return
    if any(f["dtype"] == "float16" for f in case["feeds"]) and case["op"] not in (
            "Cast", "Transpose", "Gather", "Concat", "Expand", "Slice", "Reshape", "Unsqueeze",
            "Shape", "Trilu", "ScatterND"):
        assert "unsupported data type" in str(t.run_err())
        return
    got = t.run()
    exp = decode(case["expected"], got.dtype)
    assert got.size == exp.size, (got.shape, exp.size)
    if case["output_dims"] is not None:
        assert list(got.shape) == case["output_dims"], (got.shape, case["output_dims"])
    tol = case["tolerance"]
    if got.dtype.kind == "f":
        # reference bar: exact vectors where it asserts equality on results that are exact in
        # fp32 (sums/products of small integers), approx otherwise
        np.testing.assert_allclose(got.reshape(-1), exp, rtol=1e-5, atol=max(tol, 1e-6),
                                   equal_nan=True)
    else:
        assert np.array_equal(got.reshape(-1), exp)
    # and the oracle on the same one-op graph
    ora = np.asarray(t.run_oracle())
    assert ora.shape == got.shape
    if got.dtype.kind == "f":
        assert_close(got, ora.astype(got.dtype))
    else:
        assert_exact(got, ora.astype(got.dtype))


def test_two_stage_add_with_constant(device):
    """backend/add.rs:140-154 (a run whose input is the previous run's output)."""
    ab = OpTest("Add").input([2, 2], [1, 2, 3, 4], np.float32).input([2, 2], [1, 2, 3, 4], np.float32).run()
    out = OpTest("Add").input([2, 2], ab).constant([2, 2], [1, 2, 3, 4], np.float32).run()
    assert out.reshape(-1).tolist() == [3.0, 6.0, 9.0, 12.0]
    out = OpTest("Add").input([2, 2], ab).constant([1, 2], [3, 4], np.float32).run()
    assert out.reshape(-1).tolist() == [5.0, 8.0, 9.0, 12.0]  # backend/add.rs:157-171


@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div", "Equal", "Greater", "Where", "Sqrt",
                                "Sin", "Cos", "Sigmoid", "ReduceMean", "Softmax", "MatMul",
                                "Transpose", "Gather", "Concat", "Trilu", "Reshape"])
def test_rejects_bool_data(device, op):
    """Every arithmetic / movement backend of the reference rejects bool payloads with a message
    that contains "unsupported" (e.g. backend/gather.rs:455-465)."""
    x = np.array([True, False, True, True])
    t = OpTest(op)
    if op == "Where":
        t.input([4], x).input([4], x).input([4], x)
    elif op in ("Add", "Sub", "Mul", "Div", "Equal", "Greater", "MatMul"):
        t.input([2, 2], x).input([2, 2], x)
    elif op == "Gather":
        t.input([4], x).input([1], [0], np.int64)
    elif op == "Concat":
        t.input([4], x).input([4], x).attr("axis", 0)
    elif op == "Reshape":
        t.input([4], x).input([2], [2, 2], np.int64)
    elif op == "Trilu":
        t.input([2, 2], x)
    else:
        t.input([2, 2], x)
    assert "unsupported" in str(t.run_err()).lower()


def test_unsupported_cast_message(device):
    err = OpTest("Cast").input([2], [True, False]).attr("to", 7).run_err()
    assert "unsupported cast" in str(err)  # runtime/src/core/error.rs:10


def test_shape_errors(device):
    e = OpTest("Add").input([2, 3], np.zeros(6, np.float32)).input([4, 3], np.zeros(12, np.float32)).run_err()
    assert "broadcast" in str(e)
    e = OpTest("MatMul").input([2, 3], np.zeros(6, np.float32)).input([4, 3], np.zeros(12, np.float32)).run_err()
    assert "IncompatibleDimForMul" in str(e)
    e = OpTest("Gather").input([3], np.zeros(3, np.float32)).input([1], [3], np.int64).run_err()
    assert "kernel failed" in str(e)  # index == dim is rejected (the reference accepts it)
    e = OpTest("ScatterND").input([4], np.zeros(4, np.float32)).input([1, 1], [7], np.int64) \
        .input([1], [1.0], np.float32).run_err()
    assert "kernel failed" in str(e)  # ref: KernelFailed{code}, backend/scatter_nd.rs:198-203
    e = OpTest("Slice").input([4], np.zeros(4, np.float32)).input([1], [0], np.int64) \
        .input([1], [4], np.int64).input([1], [0], np.int64).input([1], [0], np.int64).run_err()
    assert "ZeroStep" in str(e)


def test_reshape_unsqueeze_views(device):
    """backend/reshape.rs:194-252, backend/unsqueeze.rs:165-247 with recognisable data."""
    data = np.arange(24, dtype=np.float32)
    out = OpTest("Reshape").input([2, 3, 4], data).input([2], [4, 6], np.int64).run()
    assert out.shape == (4, 6) and np.array_equal(out.reshape(-1), data)
    out = OpTest("Reshape").input([2, 3, 4], data).input([2], [-1, 8], np.int64).run()
    assert out.shape == (3, 8)
    out = OpTest("Reshape").input([2, 3, 4], data).input([3], [0, 0, 4], np.int64).run()
    assert out.shape == (2, 3, 4)
    out = OpTest("Reshape").input([1], [11.1], np.float32).input([0], [], np.int64).run()
    assert out.shape == () and out == np.float32(11.1)
    for axes, shape in (([0], (1, 2, 3, 4)), ([1], (2, 1, 3, 4)), ([3], (2, 3, 4, 1)),
                        ([0, 4], (1, 2, 3, 4, 1)), ([4, 0], (1, 2, 3, 4, 1)), ([-1], (2, 3, 4, 1))):
        out = OpTest("Unsqueeze").input([2, 3, 4], data).input([len(axes)], axes, np.int64).run()
        assert out.shape == shape and np.array_equal(out.reshape(-1), data)


def test_transpose_default_and_large_slice(device):
    """backend/transpose.rs:216-238 (default perm reverses), backend/slice.rs:766-788 (cuda_large)."""
    data = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    out = OpTest("Transpose").input([2, 3, 4], data).run()
    assert out.shape == (4, 3, 2) and np.array_equal(out, data.transpose(2, 1, 0))
    big = np.arange(1 * 24 * 27 * 128, dtype=np.float32).reshape(1, 24, 27, 128)
    out = OpTest("Slice").input(big.shape, big).input([1], [0], np.int64).input([1], [13], np.int64) \
        .input([1], [2], np.int64).run()
    assert np.array_equal(out, big[:, :, :13, :])
    out = OpTest("Slice").input([4], np.arange(4, dtype=np.float32)).input([1], [2], np.int64) \
        .input([1], [2], np.int64).run()
    assert out.shape == (0,)  # backend/slice.rs:749-764 (cuda_empty_output)


def test_sin_cos_vectors(device):
    """backend/sin.rs:82-95, backend/cos.rs:79-92: sin/cos of a handful of angles."""
    x = np.array([0.0, np.pi / 6, np.pi / 2, np.pi, 3 * np.pi / 4, -np.pi / 2], dtype=np.float32)
    assert_close(OpTest("Sin").input([6], x).run(), np.sin(x.astype(np.float64)).astype(np.float32))
    assert_close(OpTest("Cos").input([6], x).run(), np.cos(x.astype(np.float64)).astype(np.float32))


def test_softmax_large_row(device):
    """backend/softmax.rs:299-313: a 4096-wide row."""
    x = (np.arange(4096, dtype=np.float32) % 2)[None]
    got = OpTest("Softmax").input([1, 4096], x).run()
    e = np.exp(1.0)
    exp = np.where(x == 1, e, 1.0) / (2048 * (1 + e))
    assert_close(got, exp.astype(np.float32))


def test_matmul_batched_vs_loop(device):
    """backend/matmul.rs:563-590 (batched against a reference loop)."""
    rng = np.random.default_rng(0)
    a = rng.standard_normal((1, 5, 7)).astype(np.float32)
    b = rng.standard_normal((7, 3)).astype(np.float32)
    got = OpTest("MatMul").input(a.shape, a).input(b.shape, b).run()
    assert_close(got, np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32))
    got = OpTest("MatMul").input([7], a[0, 0]).input([7], b[:, 0].copy()).run()
    assert got.shape == ()  # d1 x d1 -> scalar


def test_reduce_mean_axes_forms(device):
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    out = OpTest("ReduceMean").input(x.shape, x).attr("axes", [1]).attr("keepdims", 0).run()
    assert_close(out, x.mean(axis=1))
    out = OpTest("ReduceMean").input(x.shape, x).input([2], [0, -1], np.int64).run()
    assert_close(out, x.mean(axis=(0, 2), keepdims=True))
    out = OpTest("ReduceMean").input(x.shape, x).run()
    assert_close(out, x.mean(keepdims=True).astype(np.float32))
    out = OpTest("ReduceMean").input(x.shape, x).input([0], [], np.int64) \
        .attr("noop_with_empty_axes", 1).run()
    assert_exact(out, x)


def test_trilu_k_input_and_concat_empty(device):
    x = np.arange(1, 13, dtype=np.float32).reshape(3, 4)
    out = OpTest("Trilu").input(x.shape, x).input([], [1], np.int64).run()
    assert_exact(out, np.triu(x, 1))
    out = OpTest("Trilu").input(x.shape, x).input([], [-1], np.int64).attr("upper", 0).run()
    assert_exact(out, np.tril(x, -1))
    past = np.zeros((1, 8, 0, 64), np.float32)   # zero-length KV on the first step
    new = np.arange(8 * 3 * 64, dtype=np.float32).reshape(1, 8, 3, 64)
    out = OpTest("Concat").input(past.shape, past).input(new.shape, new).attr("axis", 2).run()
    assert_exact(out, new)


def test_session_memory_steady_state(device):
    """After the first run with given shapes the buffer pool serves every tensor: no hipMalloc."""
    from rmlk_amd.runtime import Builder
    t = OpTest("Softmax").input([4, 256], np.zeros((4, 256), np.float32))
    graph, inputs = t.build()
    inst = Builder.from_graph(graph).build()
    inst.run(inputs)
    m0 = inst.memory_stats()
    for _ in range(3):
        inst.run(inputs)
    m1 = inst.memory_stats()
    assert m1["hip_mallocs"] == m0["hip_mallocs"] and m1["pool_bytes"] == m0["pool_bytes"]
    inst.close()


def test_small_float16_initializer_builds_and_casts(device):
    """A float16 constant of a few elements needs no host mirror (nothing reads half floats on the
    host): the session must build, and Cast must read the constant on the device."""
    from rmlk_amd.runtime import Builder, GraphBuilder
    half = np.array([0.5, -2.0, 1024.0], dtype=np.float16)
    gb = GraphBuilder()
    gb.input("x", np.float32, [3])
    gb.constant("h", half)
    gb.op("Cast", ["h"], ["hf"]).attr("to", 1)
    gb.op("Add", ["x", "hf"], ["y"])
    gb.output("y")
    inst = Builder.from_graph(gb.build()).build()
    x = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    got = inst.run({"x": x})["y"]
    assert_exact(got, x + half.astype(np.float32))
    inst.close()


def test_set_input_keeps_a_view_output_of_the_previous_run(device):
    """A graph output that is a view of an input (Reshape shares the buffer) must keep the bytes of
    the run that produced it when the next input is set, with and without a recorded graph."""
    from rmlk_amd.runtime import Builder, GraphBuilder
    gb = GraphBuilder()
    gb.input("x", np.float32, [2, 3])
    gb.constant("shape", np.array([3, 2], dtype=np.int64))
    gb.op("Reshape", ["x", "shape"], ["v"])
    gb.op("Neg", ["x"], ["n"])
    gb.output("v").output("n")
    inst = Builder.from_graph(gb.build()).build()
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    b = a + 100
    inst.set_input("x", a)
    inst.execute()
    inst.set_input("x", b)                      # no run yet: the outputs are still those of `a`
    assert_exact(inst.output("v"), a.reshape(3, 2))
    assert_exact(inst.output("n"), -a)
    inst.execute()
    assert_exact(inst.output("v"), b.reshape(3, 2))
    # with a recorded graph the input is refreshed in place and the replay gives the new results
    inst.capture()
    for arr in (a, b, a):
        inst.set_input("x", arr)
        inst.replay()
        assert_exact(inst.output("v"), arr.reshape(3, 2))
        assert_exact(inst.output("n"), -arr)
    inst.close()
