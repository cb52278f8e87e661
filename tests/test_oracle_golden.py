"""CPU: the oracle against every known-answer vector extracted from the reference's own tests
(tests/golden/reference_cases.json), the ONNX-Runtime-produced attention fixture the reference
holds, and the loop restatement of the reference kernels. Nothing here touches the GPU."""
import json
import os

import numpy as np
import pytest

from optest import decode
from oracle import graph as ograph
from oracle import loops, ops

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_cases.json")))
PROVIDER = [c for c in CASES["provider_cases"]]


class _Node:
    def __init__(self, op, inputs, outputs, attrs):
        self.op, self.inputs, self.outputs, self.attrs = op, inputs, outputs, attrs


class _Graph:
    def __init__(self, nodes, inits, outputs):
        self.nodes, self.initializers, self.outputs = nodes, inits, outputs


def case_attrs(case):
    attrs = {}
    for k, v in case["attrs"].items():
        if isinstance(v, dict) and "tensor" in v:
            t = v["tensor"]
            attrs[k] = decode(t["data"], t["dtype"] or "float32").reshape(t["dims"])
        elif isinstance(v, dict) and "floats" in v:
            attrs[k] = [float(x) for x in v["floats"]]
        else:
            attrs[k] = v
    return attrs


def one_op_graph(case):
    names, env = [], {}
    for i, f in enumerate(case["feeds"]):
        env[f"v{i}"] = decode(f["data"], f["dtype"]).reshape(f["dims"])
        names.append(f"v{i}")
    attrs = case_attrs(case)
    op = case["op"]
    return _Graph([_Node(op, names, ["y"], attrs)], {}, ["y"]), env


def expected_of(case, got):
    return decode(case["expected"], got.dtype)


@pytest.mark.parametrize("case", PROVIDER, ids=[f"{c['op']}-{c['test']}" for c in PROVIDER])
def test_oracle_matches_reference_provider_vectors(case):
    g, env = one_op_graph(case)
    if case.get("expect_error"):
        # dtype gates are properties of the operator dispatch, not of the arithmetic: only the
        # shape / argument errors concern the oracle
        if any("unsupported" in s for s in case.get("error_contains", [])):
            pytest.skip("element-type gate: checked against the runtime, not the oracle")
        with pytest.raises(Exception):
            ograph.run_graph(g, env)
        return
    got = np.asarray(ograph.run_graph(g, env)["y"])
    exp = expected_of(case, got)
    assert got.size == exp.size, (got.shape, exp.size)
    tol = case["tolerance"]
    if tol == 0.0 and got.dtype.kind != "f":
        assert np.array_equal(got.reshape(-1), exp)
    else:
        np.testing.assert_allclose(got.reshape(-1), exp, rtol=1e-6, atol=max(tol, 1e-6),
                                   equal_nan=True)


@pytest.mark.parametrize("rule", CASES["slice_shape_rules"], ids=lambda r: r["test"])
def test_slice_shape_rules(rule):
    """backend/slice.rs:497-677: output-shape rules of compute_output_shape_helper."""
    if not rule["expect_error"] and rule["expected_shape"] is None:
        ops.slice_resolve(rule["shape"], rule["starts"], rule["ends"], rule["axes"], rule["steps"])
        return  # the reference only requires that this does not fail
    if rule["expect_error"]:
        with pytest.raises(Exception):
            res = ops.slice_resolve(rule["shape"], rule["starts"], rule["ends"], rule["axes"],
                                    rule["steps"])
            if len(set(a % len(rule["shape"]) for a in rule["axes"])) != len(rule["axes"]):
                raise ops.OracleError("duplicate axes")
        return
    res = ops.slice_resolve(rule["shape"], rule["starts"], rule["ends"], rule["axes"], rule["steps"])
    assert [r[2] for r in res] == rule["expected_shape"]
    x = np.arange(int(np.prod(rule["shape"]))).reshape(rule["shape"])
    out_shape, flat = loops.slice_loop(rule["shape"], rule["starts"], rule["ends"], rule["axes"],
                                       rule["steps"], x.reshape(-1))
    assert out_shape == rule["expected_shape"]
    assert np.array_equal(np.array(flat, dtype=x.dtype).reshape(out_shape),
                          ops.slice_(x, rule["starts"], rule["ends"], rule["axes"], rule["steps"]))


@pytest.mark.parametrize("case", CASES["kernel_cases"]["reduce_mean"], ids=lambda c: c["test"])
def test_reduce_mean_kernel_vectors(case):
    """cuda/src/kernels/reduce_mean.rs:156-266"""
    x = decode(case["data"], np.float32).reshape(case["shape"])
    got = ops.reduce_mean(x, case["axes"], keepdims=1)
    assert list(got.shape) == case["out_shape"]
    np.testing.assert_allclose(got.reshape(-1), decode(case["expected"], np.float32), rtol=1e-6)
    lp = loops.reduce_mean_loop(case["shape"], case["axes"], x.reshape(-1))
    np.testing.assert_allclose(np.array(lp, dtype=np.float32), got.reshape(-1), rtol=1e-7)


def load_f32(name):
    return np.fromfile(os.path.join(HERE, "golden", name), dtype="<f4")


def attention_graph():
    """runtime/tests/graphs/attention.rs:15-41"""
    nodes = [
        _Node("Transpose", ["k"], ["kt"], {"perm": [0, 2, 1]}),
        _Node("MatMul", ["q", "kt"], ["scores"], {}),
        _Node("Div", ["scores", "scale"], ["scaled"], {}),
        _Node("Trilu", ["scaled"], ["masked"], {"upper": 0}),
        _Node("Softmax", ["masked"], ["probs"], {"axis": -1}),
        _Node("MatMul", ["probs", "v"], ["out"], {}),
    ]
    return _Graph(nodes, {"scale": np.array(2.0, dtype=np.float32)}, ["out"])


def test_attention_fixture_from_onnxruntime():
    """The one ONNX-Runtime-CPU-generated golden in the reference tree (tolerance 1e-5,
    runtime/tests/graphs/attention.rs:53-55). Pins Transpose + MatMul + Div(scalar) +
    Trilu(lower, zero fill) + Softmax + MatMul together."""
    q, k, v = (load_f32(f"attention_{n}.f32").reshape(1, 2, 4) for n in "qkv")
    exp = load_f32("attention_out.f32")
    assert exp.size == 8
    out = ograph.run_graph(attention_graph(), {"q": q, "k": k, "v": v})["out"]
    np.testing.assert_allclose(out.reshape(-1), exp, rtol=0, atol=1e-5)
    # the f32-accumulate variant used for CPU timing must agree as well
    out32 = ograph.run_graph(attention_graph(), {"q": q, "k": k, "v": v}, "f32")["out"]
    np.testing.assert_allclose(out32.reshape(-1), exp, rtol=0, atol=1e-5)


# ---- loop restatement vs numpy restatement ------------------------------------------------------
@pytest.mark.parametrize("sa,sb", [((2, 4, 1), (4, 3)), ((2, 4, 3), (3,)), ((3, 1, 2), (1, 5, 1)),
                                   ((1,), (2, 2)), ((2, 3), (2, 3))])
def test_binary_loop_vs_numpy(sa, sb):
    rng = np.random.default_rng(1)
    a = rng.integers(-9, 9, size=sa).astype(np.int64)
    b = rng.integers(1, 9, size=sb).astype(np.int64)
    out_shape = loops.compute_broadcast_output_shape(list(sa), list(sb))
    assert out_shape == list(np.broadcast_shapes(sa, sb))
    ast = loops.compute_broadcast_stride(list(sa), out_shape)
    bst = loops.compute_broadcast_stride(list(sb), out_shape)
    for fn, ref in [(lambda x, y: x + y, ops.add), (lambda x, y: x - y, ops.sub),
                    (lambda x, y: x * y, ops.mul), (lambda x, y: x > y, ops.greater),
                    (lambda x, y: x == y, ops.equal),
                    (lambda x, y: int(abs(x) // abs(y)) * (1 if (x >= 0) == (y >= 0) else -1), ops.div)]:
        got = loops.binary_loop(fn, out_shape, ast, bst, a.reshape(-1), b.reshape(-1))
        assert np.array_equal(np.array(got).reshape(out_shape), ref(a, b))
    assert loops.compute_broadcast_output_shape([2, 3], [4, 3]) is None


def test_where_loop_vs_numpy():
    rng = np.random.default_rng(2)
    c = rng.random((3, 1)) < 0.5
    x = rng.integers(0, 9, size=(1, 4))
    y = rng.integers(0, 9, size=(3, 4))
    shp = [3, 4]
    got = loops.ternary_loop(shp, loops.compute_broadcast_stride([1, 4], shp),
                             loops.compute_broadcast_stride([3, 4], shp),
                             loops.compute_broadcast_stride([3, 1], shp), x.reshape(-1),
                             y.reshape(-1), c.reshape(-1))
    assert np.array_equal(np.array(got).reshape(shp), ops.where(c, x, y))


def test_movement_loops_vs_numpy():
    x = np.arange(2 * 3 * 4 * 5).reshape(2, 3, 4, 5)
    for perm in ([0, 2, 1, 3], [3, 2, 1, 0], [1, 0, 3, 2], [0, 1, 3, 2]):
        got = loops.transpose_loop(list(x.shape), perm, x.reshape(-1))
        assert np.array_equal(np.array(got).reshape([x.shape[p] for p in perm]),
                              ops.transpose(x, perm))
    e = np.arange(6).reshape(1, 3, 1, 2)
    got = loops.expand_loop([1, 3, 1, 2], [4, 3, 5, 2], e.reshape(-1))
    assert np.array_equal(np.array(got).reshape(4, 3, 5, 2), ops.expand(e, [4, 3, 5, 2]))
    got = loops.gather_loop([2, 3, 4], 1, [2, -3, 1], x[:, :3, :4, 0].reshape(-1))
    assert np.array_equal(np.array(got).reshape(2, 3, 4),
                          ops.gather(x[:, :3, :4, 0], np.array([2, -3, 1]), 1))
    parts = [x[:, :, :1], x[:, :, 1:1], x[:, :, 1:]]
    got = loops.concat_loop([list(p.shape) for p in parts], 2, [p.reshape(-1) for p in parts])
    assert np.array_equal(np.array(got).reshape(x.shape), ops.concat(parts, 2))
    for upper in (0, 1):
        for k in (-2, 0, 1, 7):
            m = np.arange(1, 2 * 4 * 5 + 1).reshape(2, 4, 5)
            got = loops.trilu_loop(2, 4, 5, upper, k, m.reshape(-1))
            assert np.array_equal(np.array(got).reshape(2, 4, 5), ops.trilu(m, k, upper))


def test_scatter_loop_vs_numpy_and_onnx_examples():
    data = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.float32)
    idx = np.array([[4], [3], [1], [7]], dtype=np.int64)
    upd = np.array([9, 10, 11, 12], dtype=np.float32)
    exp = np.array([1, 11, 3, 10, 9, 6, 7, 12], dtype=np.float32)  # ONNX ScatterND example 1
    assert np.array_equal(ops.scatter_nd(data, idx, upd), exp)
    got, err = loops.scatter_nd_loop([8], [4, 1], idx.reshape(-1), upd, data)
    assert err == 0 and np.array_equal(np.array(got, dtype=np.float32), exp)
    _, err = loops.scatter_nd_loop([8], [1, 1], [8], [0.0], data)
    assert err == 1
    with pytest.raises(ops.OracleError):
        ops.scatter_nd(data, np.array([[8]]), np.array([0.0], dtype=np.float32))
    d3 = np.arange(4 * 4 * 4, dtype=np.float32).reshape(4, 4, 4)
    i3 = np.array([[0], [2]], dtype=np.int64)
    u3 = -np.ones((2, 4, 4), dtype=np.float32)
    for red in ("none", "add", "mul", "max", "min"):
        got, err = loops.scatter_nd_loop([4, 4, 4], [2, 1], i3.reshape(-1), u3.reshape(-1),
                                         d3.reshape(-1), red)
        assert err == 0
        assert np.array_equal(np.array(got, dtype=np.float32).reshape(4, 4, 4),
                              ops.scatter_nd(d3, i3, u3, red))


def test_matmul_and_softmax_closed_forms():
    rng = np.random.default_rng(3)
    a = rng.standard_normal((3, 5)).astype(np.float32)
    b = rng.standard_normal((5, 4)).astype(np.float32)
    np.testing.assert_allclose(ops.matmul(a, b), loops.matmul_loop(a.reshape(-1), b.reshape(-1), 3, 5, 4),
                               rtol=1e-6)
    # batched 4-D of constants: every element is k * 1 * 13 (backend/matmul.rs d4_shape_and_values)
    out = ops.matmul(np.ones((1, 24, 6, 6), np.float32), np.full((1, 24, 6, 128), 13.0, np.float32))
    assert out.shape == (1, 24, 6, 128) and np.all(out == 78.0)
    x = rng.standard_normal((4, 7)).astype(np.float32)
    np.testing.assert_allclose(ops.softmax(x).reshape(-1), loops.softmax_loop(4, 7, x.reshape(-1)),
                               rtol=1e-6)
    # uniform row -> 1/n; shift invariance; -10000 mask -> exact 0 (backend/softmax.rs:259-275)
    np.testing.assert_allclose(ops.softmax(np.full((2, 8), 3.0, np.float32)), 1 / 8, rtol=1e-7)
    np.testing.assert_allclose(ops.softmax(x + 100.0), ops.softmax(x), rtol=2e-5)
    m = ops.softmax(np.array([[0.0, -10000.0, 0.5]], dtype=np.float32))
    assert m[0, 1] == 0.0 and abs(m.sum() - 1.0) < 1e-6
    # 4096-wide row with its own closed form (backend/softmax.rs:299-313): geometric weights
    n = 4096
    row = (np.arange(n, dtype=np.float32) % 2)
    s = ops.softmax(row[None])[0]
    e = np.exp(1.0)
    np.testing.assert_allclose(s[1] / s[0], e, rtol=1e-6)
    np.testing.assert_allclose(s.sum(), 1.0, rtol=1e-6)


def test_pow_and_cast_and_intdiv_semantics():
    x = np.array([1.5, -2.0, 0.0, 3.0], dtype=np.float32)
    assert np.array_equal(ops.pow_(x, np.float32(2.0)), x * x)
    assert np.array_equal(ops.pow_(np.abs(x), np.float32(0.5)), np.sqrt(np.abs(x)))
    assert np.array_equal(ops.pow_(np.array([2, -3, 5], dtype=np.int64), np.array([10, 3, 0])),
                          np.array([1024, -27, 1]))
    # llround: half away from zero (2^-1 = 0.5 -> 1)
    assert ops.pow_(np.array([2], dtype=np.int32), np.array([-1], dtype=np.int32))[0] == 1
    assert np.array_equal(ops.cast(np.array([2.9, -2.9, 0.4], dtype=np.float32), 6), [2, -2, 0])
    assert np.array_equal(ops.cast(np.array([0.0, -0.0, 1e-9, np.nan], dtype=np.float32), 9),
                          [False, False, True, True])
    assert np.array_equal(ops.cast(np.array([True, False]), 1), np.array([1.0, 0.0], np.float32))
    assert np.array_equal(ops.div(np.array([7, -7, 7, -7], dtype=np.int32),
                                  np.array([2, 2, -2, -2], dtype=np.int32)), [3, -3, -3, 3])
    assert np.array_equal(ops.range_(np.int64(2), np.int64(11), np.int64(3)), [2, 5, 8])
    assert np.array_equal(ops.range_(np.int64(10), np.int64(1), np.int64(-4)), [10, 6, 2])
    assert ops.range_(np.float32(0), np.float32(1), np.float32(0.25)).tolist() == [0, 0.25, 0.5, 0.75]
    assert np.array_equal(ops.reduce_mean(np.full((3, 4), 2.5, np.float32), [1]), np.full((3, 1), 2.5))


def test_weight_storage_rounding_closed_forms_and_torch():
    """oracle.ops.store_weights: closed forms a wrong rounding rule fails (ties to even in both
    directions, carry into the exponent, overflow to infinity, NaN kept, signed zero), then torch's
    own CPU conversions on random floats of every magnitude."""
    import torch

    def f32(bits):
        return np.array(bits, dtype=np.uint32).view(np.float32)

    # bfloat16 keeps the upper 16 bits: 0x3F80_8000 is the tie between 0x3F80 (even) and 0x3F81
    got = ops.store_weights(f32([0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0x3FFF8000, 0x7F7FFFFF,
                                 0x80000000, 0x00000001, 0xFF800000]), "bf16").view(np.uint32)
    assert [hex(v) for v in got] == [hex(v) for v in
                                     [0x3F800000, 0x3F820000, 0x3F810000, 0x3F800000, 0x40000000, 0x7F800000,
                                      0x80000000, 0x00000000, 0xFF800000]]
    assert np.isnan(ops.store_weights(f32([0x7FC00001, 0x7F800001, 0xFFFFFFFF]), "bf16")).all()
    # binary16: 11 significant bits, so 2049 is the tie between 2048 (even) and 2050, 2051 between
    # 2050 and 2052 (even); 65520 is the tie that overflows; 2^-25 is the tie between 0 and the
    # smallest subnormal 2^-24
    np.testing.assert_array_equal(
        ops.store_weights(np.array([2049.0, 2051.0, 65519.0, 65520.0, 2.0 ** -25, 1.5 * 2.0 ** -25, -0.0],
                                   dtype=np.float32), "f16"),
        np.array([2048.0, 2052.0, 65504.0, np.inf, 0.0, 2.0 ** -24, -0.0], dtype=np.float32))
    rng = np.random.default_rng(16)
    bits = rng.integers(0, 2 ** 32, size=200000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[np.isfinite(x)]
    for name, tdt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        exp = torch.from_numpy(x.copy()).to(tdt).to(torch.float32).numpy()
        np.testing.assert_array_equal(ops.store_weights(x, name).view(np.uint32), exp.view(np.uint32))
    with pytest.raises(ops.OracleError):
        ops.store_weights(x[:4], "fp8")


# ---- the kernel crate's own known-answer tests (cuda/src/kernels/<op>.rs) ---------------------
import kernel_vectors as kv  # noqa: E402

KC = kv.KERNEL_CASES
ORACLE_BINARY = {"add": ops.add, "sub": ops.sub, "mul": ops.mul, "div": ops.div,
                 "equal": ops.equal, "greater": ops.greater}
ORACLE_UNARY = {"sqrt": ops.sqrt, "neg": ops.neg, "sin": ops.sin, "cos": ops.cos,
                "sigmoid": ops.sigmoid}


def test_kernel_vector_counts():
    """Every kernel-crate file whose tests hold literal vectors is represented."""
    want = {"reduce_mean": 10, "binary": 6, "pow": 35, "where": 1, "unary": 7, "cast": 101,
            "expand": 7, "transpose": 5, "trilu": 6, "scatter_nd": 5, "slice": 20, "gemm": 1}
    assert {k: len(v) for k, v in KC.items()} == want
    assert sorted(s["test"] for s in CASES["kernel_skipped"]) == [
        "test_expand_same_mid_axis", "test_transpose_arbitrary_3d"]


@pytest.mark.parametrize("case", KC["binary"], ids=kv.ids(KC["binary"]))
def test_kernel_binary_vectors(case):
    a, b = (kv.arr(case, k, shape=case["shape"]) for k in "ab")
    got = ORACLE_BINARY[case["op"]](a, b)
    exp = decode(case["expected"], got.dtype)
    kv.check(got, exp, case["compare"], case["epsilon"])


@pytest.mark.parametrize("case", KC["pow"], ids=kv.ids(KC["pow"]))
def test_kernel_pow_vectors(case):
    """cuda/src/kernels/pow.rs:248-775: all 35 (base, exponent) element-type pairs the crate tests,
    including the pairs the provider leaves disabled (backend/pow.rs:133-160)."""
    a = kv.arr(case, "a", "a_dtype", case["shape"])
    b = kv.arr(case, "b", "b_dtype", case["shape"])
    got = ops.pow_(a, b)
    assert got.dtype == a.dtype
    kv.check(got, decode(case["expected"], a.dtype), case["compare"], case["epsilon"])


@pytest.mark.parametrize("case", KC["where"], ids=kv.ids(KC["where"]))
def test_kernel_where_vectors(case):
    x, y = (kv.arr(case, k, shape=case["shape"]) for k in "xy")
    cond = np.array(case["cond"], dtype=bool).reshape(case["shape"])
    kv.check(ops.where(cond, x, y), decode(case["expected"], x.dtype))


@pytest.mark.parametrize("case", KC["unary"], ids=kv.ids(KC["unary"]))
def test_kernel_unary_vectors(case):
    x = kv.arr(case, "input")
    kv.check(ORACLE_UNARY[case["op"]](x), decode(case["expected"], x.dtype), case["compare"],
             case["epsilon"])


@pytest.mark.parametrize("case", KC["cast"], ids=kv.ids(KC["cast"]))
def test_kernel_cast_vectors(case):
    """cuda/src/kernels/cast.rs:372-1415."""
    x = kv.arr(case, "input", "src_dtype")
    got = ops.cast(x, ops.NP_TO_ONNX[np.dtype(case["dst_dtype"])])
    assert got.dtype == np.dtype(case["dst_dtype"])
    kv.check(got, decode(case["expected"], got.dtype))


@pytest.mark.parametrize("case", KC["expand"], ids=kv.ids(KC["expand"]))
def test_kernel_expand_vectors(case):
    x = kv.arr(case, "input", shape=case["input_shape"])
    got = ops.expand(x, case["output_shape"])
    assert list(got.shape) == case["output_shape"]
    kv.check(got, decode(case["expected"], x.dtype))
    flat = loops.expand_loop(case["input_shape"], case["output_shape"], x.reshape(-1).tolist()) \
        if hasattr(loops, "expand_loop") and x.size else None
    if flat is not None:
        kv.check(np.array(flat, dtype=x.dtype), decode(case["expected"], x.dtype))


def test_kernel_expand_mid_axis_stand_in():
    """cuda/src/kernels/expand.rs:174-189 builds its expectation with loops (each of the three
    values repeated four times, the whole twice); restated here."""
    x = np.array([1.0, 2.0, 3.0]).reshape(1, 3, 1)
    exp = np.tile(np.repeat(np.array([1.0, 2.0, 3.0]), 4), 2)
    kv.check(ops.expand(x, [2, 3, 4]), exp)


@pytest.mark.parametrize("case", KC["transpose"], ids=kv.ids(KC["transpose"]))
def test_kernel_transpose_vectors(case):
    x = kv.arr(case, "input", shape=case["input_shape"])
    if case.get("expect_error"):
        with pytest.raises(Exception):
            ops.transpose(x, case["perm"])
        return
    kv.check(ops.transpose(x, case["perm"]), decode(case["expected"], x.dtype))


def test_kernel_transpose_3d_stand_in():
    """cuda/src/kernels/transpose.rs:181-198: [2,3,4] with perm [2,0,1]; its loops say
    out[o0,o1,o2] = in[o1,o2,o0]."""
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    got = ops.transpose(x, [2, 0, 1])
    exp = np.array([x[o1, o2, o0] for o0 in range(4) for o1 in range(2) for o2 in range(3)],
                   dtype=np.int32)
    kv.check(got, exp)


@pytest.mark.parametrize("case", KC["trilu"], ids=kv.ids(KC["trilu"]))
def test_kernel_trilu_vectors(case):
    """cuda/src/kernels/trilu.rs:138-196. The reference kernel leaves what lies outside the triangle
    unwritten and its tests rely on a zero-filled output; the oracle writes the zeros."""
    x = kv.arr(case, "input", shape=case["shape"])
    kv.check(ops.trilu(x, k=case["k"], upper=int(case["upper"])), decode(case["expected"], x.dtype))


@pytest.mark.parametrize("case", KC["scatter_nd"], ids=kv.ids(KC["scatter_nd"]))
def test_kernel_scatter_nd_vectors(case):
    """cuda/src/kernels/scatter_nd.rs:318-417 over zero data (where the reference's `in + 0*out`
    and plain assignment agree)."""
    data = np.zeros(case["data_shape"], dtype=case["dtype"])
    idx = np.array(case["indices"], dtype=np.int64).reshape(case["indices_shape"])
    upd = kv.arr(case, "updates", shape=case["updates_shape"])
    kv.check(ops.scatter_nd(data, idx, upd), decode(case["expected"], data.dtype))


@pytest.mark.parametrize("case", KC["slice"], ids=kv.ids(KC["slice"]))
def test_kernel_slice_vectors(case):
    """cuda/src/kernels/slice.rs:200-700: negative steps, INT64 sentinels, clamping, absent axes /
    steps (empty slices in the reference's kernel tests)."""
    x = kv.arr(case, "input", shape=case["input_shape"])
    got = ops.slice_(x, case["starts"], case["ends"], case["axes"] or None, case["steps"] or None)
    # operator level: the shape rule of backend/slice.rs:417-452 decides the output shape
    assert list(got.shape) == case.get("onnx_output_shape", case["output_shape"])
    kv.check(got, decode(case.get("onnx_expected", case["expected"]), x.dtype))
    # kernel level: the caller gives the output shape, element i of a dim is input element
    # start + i * step (slice_op_macros.cuh:38-75)
    res = ops.slice_resolve(case["input_shape"], case["starts"], case["ends"], case["axes"] or None,
                            case["steps"] or None)
    idx = tuple(s0 + np.arange(n) * st for (s0, st, _), n in zip(res, case["output_shape"]))
    kernel_level = x[np.ix_(*idx)] if x.ndim else x
    kv.check(kernel_level, decode(case["expected"], x.dtype))


@pytest.mark.parametrize("case", KC["gemm"], ids=kv.ids(KC["gemm"]))
def test_kernel_gemm_vectors(case):
    a = kv.arr(case, "lhs", shape=case["lhs_shape"])
    b = kv.arr(case, "rhs", shape=case["rhs_shape"])
    assert not case["trans_a"] and not case["trans_b"]
    kv.check(ops.matmul(a, b), decode(case["expected"], a.dtype))
    kv.check(ops.matmul(a, b, "f32"), decode(case["expected"], a.dtype))
