"""The known-answer vectors of the reference's kernel crate (the #[test]s of cuda/src/kernels/*.rs,
extracted into tests/golden/reference_cases.json) fed to the C-ABI entry points that replace those
kernels, through `rmlk_amd.kernels`. Shapes, strides and element types are the reference tests';
the comparison is the one its assertion macro makes. Where a reference test fixes something the
operator level decides differently (Slice output shapes), both levels are replayed."""
import numpy as np
import pytest

import kernel_vectors as kv
from helpers import to_dev, to_np
from optest import decode

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

KC = kv.KERNEL_CASES
BINARY_OP = {"add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "equal": 5, "greater": 6}
UNARY_OP = {"sqrt": 0, "neg": 1, "sin": 2, "cos": 3, "sigmoid": 4}
# element types of rmlk_hip_binary's POW (include/rmlk_hip.h): the pairs of backend/pow.rs:123-132
# plus DOUBLE; the kernel crate also tests u8 / i8 / f16 pairs that its provider leaves disabled
POW_TYPES = {"float32", "float64", "int32", "int64"}


def _k():
    from rmlk_amd import kernels
    return kernels


def dense(shape):
    out, acc = [0] * len(shape), 1
    for i in range(len(shape) - 1, -1, -1):
        out[i] = acc
        acc *= shape[i]
    return out


def empty_like_np(dtype, n, device):
    return to_dev(np.zeros(n, dtype=dtype), device)


@pytest.mark.parametrize("case", KC["binary"], ids=kv.ids(KC["binary"]))
def test_binary(device, case):
    """cuda/src/kernels/{add,sub,mul,div,equal,greater}.rs test_f32"""
    k = _k()
    a, b = (kv.arr(case, key) for key in "ab")
    out_dtype = np.bool_ if case["op"] in ("equal", "greater") else a.dtype
    out = empty_like_np(out_dtype, a.size, device)
    st = dense(case["shape"])
    k.binary(BINARY_OP[case["op"]], to_dev(a, device), to_dev(b, device), out, case["shape"], st, st)
    kv.check(to_np(out), decode(case["expected"], out_dtype), case["compare"], case["epsilon"])


@pytest.mark.parametrize("case", KC["pow"], ids=kv.ids(KC["pow"]))
def test_pow(device, case):
    """cuda/src/kernels/pow.rs:248-775"""
    k = _k()
    a, b = kv.arr(case, "a", "a_dtype"), kv.arr(case, "b", "b_dtype")
    out = empty_like_np(a.dtype, a.size, device)
    st = dense(case["shape"])
    call = lambda: k.binary(BINARY_OP["pow"], to_dev(a, device), to_dev(b, device), out,  # noqa: E731
                            case["shape"], st, st)
    if case["a_dtype"] not in POW_TYPES or case["b_dtype"] not in POW_TYPES:
        # not an element-type pair of the boundary (nor of the reference's provider)
        with pytest.raises(k.RmlkError):
            call()
        return
    call()
    kv.check(to_np(out), decode(case["expected"], a.dtype), case["compare"], case["epsilon"])


@pytest.mark.parametrize("case", KC["where"], ids=kv.ids(KC["where"]))
def test_where(device, case):
    """cuda/src/kernels/whereop.rs:126-173"""
    k = _k()
    x, y = kv.arr(case, "x"), kv.arr(case, "y")
    cond = np.array(case["cond"], dtype=np.bool_)
    out = empty_like_np(x.dtype, x.size, device)
    st = dense(case["shape"])
    k.where(to_dev(x, device), to_dev(y, device), to_dev(cond, device), out, case["shape"], st, st, st)
    kv.check(to_np(out), decode(case["expected"], x.dtype))


@pytest.mark.parametrize("case", KC["unary"], ids=kv.ids(KC["unary"]))
def test_unary(device, case):
    """cuda/src/kernels/{sqrt,neg,sin,cos}.rs test_f32, sigmoid.rs:66-91"""
    k = _k()
    x = kv.arr(case, "input")
    out = empty_like_np(x.dtype, x.size, device)
    k.unary(UNARY_OP[case["op"]], to_dev(x, device), out)
    kv.check(to_np(out), decode(case["expected"], x.dtype), case["compare"], case["epsilon"])


@pytest.mark.parametrize("case", KC["cast"], ids=kv.ids(KC["cast"]))
def test_cast(device, case):
    """cuda/src/kernels/cast.rs:372-1415"""
    k = _k()
    x = kv.arr(case, "input", "src_dtype")
    out = empty_like_np(case["dst_dtype"], x.size, device)
    k.cast(to_dev(x, device), out)
    kv.check(to_np(out), decode(case["expected"], case["dst_dtype"]))


@pytest.mark.parametrize("case", KC["reduce_mean"], ids=kv.ids(KC["reduce_mean"]))
def test_reduce_mean(device, case):
    """cuda/src/kernels/reduce_mean.rs:156-266"""
    k = _k()
    x = decode(case["data"], np.float32)
    exp = decode(case["expected"], np.float32)
    out = empty_like_np(np.float32, exp.size, device)
    k.reduce_mean(to_dev(x, device), out, case["shape"], case["axes"])
    kv.check(to_np(out), exp, "relative", 1e-6)


@pytest.mark.parametrize("case", KC["expand"], ids=kv.ids(KC["expand"]))
def test_expand(device, case):
    """cuda/src/kernels/expand.rs:153-247"""
    k = _k()
    x = kv.arr(case, "input")
    exp = decode(case["expected"], x.dtype)
    out = empty_like_np(x.dtype, exp.size, device)
    k.expand(to_dev(x, device), out, case["input_shape"], case["output_shape"])
    kv.check(to_np(out), exp)


def test_expand_mid_axis_stand_in(device):
    """cuda/src/kernels/expand.rs:174-189 (expectation built by loops there: each of the three
    values four times, the whole twice)."""
    k = _k()
    x = np.array([1.0, 2.0, 3.0])
    out = empty_like_np(np.float64, 24, device)
    k.expand(to_dev(x, device), out, [1, 3, 1], [2, 3, 4])
    kv.check(to_np(out), np.tile(np.repeat(x, 4), 2))


@pytest.mark.parametrize("case", KC["transpose"], ids=kv.ids(KC["transpose"]))
def test_transpose(device, case):
    """cuda/src/kernels/transpose.rs:153-218"""
    k = _k()
    x = kv.arr(case, "input")
    if case.get("expect_error"):
        # the reference's launch helper asserts perm.len() == rank; so does the wrapper
        with pytest.raises(AssertionError):
            k.transpose(to_dev(x, device), empty_like_np(x.dtype, x.size, device),
                        case["input_shape"], case["perm"])
        return
    exp = decode(case["expected"], x.dtype)
    out = empty_like_np(x.dtype, exp.size, device)
    # a scalar crosses the boundary as shape [1] (rmlk_dims has rank >= 1)
    k.transpose(to_dev(x, device), out, case["input_shape"] or [1], case["perm"] or [0])
    kv.check(to_np(out), exp)


def test_transpose_3d_stand_in(device):
    """cuda/src/kernels/transpose.rs:181-198: out[o0,o1,o2] = in[o1,o2,o0] for perm [2,0,1]."""
    k = _k()
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    out = empty_like_np(np.int32, 24, device)
    k.transpose(to_dev(x, device), out, [2, 3, 4], [2, 0, 1])
    exp = np.array([x[o1, o2, o0] for o0 in range(4) for o1 in range(2) for o2 in range(3)],
                   dtype=np.int32)
    kv.check(to_np(out), exp)


@pytest.mark.parametrize("case", KC["trilu"], ids=kv.ids(KC["trilu"]))
def test_trilu(device, case):
    """cuda/src/kernels/trilu.rs:138-196. The output buffer starts as garbage here: the zeros
    outside the triangle are written by the kernel, not inherited from the allocation."""
    k = _k()
    x = kv.arr(case, "input")
    out = to_dev(np.full(x.size, 77, dtype=x.dtype), device)
    b, r, c = case["shape"]
    k.trilu(to_dev(x, device), out, b, r, c, case["upper"], case["k"])
    kv.check(to_np(out), decode(case["expected"], x.dtype))


@pytest.mark.parametrize("copy", [False, True], ids=["in_place", "with_copy"])
@pytest.mark.parametrize("case", KC["scatter_nd"], ids=kv.ids(KC["scatter_nd"]))
def test_scatter_nd(device, case, copy):
    """cuda/src/kernels/scatter_nd.rs:318-417 (zero data; rank-1 indices of the reference's kernel
    convention are recorded as [n, 1])."""
    k = _k()
    data = np.zeros(int(np.prod(case["data_shape"])), dtype=case["dtype"])
    idx = np.array(case["indices"], dtype=np.int64)
    upd = kv.arr(case, "updates")
    tuple_size = case["indices_shape"][-1]
    n_tuples = idx.size // tuple_size
    err = torch.zeros(1, dtype=torch.int32, device=device)
    if copy:
        out = to_dev(np.full(data.size, 55, dtype=data.dtype), device)
        k.scatter_nd_copy(to_dev(idx, device), to_dev(upd, device), to_dev(data, device), out,
                          case["data_shape"], n_tuples, tuple_size, err_flag=err)
    else:
        out = to_dev(data, device)
        k.scatter_nd(to_dev(idx, device), to_dev(upd, device), out, case["data_shape"], n_tuples,
                     tuple_size, err_flag=err)
    assert int(err.item()) == 0
    kv.check(to_np(out), decode(case["expected"], data.dtype))


@pytest.mark.parametrize("case", KC["slice"], ids=kv.ids(KC["slice"]))
def test_slice_kernel_level(device, case):
    """cuda/src/kernels/slice.rs:200-700 at the kernel's level: the caller gives the output shape
    (the reference's tests do, three of them one the operator would not produce), the kernel gets
    the resolved start and the step per dim. The starts come from the CPU oracle's restatement of
    the clamp rules (slice_op_macros.cuh:38-75)."""
    from oracle import ops
    k = _k()
    x = kv.arr(case, "input")
    exp = decode(case["expected"], x.dtype)
    out = empty_like_np(x.dtype, exp.size, device)
    if not case["input_shape"]:
        pytest.skip("rank 0: nothing to resolve; covered at the operator level")
    res = ops.slice_resolve(case["input_shape"], case["starts"], case["ends"], case["axes"] or None,
                            case["steps"] or None)
    starts = [s if n else 0 for (s, _, _), n in zip(res, case["output_shape"])]
    k.slice_(to_dev(x, device), out, case["input_shape"], starts, [st for _, st, _ in res],
             case["output_shape"])
    kv.check(to_np(out), exp)


@pytest.mark.parametrize("case", KC["slice"], ids=kv.ids(KC["slice"]))
def test_slice_operator_level(device, case):
    """The same cases as one-node Slice graphs: starts, ends, axes and steps reach the operator
    as the reference's kernel receives them (INT64 sentinels, negative and oversized values, absent
    axes / steps as absent inputs) and the host rule decides the output shape
    (backend/slice.rs:357-463)."""
    from rmlk_amd.runtime import Builder, GraphBuilder
    x = kv.arr(case, "input", shape=case["input_shape"])
    g = GraphBuilder()
    g.input("x", x.dtype, x.shape)
    names = ["x"]
    for key in ("starts", "ends", "axes", "steps"):
        vals = case[key]
        if key in ("axes", "steps") and not vals:
            names.append(None)
            continue
        g.constant(key, np.array(vals, dtype=np.int64))
        names.append(key)
    while names[-1] is None:
        names.pop()
    g.op("Slice", names, ["y"])
    g.output("y")
    inst = Builder.from_graph(g.build()).build()
    try:
        got = inst.run({"x": x})["y"]
    finally:
        inst.close()
    assert list(got.shape) == case.get("onnx_output_shape", case["output_shape"])
    kv.check(got, decode(case.get("onnx_expected", case["expected"]), x.dtype))


@pytest.mark.parametrize("case", KC["gemm"], ids=kv.ids(KC["gemm"]))
def test_gemm(device, case):
    """cuda/src/kernels/gemm.rs:303-340"""
    k = _k()
    a, b = kv.arr(case, "lhs"), kv.arr(case, "rhs")
    batch, m, kk = case["lhs_shape"]
    n = case["rhs_shape"][2]
    out = empty_like_np(a.dtype, batch * m * n, device)
    k.matmul(to_dev(a, device), to_dev(b, device), out, batch, m, n, kk, kk, n, n, m * kk, kk * n,
             m * n, case["trans_a"], case["trans_b"])
    kv.check(to_np(out), decode(case["expected"], a.dtype))
