"""CPU oracle: numpy restatement of the operator path of the reference (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
product (rmlk_amd) never does.

Every function states which reference file it follows. Where the reference deviates from ONNX /
ONNX Runtime (its own test oracle), the ONNX behaviour is restated and the deviation is named:
  - Softmax: max-subtracted (reference uses cuDNN SOFTMAX_FAST, backend/softmax.rs:98).
  - Trilu: zeros outside the triangle (reference leaves them unwritten, trilu_op_macros.cuh:39-41).
  - ScatterND "none": assignment (reference computes in + 0*out, ptx/scatter_nd.cu:10).
  - Gather / index normalisation: idx == dim is rejected (reference accepts it, utils/mod.rs:170).
  - integer x / 0 = 0 (reference: undefined).

Pinning status: every function here is checked in tests/test_oracle_*.py against the
known-answer vectors extracted from the reference's own tests (tests/golden/reference_cases.json),
against the pure-Python loop restatement of the reference kernels (oracle/loops.py) and against
closed forms. The whole-graph Llama results have no reference-held vectors: parity unpinned for
those (see oracle/graph.py).
"""
from __future__ import annotations

import numpy as np

# ONNX TensorProto.DataType numbers (schema/src/tensor.rs:404-430 maps DataType to these).
ONNX_DTYPES = {
    1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32, 7: np.int64,
    9: np.bool_, 10: np.float16, 11: np.float64, 12: np.uint32, 13: np.uint64,
}
NP_TO_ONNX = {np.dtype(v): k for k, v in ONNX_DTYPES.items()}


class OracleError(Exception):
    """An input the reference's operator dispatch rejects."""


def normalize_index(index: int, size: int) -> int:
    """runtime/src/utils/mod.rs:155-175, with idx == size rejected (the reference accepts it)."""
    i = int(index)
    if i < 0:
        i += size
    if i < 0 or i >= size:
        raise OracleError(f"index {index} out of range for size {size}")
    return i


# ---- broadcast binary ops (cuda/src/ptx/{add,sub,mul,div,equal,greater}.cu) ----------------------
def _binary_check(a, b):
    a = np.asarray(a)
    b = np.asarray(b)
    try:
        np.broadcast_shapes(a.shape, b.shape)
    except ValueError as e:  # backend/binary.rs:164-168
        raise OracleError("incompatible shapes for broadcasting") from e
    return a, b


def add(a, b):
    a, b = _binary_check(a, b)
    with np.errstate(all="ignore"):
        return (a + b).astype(a.dtype)


def sub(a, b):
    a, b = _binary_check(a, b)
    with np.errstate(all="ignore"):
        return (a - b).astype(a.dtype)


def mul(a, b):
    a, b = _binary_check(a, b)
    with np.errstate(all="ignore"):
        return (a * b).astype(a.dtype)


def div(a, b):
    """cuda/src/ptx/div.cu:6-12: IEEE for floats; C truncating division for integers."""
    a, b = _binary_check(a, b)
    if np.issubdtype(a.dtype, np.integer):
        a_, b_ = np.broadcast_arrays(a, b)
        info = np.iinfo(a.dtype)
        zero = b_ == 0
        wrap = (a_ == info.min) & (b_ == -1)  # MIN / -1 wraps to MIN
        safe_b = np.where(zero | wrap, 1, b_).astype(a.dtype)
        with np.errstate(all="ignore"):
            q = a_ // safe_b  # floor
            r = a_ - q * safe_b
            q = q + ((r != 0) & ((a_ < 0) != (safe_b < 0)))  # floor -> truncation
        q = np.where(zero, 0, q)
        q = np.where(wrap, info.min, q)
        return q.astype(a.dtype)
    with np.errstate(all="ignore"):
        return (a / b).astype(a.dtype)


def equal(a, b):
    a, b = _binary_check(a, b)
    return np.equal(a, b)


def greater(a, b):
    a, b = _binary_check(a, b)
    return np.greater(a, b)


def _llround(x):
    """C llround: half away from zero."""
    return np.where(x >= 0, np.floor(x + 0.5), -np.floor(-x + 0.5))


def pow_(a, b):
    """cuda/src/ptx/pow.cu:18-65. float base: powf(x, (float)y); int base: llround(pow(double)).

    Exponents 2, 3, 0.5 are x*x, x*x*x, sqrt(x) (what ONNX Runtime's CPU Pow does and what the
    HIP kernel does), which are correctly rounded.
    """
    a, b = _binary_check(a, b)
    with np.errstate(all="ignore"):
        if np.issubdtype(a.dtype, np.floating):
            e = b.astype(a.dtype)
            a_, e_ = np.broadcast_arrays(a, e)
            generic = np.power(a_.astype(np.float64), e_.astype(np.float64)).astype(a.dtype)
            out = generic
            out = np.where(e_ == 2, (a_ * a_).astype(a.dtype), out)
            out = np.where(e_ == 3, ((a_ * a_).astype(a.dtype) * a_).astype(a.dtype), out)
            out = np.where(e_ == 0.5, np.sqrt(a_).astype(a.dtype), out)
            return out.astype(a.dtype)
        r = np.power(a.astype(np.float64), b.astype(np.float64))
        return _llround(r).astype(a.dtype)


def where(cond, x, y):
    """cuda/src/ptx/headers/ternary_op_macro.cuh:1-34; ONNX input order (cond, x, y)."""
    cond = np.asarray(cond)
    x = np.asarray(x)
    y = np.asarray(y)
    try:
        np.broadcast_shapes(cond.shape, x.shape, y.shape)
    except ValueError as e:
        raise OracleError("incompatible shapes for broadcasting") from e
    return np.where(cond.astype(bool), x, y).astype(x.dtype)


# ---- unary (cuda/src/ptx/{sqrt,neg,sin,cos}.cu, cuda/src/kernels/sigmoid.rs) ----------------------
def _f64_round(fn, x):
    x = np.asarray(x)
    with np.errstate(all="ignore"):
        return fn(x.astype(np.float64)).astype(x.dtype)


def sqrt(x):
    return _f64_round(np.sqrt, x)


def neg(x):
    x = np.asarray(x)
    with np.errstate(all="ignore"):
        return (-x).astype(x.dtype)


def sin(x):
    return _f64_round(np.sin, x)


def cos(x):
    return _f64_round(np.cos, x)


def sigmoid(x):
    return _f64_round(lambda v: 1.0 / (1.0 + np.exp(-v)), x)


def cast(x, to: int):
    """cuda/src/ptx/cast.cu:6-124: C static_cast. float -> int truncates toward zero; values the
    target cannot hold follow the rule stated below."""
    x = np.asarray(x)
    dst = np.dtype(ONNX_DTYPES[int(to)])
    if dst == np.bool_:
        return x != 0
    if x.dtype == np.bool_:
        return x.astype(dst)
    if np.issubdtype(x.dtype, np.floating) and np.issubdtype(dst, np.integer):
        # NaN -> 0; out of range saturates at the limits of the 32-bit type of the same signedness
        # (64-bit for 64-bit targets); 8- and 16-bit targets keep the low bits of that 32-bit value
        # (the reference's vector half 32768.0 -> int16 -32768, cuda/src/kernels/cast.rs:524-539)
        wide = dst if dst.itemsize == 8 else np.dtype(np.int32 if dst.kind == "i" else np.uint32)
        info = np.iinfo(wide)
        with np.errstate(all="ignore"):
            v = np.trunc(x.astype(np.float64))
            v = np.where(np.isnan(v), 0.0, v)
            big = v >= float(info.max)
            small = v <= float(info.min)
            mid = np.where(big | small, 0.0, v).astype(wide)
            w = np.where(big, info.max, np.where(small, info.min, mid)).astype(wide)
        return w.astype(dst)
    with np.errstate(all="ignore"):
        return x.astype(dst)


# ---- reductions -------------------------------------------------------------------------------
def reduce_mean(x, axes=None, keepdims=1, noop_with_empty_axes=0):
    """cuda/src/ptx/reduce_mean.cu:5-9 accumulates in double and divides in double
    (aggregation_op_macros.cuh:26-47); axes rules follow backend/reduce_mean.rs:77-130."""
    x = np.asarray(x)
    rank = max(x.ndim, 1)
    if axes is None or len(axes) == 0:
        if axes is not None and noop_with_empty_axes:
            return x.copy()
        ax = tuple(range(x.ndim))
    else:
        ax = tuple(sorted({normalize_index(a, rank) for a in axes}))
    with np.errstate(all="ignore"):
        return np.mean(x, axis=ax, dtype=np.float64, keepdims=bool(keepdims)).astype(x.dtype)


def softmax(x, axis=-1):
    """exp(x - max) / sum along `axis` (ONNX opset 13 semantics, what ONNX Runtime computes)."""
    x = np.asarray(x)
    ax = normalize_index(axis, x.ndim)
    with np.errstate(all="ignore"):
        v = x.astype(np.float64)
        m = np.max(v, axis=ax, keepdims=True)
        e = np.exp(v - m)
        return (e / np.sum(e, axis=ax, keepdims=True)).astype(x.dtype)


def matmul(a, b, accumulate="f64"):
    """numpy.matmul semantics (ONNX MatMul); shape rules of backend/matmul.rs:234-305.

    accumulate="f64" is the truth used for parity; "f32" is BLAS sgemm, used when timing.
    """
    a = np.asarray(a)
    b = np.asarray(b)
    if a.ndim == 0 or b.ndim == 0:
        raise OracleError("ZeroRank")
    ka = a.shape[-1]
    kb = b.shape[0] if b.ndim == 1 else b.shape[-2]
    if ka != kb:
        raise OracleError("IncompatibleDimForMul")
    try:
        if accumulate == "f64":
            return np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(a.dtype)
        return np.matmul(a, b)
    except ValueError as e:
        raise OracleError("IncompatibleDimForBroadcast") from e


# ---- data movement ----------------------------------------------------------------------------
def transpose(x, perm=None):
    """cuda/src/ptx/headers/transpose_op_macros.cuh:1-25; default perm reverses the dims."""
    x = np.asarray(x)
    if perm is None:
        perm = list(range(x.ndim))[::-1]
    return np.asarray(order="C", a=np.transpose(x, [int(p) for p in perm]))


def expand(x, shape):
    """cuda/src/ptx/headers/expand_op_macros.cuh:1-31; ONNX Expand: two-way broadcast."""
    x = np.asarray(x)
    try:
        out_shape = np.broadcast_shapes(x.shape, tuple(int(s) for s in shape))
    except ValueError as e:
        raise OracleError("incompatible shapes for expand") from e
    return np.asarray(order="C", a=np.broadcast_to(x, out_shape))


def slice_resolve(shape, starts, ends, axes=None, steps=None):
    """ONNX Slice clamp rules as the reference applies them
    (backend/slice.rs:357-463, slice_op_macros.cuh:38-75).
    Returns per-dim (start, step, count)."""
    rank = len(shape)
    if axes is None:
        axes = list(range(len(starts)))
    if steps is None:
        steps = [1] * len(starts)
    if len(steps) != len(axes):
        raise OracleError("StepsAndAxesLengthMismatch")
    if len(axes) != len(starts) or len(starts) != len(ends):
        raise OracleError("axes must have the same length as starts")
    res = [(0, 1, int(shape[d])) for d in range(rank)]
    for i, raw_axis in enumerate(axes):
        axis = int(raw_axis)
        if axis < 0:
            axis += rank
        if axis < 0 or axis >= rank:
            raise OracleError("AxisOutOfRange")
        step = int(steps[i])
        if step == 0:
            raise OracleError("ZeroStep")
        dim = int(shape[axis])
        start = int(starts[i])
        if start < 0:
            start += dim
        if start < 0:
            start = 0
        if step > 0 and start > dim:
            start = dim
        elif step < 0 and start >= dim:
            start = dim - 1
        end = int(ends[i])
        if end < 0:
            end += dim
        if end < -1:
            end = -1
        if step > 0 and end > dim:
            end = dim
        elif step < 0 and end >= dim:
            end = dim - 1
        if (step < 0 and start < end) or (step > 0 and start >= end):
            count = 0
        elif step > 0:
            count = -(-(end - start) // step)
        else:
            count = -(-(start - end) // (-step))
        res[axis] = (start, step, count)
    return res


def slice_(x, starts, ends, axes=None, steps=None):
    x = np.asarray(x)
    res = slice_resolve(x.shape, list(np.asarray(starts).reshape(-1)),
                        list(np.asarray(ends).reshape(-1)),
                        None if axes is None else list(np.asarray(axes).reshape(-1)),
                        None if steps is None else list(np.asarray(steps).reshape(-1)))
    idx = tuple(np.arange(c, dtype=np.int64) * st + s for (s, st, c) in res)
    return np.asarray(order="C", a=x[np.ix_(*idx)]) if x.ndim else x.copy()


def concat(xs, axis):
    """backend/concat.rs:28-76, 138-199: same rank, same dims off-axis; scalars rejected."""
    xs = [np.asarray(x) for x in xs]
    if xs[0].ndim == 0:
        raise OracleError("ScalarsAreNotAllowed")
    ax = normalize_index(axis, xs[0].ndim)
    for x in xs:
        if x.ndim != xs[0].ndim:
            raise OracleError("ShapeMismatch")
        for d in range(x.ndim):
            if d != ax and x.shape[d] != xs[0].shape[d]:
                raise OracleError("DimensionMismatch")
    return np.concatenate(xs, axis=ax)


def gather(data, indices, axis=0):
    """backend/gather.rs:164-258: out.shape = data[:axis] ++ idx.shape ++ data[axis+1:]."""
    data = np.asarray(data)
    indices = np.asarray(indices)
    if data.ndim == 0:
        raise OracleError("ScalarInputDataNotAllowed")
    ax = normalize_index(axis, data.ndim)
    dim = data.shape[ax]
    flat = [normalize_index(i, dim) for i in indices.reshape(-1)]
    idx = np.array(flat, dtype=np.int64).reshape(indices.shape)
    return np.asarray(order="C", a=np.take(data, idx, axis=ax))


def scatter_nd(data, indices, updates, reduction="none"):
    """cuda/src/ptx/headers/scatter_op_macros.cuh:19-93 with "none" as plain assignment.
    Tuples are applied in order (duplicates: last one wins for "none")."""
    data = np.asarray(data)
    indices = np.asarray(indices)
    updates = np.asarray(updates)
    out = data.copy()
    if indices.ndim < 1:
        raise OracleError("indices rank must be >= 1")
    t = indices.shape[-1]
    if t > data.ndim:
        raise OracleError("index tuple longer than data rank")
    tuples = indices.reshape(-1, t)
    slice_shape = data.shape[t:]
    upd = updates.reshape((tuples.shape[0],) + tuple(slice_shape))
    for n, tup in enumerate(tuples):
        key = tuple(normalize_index(int(v), data.shape[d]) for d, v in enumerate(tup))
        with np.errstate(all="ignore"):
            if reduction == "none":
                out[key] = upd[n]
            elif reduction == "add":
                out[key] = out[key] + upd[n]
            elif reduction == "mul":
                out[key] = out[key] * upd[n]
            elif reduction == "max":
                out[key] = np.where(upd[n] > out[key], upd[n], out[key])
            elif reduction == "min":
                out[key] = np.where(upd[n] < out[key], upd[n], out[key])
            else:
                raise OracleError(f"unknown reduction {reduction}")
    return out


def trilu(x, k=0, upper=1):
    """cuda/src/ptx/headers/trilu_op_macros.cuh:1-43 with zero fill; a rank-2 input is one matrix
    (runtime/src/utils/mod.rs:226-239)."""
    x = np.asarray(x)
    if x.ndim < 2:
        raise OracleError("trilu needs rank >= 2")
    return (np.triu(x, int(k)) if upper else np.tril(x, int(k))).astype(x.dtype)


# ---- metadata ops (backend/{reshape,unsqueeze,shape,range,constant_of_shape}.rs) ---------------
def reshape(x, shape, allowzero=0):
    x = np.asarray(x)
    shape = [int(s) for s in np.asarray(shape).reshape(-1)]
    out = []
    for i, s in enumerate(shape):
        if s == 0 and not allowzero:
            out.append(x.shape[i])
        else:
            out.append(s)
    if out.count(-1) > 1:
        raise OracleError("more than one -1 in reshape")
    return x.reshape(out)


def unsqueeze(x, axes):
    x = np.asarray(x)
    axes = [int(a) for a in np.asarray(axes).reshape(-1)]
    rank = x.ndim + len(axes)
    norm = sorted(normalize_index(a, rank) for a in axes)
    if len(set(norm)) != len(norm):
        raise OracleError("duplicate axes")
    out = x
    for a in norm:
        out = np.expand_dims(out, a)
    return out


def shape_(x, start=0, end=None):
    x = np.asarray(x)
    rank = x.ndim
    s = int(start)
    e = rank if end is None else int(end)
    if s < 0:
        s += rank
    if e < 0:
        e += rank
    s = min(max(s, 0), rank)
    e = min(max(e, 0), rank)
    return np.array(x.shape[s:e], dtype=np.int64)


def range_(start, limit, delta):
    """ONNX Range: max(ceil((limit - start) / delta), 0) elements. (The reference truncates the
    integer count, backend/range.rs:140-151; identical whenever delta divides the span.)"""
    start = np.asarray(start)
    dt = start.dtype
    s, l, d = start.reshape(()).item(), np.asarray(limit).reshape(()).item(), np.asarray(delta).reshape(()).item()
    if d == 0:
        raise OracleError("zero delta")
    n = max(int(np.ceil((l - s) / d)), 0)
    return (s + np.arange(n) * d).astype(dt)


def constant_of_shape(shape, value=None):
    shape = [int(s) for s in np.asarray(shape).reshape(-1)]
    if value is None:
        value = np.zeros((1,), dtype=np.float32)
    value = np.asarray(value).reshape(-1)
    return np.full(shape, value[0], dtype=value.dtype)


def store_weights(w, storage: str):
    """Constant weights rounded once to a 16-bit storage type and widened again: what a product over
    stored weights multiplies with. `storage`: "f16" (IEEE binary16, numpy's own conversion) or
    "bf16" (the upper 16 bits of the float after rounding to nearest, ties to even; NaN stays NaN).
    No counterpart in the reference, whose provider holds fp32 only
    (runtime/src/providers/cuda/data.rs:109-126). Pinned in tests/test_oracle_golden.py: ties,
    overflow and special values in closed form, and torch's CPU conversion on random floats."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    if storage == "f16":
        with np.errstate(over="ignore"):
            return w.astype(np.float16).astype(np.float32)
    if storage != "bf16":
        raise OracleError(f"unknown weight storage {storage!r}")
    u = w.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(nan, ((u >> 16) | 0x40) << 16, rounded)
    return (rounded & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(w.shape)
