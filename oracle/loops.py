"""CPU oracle, second opinion: pure-Python loop restatement of the reference's kernels and host
helpers, following their index arithmetic step by step (TEST INFRASTRUCTURE ONLY; small inputs).

oracle/ops.py states WHAT each op computes through numpy routines; this module states HOW the
reference walks its info buffers (shape / stride vectors), so that a transposed operand, a wrong
stride or a dropped dim in either shows up as a disagreement between the two.
All tensors are flat Python lists / 1-D numpy arrays in row-major order.
"""
from __future__ import annotations

import math

import numpy as np


# ---- host helpers: runtime/src/utils/mod.rs ---------------------------------------------------
def compute_stride(shape):
    """utils/mod.rs:40-53: dense row-major strides."""
    stride = [0] * len(shape)
    acc = 1
    for i in range(len(shape) - 1, -1, -1):
        stride[i] = acc
        acc *= shape[i]
    return stride


def compute_broadcast_output_shape(a, b):
    """utils/mod.rs:114-143: right-aligned, missing dims are 1; None when incompatible."""
    n = max(len(a), len(b))
    out = []
    for i in range(n):
        ia = i - (n - len(a))
        ib = i - (n - len(b))
        da = a[ia] if ia >= 0 else 1
        db = b[ib] if ib >= 0 else 1
        if da != db and da != 1 and db != 1:
            return None
        out.append(max(da, db))
    return out


def compute_broadcast_stride(shape, out_shape):
    """utils/mod.rs:56-112: the operand's dense stride on dims it spans, 0 on broadcast dims."""
    dense = compute_stride(shape)
    n = len(out_shape)
    out = [0] * n
    for i in range(n):
        j = i - (n - len(shape))
        if j >= 0 and shape[j] == out_shape[i] and shape[j] != 1:
            out[i] = dense[j]
    return out


def _unravel(i, dims):
    """Last-dim-fastest decomposition used by every reference kernel (`% dims[d]`, `/= dims[d]`)."""
    idx = [0] * len(dims)
    for d in range(len(dims) - 1, -1, -1):
        idx[d] = i % dims[d]
        i //= dims[d]
    return idx


# ---- device kernels ---------------------------------------------------------------------------
def binary_loop(fn, dims, a_strides, b_strides, a, b):
    """cuda/src/ptx/headers/binary_op_macros.cuh:14-42."""
    n = math.prod(dims)
    out = []
    for i in range(n):
        idx = _unravel(i, dims)
        ai = sum(x * s for x, s in zip(idx, a_strides))
        bi = sum(x * s for x, s in zip(idx, b_strides))
        out.append(fn(a[ai], b[bi]))
    return out


def ternary_loop(dims, x_strides, y_strides, z_strides, x, y, z):
    """cuda/src/ptx/headers/ternary_op_macro.cuh:1-34 with where.cu's `z ? x : y`."""
    n = math.prod(dims)
    out = []
    for i in range(n):
        idx = _unravel(i, dims)
        xi = sum(a * s for a, s in zip(idx, x_strides))
        yi = sum(a * s for a, s in zip(idx, y_strides))
        zi = sum(a * s for a, s in zip(idx, z_strides))
        out.append(x[xi] if z[zi] else y[yi])
    return out


def reduce_mean_loop(shape, axes, data):
    """cuda/src/ptx/headers/aggregation_op_macros.cuh:1-49: one output element at a time, a
    double accumulator over the reduced coordinates, divided by the reduced count."""
    rank = len(shape)
    strides = compute_stride(shape)
    reduced = [d in axes for d in range(rank)]
    kept_dims = [shape[d] for d in range(rank) if not reduced[d]]
    red_dims = [shape[d] for d in range(rank) if reduced[d]]
    n_out = math.prod(kept_dims)
    n_red = math.prod(red_dims)
    out = []
    for o in range(n_out):
        kept_idx = _unravel(o, kept_dims)
        acc = 0.0
        for k in range(n_red):
            red_idx = _unravel(k, red_dims)
            coord = []
            ki = ri = 0
            for d in range(rank):
                if reduced[d]:
                    coord.append(red_idx[ri])
                    ri += 1
                else:
                    coord.append(kept_idx[ki])
                    ki += 1
            acc += float(data[sum(c * s for c, s in zip(coord, strides))])
        out.append(acc / float(n_red))
    return out


def expand_loop(in_shape, out_shape, data):
    """cuda/src/ptx/headers/expand_op_macros.cuh:1-31."""
    in_strides = compute_stride(in_shape)
    shift = len(out_shape) - len(in_shape)
    out = []
    for i in range(math.prod(out_shape)):
        idx = _unravel(i, out_shape)
        off = 0
        for d in range(len(out_shape)):
            j = d - shift
            if j >= 0 and in_shape[j] != 1:
                off += idx[d] * in_strides[j]
        out.append(data[off])
    return out


def transpose_loop(in_shape, perm, data):
    """cuda/src/ptx/headers/transpose_op_macros.cuh:1-25."""
    in_strides = compute_stride(in_shape)
    out_shape = [in_shape[p] for p in perm]
    out = []
    for i in range(math.prod(out_shape)):
        idx = _unravel(i, out_shape)
        out.append(data[sum(idx[d] * in_strides[perm[d]] for d in range(len(perm)))])
    return out


def slice_loop(in_shape, starts, ends, axes, steps, data):
    """cuda/src/ptx/headers/slice_op_macros.cuh:1-97: per-axis clamp, then
    in_idx = step * out_idx + start. Output shape from backend/slice.rs:357-463."""
    rank = len(in_shape)
    st = [0] * rank
    en = list(in_shape)
    sp = [1] * rank
    n_ax = len(axes) if axes is not None else len(starts)
    for k in range(n_ax):
        axis = k if axes is None else (axes[k] + rank if axes[k] < 0 else axes[k])
        if steps is not None:
            sp[axis] = steps[k]
        dim = in_shape[axis]
        s = starts[k]
        if s < 0:
            s += dim
        if s < 0:
            s = 0
        if sp[axis] >= 0 and s > dim:
            s = dim
        elif sp[axis] < 0 and s >= dim:
            s = dim - 1
        e = ends[k]
        if e < 0:
            e += dim
        if e < -1:
            e = -1
        if sp[axis] >= 0 and e > dim:
            e = dim
        elif sp[axis] < 0 and e >= dim:
            e = dim - 1
        st[axis], en[axis] = s, e
    out_shape = []
    for d in range(rank):
        if (sp[d] < 0 and st[d] < en[d]) or (sp[d] > 0 and st[d] >= en[d]):
            out_shape.append(0)
        elif sp[d] > 0:
            out_shape.append(-(-(en[d] - st[d]) // sp[d]))
        else:
            out_shape.append(-(-(st[d] - en[d]) // -sp[d]))
    in_strides = compute_stride(in_shape)
    out = []
    for i in range(math.prod(out_shape)):
        idx = _unravel(i, out_shape)
        out.append(data[sum((sp[d] * idx[d] + st[d]) * in_strides[d] for d in range(rank))])
    return out_shape, out


def scatter_nd_loop(data_shape, idx_shape, indices, updates, data, reduction="none"):
    """cuda/src/ptx/headers/scatter_op_macros.cuh:19-93; returns (output, error_code)."""
    out = list(data)
    t = idx_shape[-1] if len(idx_shape) > 1 else 1
    n_tuples = math.prod(idx_shape[:-1]) if len(idx_shape) > 1 else 1
    data_strides = compute_stride(data_shape)
    slice_len = math.prod(data_shape[t:])
    for n in range(n_tuples):
        off = 0
        for i in range(t):
            ix = int(indices[n * t + i])
            dim = data_shape[i]
            if ix < 0:
                ix += dim
            if ix < 0 or ix >= dim:
                return out, 1
            off += ix * data_strides[i]
        for i in range(slice_len):
            if off + i >= len(out):
                return out, 2
            u = updates[n * slice_len + i]
            cur = out[off + i]
            if reduction == "none":
                out[off + i] = u
            elif reduction == "add":
                out[off + i] = u + cur
            elif reduction == "mul":
                out[off + i] = u * cur
            elif reduction == "max":
                out[off + i] = u if u > cur else cur
            else:
                out[off + i] = u if u < cur else cur
    return out, 0


def trilu_loop(batch, rows, cols, upper, k, data):
    """cuda/src/ptx/headers/trilu_op_macros.cuh:1-43 over a zero-initialised output."""
    out = [type(data[0])(0)] * (batch * rows * cols) if len(data) else []
    for i in range(batch * rows * cols):
        col = i % cols
        row = (i // cols) % rows
        if upper:
            start, end = max(k + row, 0), cols
        else:
            start, end = 0, min(k + row + 1, cols)
        if start <= col < end:
            out[i] = data[i]
    return out


def gather_loop(shape, axis, indices, data):
    """runtime/src/providers/cuda/backend/gather.rs:199-258: per outer batch, per index, copy a
    run of prod(shape[axis+1:]) elements."""
    strides = compute_stride(shape)
    outer = math.prod(shape[:axis])
    run = math.prod(shape[axis + 1:])
    outer_stride = strides[axis] * shape[axis]
    out = []
    for b in range(outer):
        for ix in indices:
            ix = int(ix)
            if ix < 0:
                ix += shape[axis]
            start = b * outer_stride + ix * strides[axis]
            out.extend(data[start:start + run])
    return out


def concat_loop(shapes, axis, datas):
    """runtime/src/providers/cuda/backend/concat.rs:28-76."""
    outer = math.prod(shapes[0][:axis])
    step = math.prod(shapes[0][axis + 1:])
    out_axis = sum(s[axis] for s in shapes)
    out = [None] * (outer * out_axis * step)
    axis_off = 0
    for shape, data in zip(shapes, datas):
        dim = shape[axis]
        for o in range(outer):
            for j in range(dim):
                dst = o * out_axis * step + (axis_off + j) * step
                src = o * dim * step + j * step
                out[dst:dst + step] = data[src:src + step]
        axis_off += dim
    return out


def matmul_loop(a, b, m, k, n):
    """Triple loop in double: the definition cuBLAS is asked for
    (cuda/src/kernels/gemm.rs:191-232: C = A . B, alpha 1, beta 0)."""
    out = np.zeros((m, n), dtype=np.float64)
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for p in range(k):
                acc += float(a[i * k + p]) * float(b[p * n + j])
            out[i, j] = acc
    return out


def softmax_loop(rows, cols, data):
    """Row softmax in double, max-subtracted."""
    out = []
    for r in range(rows):
        row = [float(v) for v in data[r * cols:(r + 1) * cols]]
        m = max(row)
        e = [math.exp(v - m) if not (math.isinf(v) and v < 0 and math.isinf(m)) else float("nan")
             for v in row]
        s = sum(e)
        out.extend(v / s for v in e)
    return out
