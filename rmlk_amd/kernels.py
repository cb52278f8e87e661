"""Kernel-level wrappers over the C ABI: the Python mirror of the reference's kernel crate
(`rmlk_cuda::kernels::<op>::compute`, cuda/src/kernels/mod.rs:1-29).

Like the reference's wrappers, the caller owns every buffer: inputs and the pre-allocated output
are torch tensors on the GPU (torch is only the owner of device memory and of the stream here);
shape and stride vectors are host lists. Contract violations raise `AssertionError` (the
reference's wrappers `assert!`), launch failures raise `RmlkError`.
"""
from __future__ import annotations

import ctypes

import torch

from ._lib import Dims, RmlkError, check, lib

# ONNX TensorProto.DataType numbers (include/rmlk_hip.h rmlk_dtype)
FLOAT, UINT8, INT8, UINT16, INT16, INT32, INT64, BOOL, FLOAT16, DOUBLE, UINT32, UINT64 = (
    1, 2, 3, 4, 5, 6, 7, 9, 10, 11, 12, 13)
BFLOAT16 = 16   # only as the storage type of constant weights

TORCH_TO_DTYPE = {
    torch.float32: FLOAT, torch.uint8: UINT8, torch.int8: INT8, torch.int16: INT16,
    torch.int32: INT32, torch.int64: INT64, torch.bool: BOOL, torch.float16: FLOAT16,
    torch.float64: DOUBLE, torch.uint16: UINT16, torch.uint32: UINT32, torch.uint64: UINT64,
}
DTYPE_TO_TORCH = {v: k for k, v in TORCH_TO_DTYPE.items()}

ADD, SUB, MUL, DIV, POW, EQUAL, GREATER = range(7)
SQRT, NEG, SIN, COS, SIGMOID = range(5)
SCATTER_NONE, SCATTER_ADD, SCATTER_MUL, SCATTER_MAX, SCATTER_MIN = range(5)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t) -> int:
    if t is None:
        return 0
    assert t.is_cuda and t.is_contiguous(), "device tensors must be dense"
    return t.data_ptr()


def dtype_of(t: torch.Tensor) -> int:
    return TORCH_TO_DTYPE[t.dtype]


def storage_of(w: torch.Tensor) -> int:
    """Storage type of a weight matrix handed to the products over constant weights."""
    return BFLOAT16 if w.dtype == torch.bfloat16 else TORCH_TO_DTYPE[w.dtype]


def store_weights(w: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float tensor w rounded (to nearest even) to torch.float16 or torch.bfloat16 on the device."""
    out = torch.empty(w.shape, dtype=dtype, device=w.device)
    wd = BFLOAT16 if dtype == torch.bfloat16 else TORCH_TO_DTYPE[dtype]
    check(lib().rmlk_hip_store_weights(_stream(), wd, w.numel(), _ptr(w), _ptr(out)), "rmlk_hip_store_weights")
    return out


def weights_fit(w: torch.Tensor, dtype: torch.dtype) -> bool:
    """True when every value of the float tensor w survives storage as torch.float16 / torch.bfloat16."""
    flag = torch.ones(1, dtype=torch.int32, device=w.device)
    wd = BFLOAT16 if dtype == torch.bfloat16 else TORCH_TO_DTYPE[dtype]
    check(lib().rmlk_hip_weights_fit(_stream(), wd, w.numel(), _ptr(w), _ptr(flag)), "rmlk_hip_weights_fit")
    return bool(flag.item())


def binary(op: int, a, b, out, out_shape, a_stride, b_stride) -> None:
    """ref: cuda/src/kernels/binary.rs:58-100 (compute_with_types). Strides are per output dim,
    0 on broadcast dims."""
    assert len(out_shape) == len(a_stride) == len(b_stride)
    n = 1
    for d in out_shape:
        n *= d
    assert out.numel() == n, "output length must equal the product of the output shape"
    st = lib().rmlk_hip_binary(_stream(), op, dtype_of(a), dtype_of(b), Dims.of(out_shape),
                               Dims.of(a_stride), Dims.of(b_stride), _ptr(a), _ptr(b), _ptr(out))
    check(st, "rmlk_hip_binary")


def where(x, y, cond, out, out_shape, x_stride, y_stride, cond_stride) -> None:
    """ref: cuda/src/kernels/whereop.rs:57-101 (kernel operand order x, y, cond)."""
    assert cond.dtype == torch.bool or cond.dtype == torch.uint8
    st = lib().rmlk_hip_where(_stream(), dtype_of(x), Dims.of(out_shape), Dims.of(x_stride),
                              Dims.of(y_stride), Dims.of(cond_stride), _ptr(x), _ptr(y),
                              _ptr(cond), _ptr(out))
    check(st, "rmlk_hip_where")


def unary(op: int, x, out) -> None:
    """ref: cuda/src/kernels/unary.rs:10-42."""
    assert x.numel() == out.numel(), "input and output lengths must match"
    check(lib().rmlk_hip_unary(_stream(), op, dtype_of(x), x.numel(), _ptr(x), _ptr(out)),
          "rmlk_hip_unary")


def cast(x, out) -> None:
    """ref: cuda/src/kernels/unary.rs:47-80 (explicit_io_types_compute)."""
    assert x.numel() == out.numel()
    check(lib().rmlk_hip_cast(_stream(), dtype_of(x), dtype_of(out), x.numel(), _ptr(x),
                              _ptr(out)), "rmlk_hip_cast")


def reduce_mean(x, out, in_shape, axes) -> None:
    """ref: cuda/src/kernels/reduce_mean.rs:40-93."""
    arr = (ctypes.c_int64 * len(axes))(*[int(a) for a in axes])
    check(lib().rmlk_hip_reduce_mean(_stream(), dtype_of(x), Dims.of(in_shape), arr, len(axes),
                                     _ptr(x), _ptr(out)), "rmlk_hip_reduce_mean")


def softmax(x, out, outer: int, axis_len: int, inner: int = 1) -> None:
    """ref: cuda/src/kernels/softmax.rs:5-37."""
    assert x.numel() == out.numel() == outer * axis_len * inner
    check(lib().rmlk_hip_softmax(_stream(), dtype_of(x), outer, axis_len, inner, _ptr(x),
                                 _ptr(out)), "rmlk_hip_softmax")


def matmul_workspace_size(batch: int, m: int, n: int, k: int, dtype: int = FLOAT) -> int:
    return int(lib().rmlk_hip_matmul_workspace_size(dtype, batch, m, n, k))


def matmul_describe(batch: int, m: int, n: int, k: int, dtype: int = FLOAT) -> str:
    buf = ctypes.create_string_buffer(64)
    lib().rmlk_hip_matmul_describe(dtype, batch, m, n, k, buf, 64)
    return buf.value.decode()


def matmul(a, b, c, batch, m, n, k, lda, ldb, ldc, stride_a, stride_b, stride_c, trans_a=False,
           trans_b=False, workspace=None) -> None:
    """ref: cuda/src/kernels/gemm.rs:112-136 (compute with a StridedBatchedConfig)."""
    need = matmul_workspace_size(batch, m, n, k, dtype_of(a))
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=a.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    st = lib().rmlk_hip_matmul(_stream(), dtype_of(a), batch, m, n, k, _ptr(a), lda, stride_a,
                               int(trans_a), _ptr(b), ldb, stride_b, int(trans_b), _ptr(c), ldc,
                               stride_c, _ptr(workspace), ws_bytes)
    check(st, "rmlk_hip_matmul")


def matmul_noalloc(a, b, c, batch, m, n, k, lda, ldb, ldc, stride_a, stride_b, stride_c, trans_a=False,
                   trans_b=False) -> None:
    """rmlk_hip_matmul with the split-K partials in the library's fixed device array: the call
    allocates nothing (no counterpart in the reference; for callers that cannot allocate)."""
    st = lib().rmlk_hip_matmul_noalloc(_stream(), dtype_of(a), batch, m, n, k, _ptr(a), lda, stride_a,
                                       int(trans_a), _ptr(b), ldb, stride_b, int(trans_b), _ptr(c), ldc,
                                       stride_c)
    check(st, "rmlk_hip_matmul_noalloc")


def transpose(x, out, in_shape, perm) -> None:
    """ref: cuda/src/kernels/transpose.rs:38-80."""
    assert len(perm) == len(in_shape), "perm.len() must match rank"
    arr = (ctypes.c_int64 * len(perm))(*[int(p) for p in perm])
    check(lib().rmlk_hip_transpose(_stream(), dtype_of(x), Dims.of(in_shape), arr, _ptr(x),
                                   _ptr(out)), "rmlk_hip_transpose")


def expand(x, out, in_shape, out_shape) -> None:
    """ref: cuda/src/kernels/expand.rs:35-76."""
    check(lib().rmlk_hip_expand(_stream(), dtype_of(x), Dims.of(in_shape), Dims.of(out_shape),
                                _ptr(x), _ptr(out)), "rmlk_hip_expand")


def slice_(x, out, in_shape, starts, steps, out_shape) -> None:
    """ref: cuda/src/kernels/slice.rs:61-122, with starts / steps already resolved per dim."""
    check(lib().rmlk_hip_slice(_stream(), dtype_of(x), Dims.of(in_shape), Dims.of(starts),
                               Dims.of(steps), Dims.of(out_shape), _ptr(x), _ptr(out)),
          "rmlk_hip_slice")


def concat_into(x, out, in_shape, out_shape, axis: int, axis_offset: int) -> None:
    """ref: runtime/src/providers/cuda/backend/concat.rs:28-76 (one input)."""
    check(lib().rmlk_hip_concat(_stream(), dtype_of(x), Dims.of(in_shape), Dims.of(out_shape),
                                axis, axis_offset, _ptr(x), _ptr(out)), "rmlk_hip_concat")


def concat(xs, out, in_shapes, out_shape, axis: int) -> None:
    """All inputs of a Concat in one call. ref: runtime/src/providers/cuda/backend/concat.rs:28-76."""
    assert len(xs) == len(in_shapes) and len(xs) >= 1
    shapes = (Dims * len(xs))(*[Dims.of(s) for s in in_shapes])
    ptrs = (ctypes.c_void_p * len(xs))(*[_ptr(x) if x.numel() else 0 for x in xs])
    check(lib().rmlk_hip_concat_many(_stream(), dtype_of(out), len(xs), shapes, ptrs, Dims.of(out_shape),
                                     axis, _ptr(out)), "rmlk_hip_concat_many")


def gather(data, idx, out, data_shape, axis: int, err_flag=None) -> None:
    """ref: runtime/src/providers/cuda/backend/gather.rs:199-258."""
    check(lib().rmlk_hip_gather(_stream(), dtype_of(data), dtype_of(idx), Dims.of(data_shape),
                                axis, idx.numel(), _ptr(data), _ptr(idx), _ptr(out),
                                _ptr(err_flag)), "rmlk_hip_gather")


def scatter_nd(idx, updates, out, data_shape, n_tuples: int, tuple_size: int,
               reduction: int = SCATTER_NONE, err_flag=None) -> None:
    """ref: cuda/src/kernels/scatter_nd.rs:91-210. `out` already holds the data."""
    assert idx.dtype == torch.int64
    check(lib().rmlk_hip_scatter_nd(_stream(), reduction, dtype_of(out), Dims.of(data_shape),
                                    n_tuples, tuple_size, _ptr(idx), _ptr(updates), _ptr(out),
                                    _ptr(err_flag)), "rmlk_hip_scatter_nd")


def scatter_nd_copy(idx, updates, data, out, data_shape, n_tuples: int, tuple_size: int,
                    err_flag=None) -> None:
    """ScatterND (reduction none) with its copy of `data` in one pass.
    ref: runtime/src/providers/cuda/backend/scatter_nd.rs:128-129 + cuda/src/kernels/scatter_nd.rs:91-210."""
    assert idx.dtype == torch.int64 and data.dtype == out.dtype
    check(lib().rmlk_hip_scatter_nd_copy(_stream(), dtype_of(out), Dims.of(data_shape), n_tuples,
                                         tuple_size, _ptr(idx), _ptr(updates), _ptr(data), _ptr(out),
                                         _ptr(err_flag)), "rmlk_hip_scatter_nd_copy")


def trilu(x, out, batch: int, rows: int, cols: int, upper: bool, k: int) -> None:
    """ref: cuda/src/kernels/trilu.rs:36-78."""
    assert x.numel() == out.numel() == batch * rows * cols
    check(lib().rmlk_hip_trilu(_stream(), dtype_of(x), batch, rows, cols, int(upper), k, _ptr(x),
                               _ptr(out)), "rmlk_hip_trilu")


def rmsnorm(x, gamma, out, rows: int, cols: int, eps: float, reciprocal_form: bool = False) -> None:
    """Fused Pow(2) -> ReduceMean(-1) -> Add(eps) -> Sqrt -> Div -> Mul(gamma)."""
    assert x.numel() == out.numel() == rows * cols and gamma.numel() == cols
    check(lib().rmlk_hip_rmsnorm(_stream(), dtype_of(x), rows, cols, _ptr(x), _ptr(gamma),
                                 float(eps), int(reciprocal_form), _ptr(out)), "rmlk_hip_rmsnorm")


def add_rmsnorm(a, b, gamma, sum_out, out, rows: int, cols: int, eps: float,
                reciprocal_form: bool = False) -> None:
    """Fused Add -> RMSNorm chain: sum_out = a + b, out = RMSNorm(sum_out)."""
    assert a.numel() == b.numel() == sum_out.numel() == out.numel() == rows * cols
    check(lib().rmlk_hip_add_rmsnorm(_stream(), dtype_of(a), rows, cols, _ptr(a), _ptr(b),
                                     _ptr(gamma), float(eps), int(reciprocal_form), _ptr(sum_out),
                                     _ptr(out)), "rmlk_hip_add_rmsnorm")


def scale_mask_softmax(x, mask, out, shape, mask_stride, scale: float, scale_is_mul=False) -> None:
    """Fused Div|Mul(x, scale) -> Add(mask) -> Softmax(axis -1)."""
    check(lib().rmlk_hip_scale_mask_softmax(_stream(), dtype_of(x), Dims.of(shape),
                                            Dims.of(mask_stride), int(scale_is_mul), float(scale),
                                            _ptr(x), _ptr(mask), _ptr(out)),
          "rmlk_hip_scale_mask_softmax")


def swiglu(gate, up, out) -> None:
    """Fused Sigmoid -> Mul -> Mul: (gate * sigmoid(gate)) * up."""
    assert gate.numel() == up.numel() == out.numel()
    check(lib().rmlk_hip_swiglu(_stream(), dtype_of(gate), gate.numel(), _ptr(gate), _ptr(up),
                                _ptr(out)), "rmlk_hip_swiglu")


def attention(q, k, v, mask, out, batch: int, kv_heads: int, rep: int, q_len: int, kv_len: int,
              head_dim: int, mask_stride, scale: float, scale_is_mul: bool = False,
              out_seq_major: bool = False) -> None:
    """Fused grouped-query attention: Softmax(q . k^T (*|/) scale + mask) . v in one kernel; out is
    [B, H, S, D], or [B, S, H, D] with out_seq_major."""
    check(lib().rmlk_hip_attention(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                   head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask),
                                   Dims.of(mask_stride), int(scale_is_mul), float(scale),
                                   int(out_seq_major), _ptr(out)),
          "rmlk_hip_attention")


def attention_skipping(q, k, v, mask, out, batch: int, kv_heads: int, rep: int, q_len: int, kv_len: int,
                       head_dim: int, mask_stride, scale: float, scale_is_mul: bool = False,
                       out_seq_major: bool = False, out_pieces=None) -> int:
    """`attention` with the workspace that lets it skip the key chunks a query tile cannot see; returns
    the workspace size the library asked for (0: skipping does not apply to this shape). out_pieces
    (with out_seq_major): the result also as the three bfloat16 pieces bf16x3_split would make of it."""
    ms = Dims.of(mask_stride)
    need = int(lib().rmlk_hip_attention_workspace_size(dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                                       head_dim, ms))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    if out_pieces is not None:
        assert out_seq_major
        check(lib().rmlk_hip_attention_ws_pieces(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                                 head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask), ms,
                                                 int(scale_is_mul), float(scale), _ptr(ws) if need else None, need,
                                                 _ptr(out), _ptr(out_pieces)), "rmlk_hip_attention_ws_pieces")
        return need
    check(lib().rmlk_hip_attention_ws(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                      head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask), ms,
                                      int(scale_is_mul), float(scale), int(out_seq_major),
                                      _ptr(ws) if need else None, need, _ptr(out)),
          "rmlk_hip_attention_ws")
    return need


def attention_map(mask, batch: int, kv_heads: int, rep: int, q_len: int, kv_len: int, head_dim: int,
                  mask_stride):
    """The map of visible (query tile, key chunk) pairs of `mask`, made once for several launches of
    `attention_mapped` over that mask; None where skipping does not apply to the shape."""
    ms = Dims.of(mask_stride)
    need = int(lib().rmlk_hip_attention_map_size(dtype_of(mask), batch, kv_heads, rep, q_len, kv_len, head_dim, ms))
    if need == 0:
        return None
    m = torch.empty(need, dtype=torch.uint8, device=mask.device)
    check(lib().rmlk_hip_attention_map(_stream(), dtype_of(mask), batch, kv_heads, rep, q_len, kv_len, head_dim,
                                       _ptr(mask), ms, _ptr(m), need), "rmlk_hip_attention_map")
    return m


def attention_mapped(q, k, v, mask, out, tile_map, batch: int, kv_heads: int, rep: int, q_len: int, kv_len: int,
                     head_dim: int, mask_stride, scale: float, scale_is_mul: bool = False,
                     out_seq_major: bool = False, out_pieces=None) -> None:
    """`attention_skipping` over a map that `attention_map` made for this mask and these sizes."""
    if out_pieces is not None:
        assert out_seq_major
        check(lib().rmlk_hip_attention_mapped_pieces(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                                     head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask),
                                                     Dims.of(mask_stride), int(scale_is_mul), float(scale),
                                                     _ptr(tile_map), tile_map.numel(), _ptr(out), _ptr(out_pieces)),
              "rmlk_hip_attention_mapped_pieces")
        return
    check(lib().rmlk_hip_attention_mapped(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len, head_dim,
                                          _ptr(q), _ptr(k), _ptr(v), _ptr(mask), Dims.of(mask_stride),
                                          int(scale_is_mul), float(scale), int(out_seq_major), _ptr(tile_map),
                                          tile_map.numel(), _ptr(out)), "rmlk_hip_attention_mapped")


def attention_few_rows(q, k, v, mask, out, batch: int, kv_heads: int, rep: int, q_len: int, kv_len: int,
                       head_dim: int, mask_stride, scale: float, scale_is_mul: bool = False,
                       out_seq_major: bool = False) -> None:
    """The attention of a decode step (rep * q_len <= 16 query rows per KV head): keys split over blocks."""
    need = int(lib().rmlk_hip_attention_few_rows_workspace_size(dtype_of(q), batch, kv_heads, rep, q_len,
                                                                kv_len, head_dim))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    check(lib().rmlk_hip_attention_few_rows(_stream(), dtype_of(q), batch, kv_heads, rep, q_len, kv_len,
                                            head_dim, _ptr(q), _ptr(k), _ptr(v), _ptr(mask),
                                            Dims.of(mask_stride), int(scale_is_mul), float(scale),
                                            int(out_seq_major), _ptr(ws), need, _ptr(out)),
          "rmlk_hip_attention_few_rows")


def attention_few_rows_one_launch(q, k, v, mask, out, counters, batch: int, kv_heads: int, rep: int,
                                  q_len: int, kv_len: int, head_dim: int, mask_stride, scale: float,
                                  scale_is_mul: bool = False, out_seq_major: bool = False) -> None:
    """`attention_few_rows` without the merge launch; `counters`: batch * kv_heads int32, zero before the
    first call and zero again after every call."""
    need = int(lib().rmlk_hip_attention_few_rows_workspace_size(dtype_of(q), batch, kv_heads, rep, q_len,
                                                                kv_len, head_dim))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    check(lib().rmlk_hip_attention_few_rows_one_launch(_stream(), dtype_of(q), batch, kv_heads, rep, q_len,
                                                       kv_len, head_dim, _ptr(q), _ptr(k), _ptr(v),
                                                       _ptr(mask), Dims.of(mask_stride), int(scale_is_mul),
                                                       float(scale), int(out_seq_major), _ptr(ws), need,
                                                       _ptr(counters), _ptr(out)),
          "rmlk_hip_attention_few_rows_one_launch")


def gemv_kmajor(x, wt, y, n: int, k: int) -> None:
    """y[n] = sum_k x[k] * wt[n][k]: one-row product with K-contiguous weights, no combine launch."""
    check(lib().rmlk_hip_gemv_kmajor(_stream(), dtype_of(x), n, k, _ptr(x), storage_of(wt), _ptr(wt), k, _ptr(y)),
          "rmlk_hip_gemv_kmajor")


def gemv_kmajor_swiglu(x, wt, y, n: int, k: int, gate_row: int, up_row: int) -> None:
    """y[i] = swiglu(x . wt[gate_row + i], x . wt[up_row + i]) in one launch (K-contiguous weights)."""
    check(lib().rmlk_hip_gemv_kmajor_swiglu(_stream(), dtype_of(x), n, k, _ptr(x), storage_of(wt), _ptr(wt), k,
                                            gate_row, up_row, _ptr(y)), "rmlk_hip_gemv_kmajor_swiglu")


def gemv_kmajor_add(x, wt, residual, y, n: int, k: int) -> None:
    """y = x . wt^T + residual (K-contiguous weights, one launch)."""
    check(lib().rmlk_hip_gemv_kmajor_add(_stream(), dtype_of(x), n, k, _ptr(x), storage_of(wt), _ptr(wt), k,
                                         _ptr(residual), _ptr(y)), "rmlk_hip_gemv_kmajor_add")


def gemv_kmajor_normed(x, gamma, wt, y, n: int, k: int, eps: float, reciprocal_form: bool = False) -> None:
    """y = (RMSNorm(x) * gamma) . wt^T, the normalised row never stored."""
    check(lib().rmlk_hip_gemv_kmajor_normed(_stream(), dtype_of(x), n, k, _ptr(x), _ptr(gamma), eps,
                                            int(reciprocal_form), storage_of(wt), _ptr(wt), k, _ptr(y)),
          "rmlk_hip_gemv_kmajor_normed")


def gemv_kmajor_swiglu_normed(x, gamma, wt, y, n: int, k: int, gate_row: int, up_row: int, eps: float,
                              reciprocal_form: bool = False) -> None:
    """gemv_kmajor_swiglu over RMSNorm(x) * gamma."""
    check(lib().rmlk_hip_gemv_kmajor_swiglu_normed(_stream(), dtype_of(x), n, k, _ptr(x), _ptr(gamma), eps,
                                                   int(reciprocal_form), storage_of(wt), _ptr(wt), k, gate_row,
                                                   up_row, _ptr(y)), "rmlk_hip_gemv_kmajor_swiglu_normed")


def matmul_grouped(a, b, outs, m: int, k: int, widths, workspace=None, trans_b: bool = False) -> None:
    """outs[i] = a[m, k] . (the next widths[i] columns of the joint matrix b: row-major [k, sum], or with
    trans_b K-contiguous [sum, k])."""
    n = len(widths)
    w = (ctypes.c_int64 * n)(*[int(x) for x in widths])
    need = int(lib().rmlk_hip_matmul_grouped_workspace_size(dtype_of(a), m, k, n, w))
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=a.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    ptrs = (ctypes.c_void_p * n)(*[_ptr(o) for o in outs])
    check(lib().rmlk_hip_matmul_grouped(_stream(), dtype_of(a), m, k, _ptr(a), k, storage_of(b), _ptr(b),
                                        k if trans_b else int(sum(widths)), int(trans_b), n, w, ptrs,
                                        _ptr(workspace), ws_bytes),
          "rmlk_hip_matmul_grouped")


def matmul_swiglu(a, b, out, m: int, n: int, k: int, ldb: int, gate_offset: int, up_offset: int,
                  trans_b: bool = False) -> None:
    """out[m, n] = swiglu(a . b[:, gate_offset:+n], a . b[:, up_offset:+n]) (trans_b: b is [., k] and the
    offsets count its rows); RmlkError with status RMLK_ERR_UNSUPPORTED (-2) for shapes the one-launch
    kernel does not cover."""
    check(lib().rmlk_hip_matmul_swiglu(_stream(), dtype_of(a), m, n, k, _ptr(a), k, storage_of(b), _ptr(b), ldb,
                                       int(trans_b), gate_offset, up_offset, _ptr(out), n),
          "rmlk_hip_matmul_swiglu")


def bf16x3_split(a: torch.Tensor) -> torch.Tensor:
    """The three bfloat16 pieces of the dense float matrix a [m, k] (a = hi + mid + lo exactly), as the
    planes [3][m rounded up to 128][k] that matmul_bf16x3 reads (an int16 tensor)."""
    m, k = a.shape
    pieces = torch.empty(lib().rmlk_hip_bf16x3_pieces_size(m, k) // 2, dtype=torch.int16, device=a.device)
    check(lib().rmlk_hip_bf16x3_split(_stream(), m, k, _ptr(a), k, _ptr(pieces)), "rmlk_hip_bf16x3_split")
    return pieces


def rmsnorm_pieces(x, gamma, eps: float, out, pieces, add=None, sum_out=None, splits: int = 1,
                   reciprocal_form: bool = False) -> None:
    """RMSNorm of the rows of x [rows, cols] (of x[0] + .. + x[splits-1] for x [splits, rows, cols]; plus
    `add`, the formed rows then also stored to sum_out) into out and, as three bfloat16 pieces, into
    `pieces` (the tensor bf16x3_split would return)."""
    rows, cols = out.shape
    check(lib().rmlk_hip_rmsnorm_pieces(_stream(), rows, cols, _ptr(x), splits, rows * cols,
                                        _ptr(add) if add is not None else None, _ptr(gamma), eps,
                                        int(reciprocal_form), _ptr(sum_out) if sum_out is not None else None,
                                        _ptr(out), _ptr(pieces)), "rmlk_hip_rmsnorm_pieces")


def bf16x3_splits(m: int, n: int, k: int) -> int:
    """Slabs of K with which matmul_bf16x3 fills the GPU for this size; 0: a size it does not take."""
    return int(lib().rmlk_hip_bf16x3_splits(m, n, k))


def matmul_bf16x3(pieces, wt, out, m: int, n: int, k: int, splits: int = 1) -> None:
    """out[m, n] (splits == 1) or out[splits, m, n] (one partial product per slab of K) = a . wt^T over
    the pieces of a (bf16x3_split) and bfloat16 weights wt [n, k], on the bf16 matrix cores."""
    assert wt.dtype == torch.bfloat16
    check(lib().rmlk_hip_matmul_bf16x3(_stream(), m, n, k, _ptr(pieces), _ptr(wt), k, splits, _ptr(out), n, m * n),
          "rmlk_hip_matmul_bf16x3")


def matmul_bf16x3_grouped(pieces, wt, outs, m: int, k: int, widths) -> None:
    """outs[i] [m, widths[i]] = a . (the next widths[i] rows of wt)^T over the pieces of a, one launch."""
    assert wt.dtype == torch.bfloat16 and len(outs) == len(widths)
    w = (ctypes.c_int64 * len(widths))(*widths)
    o = (ctypes.c_void_p * len(outs))(*[_ptr(t) for t in outs])
    check(lib().rmlk_hip_matmul_bf16x3_grouped(_stream(), m, k, _ptr(pieces), _ptr(wt), k, len(widths), w, o),
          "rmlk_hip_matmul_bf16x3_grouped")


def matmul_bf16x3_swiglu(pieces, wt, out, m: int, n: int, k: int, gate_row: int, up_row: int,
                         out_pieces=None) -> None:
    """out[m, n] = swiglu(a . wt[gate_row:+n]^T, a . wt[up_row:+n]^T) over the pieces of a; out_pieces:
    where the same launch also stores the pieces of out (the tensor bf16x3_split(out) would return)."""
    assert wt.dtype == torch.bfloat16
    check(lib().rmlk_hip_matmul_bf16x3_swiglu(_stream(), m, n, k, _ptr(pieces), _ptr(wt), k, gate_row, up_row,
                                              _ptr(out), n, _ptr(out_pieces) if out_pieces is not None else None),
          "rmlk_hip_matmul_bf16x3_swiglu")


def rotary(x, cos, sin, out, shape, x_stride, cos_stride, sin_stride) -> None:
    """Fused half-rotation rotary embedding over a strided [B,H,S,D] view of x."""
    check(lib().rmlk_hip_rotary(_stream(), dtype_of(x), Dims.of(shape), Dims.of(x_stride),
                                Dims.of(cos_stride), Dims.of(sin_stride), _ptr(x), _ptr(cos),
                                _ptr(sin), _ptr(out)), "rmlk_hip_rotary")


def head_rows(streams, err_flag=None) -> None:
    """Several streams of head rows in one launch. Each stream is a dict: x, shape [B,H,S,D],
    x_stride, out, and optionally cos, sin, cos_stride, sin_stride (rotate) and idx, data_shape
    (scatter the rows into `out` by index tuples)."""
    arr = _row_streams(streams)
    dt = dtype_of(streams[0]["x"]) if streams else 1
    check(lib().rmlk_hip_head_rows(_stream(), dt, len(streams), arr,
                                   _ptr(err_flag) if err_flag is not None else None),
          "rmlk_hip_head_rows")


def _row_streams(streams, with_x=True):
    from ._lib import RowStream
    arr = (RowStream * len(streams))()
    for st, d in zip(arr, streams):
        st.shape = Dims.of(d["shape"])
        if with_x:
            st.x_stride = Dims.of(d["x_stride"])
            st.x = _ptr(d["x"])
        if d.get("cos") is not None:
            st.cos, st.sin = _ptr(d["cos"]), _ptr(d["sin"])
            st.cos_stride, st.sin_stride = Dims.of(d["cos_stride"]), Dims.of(d["sin_stride"])
        st.out = _ptr(d["out"])
        if d.get("idx") is not None:
            st.idx = _ptr(d["idx"])
            st.data_shape = Dims.of(d["data_shape"])
            st.tuple_size = len(d["data_shape"]) - 1
        if d.get("partials"):
            st.partials, st.partial_stride = int(d["partials"]), int(d["partial_stride"])
    return arr


def gemv_kmajor_head_rows(x, wt, k: int, streams, first_cols, gamma=None, eps: float = 0.0,
                          reciprocal_form: bool = False, err_flag=None) -> None:
    """The q/k/v projection of one token (x . wt^T over K-contiguous weights, over RMSNorm(x) * gamma
    when gamma is given) with its result handed on as head rows (see head_rows; streams carry no x)
    in one launch. first_cols[i]: first product column of stream i."""
    arr = _row_streams(streams, with_x=False)
    cols = (ctypes.c_int64 * len(streams))(*[int(c) for c in first_cols])
    check(lib().rmlk_hip_gemv_kmajor_head_rows(_stream(), dtype_of(x), k, _ptr(x), _ptr(gamma), eps,
                                               int(reciprocal_form), storage_of(wt), _ptr(wt), k, len(streams),
                                               arr, cols,
                                               _ptr(err_flag) if err_flag is not None else None),
          "rmlk_hip_gemv_kmajor_head_rows")


def memcpy_dtod_many(dsts, srcs) -> None:
    """dsts[i] <- srcs[i] (dense device tensors of equal byte size each), 32 copies per launch."""
    n = len(dsts)
    d = (ctypes.c_void_p * n)(*[_ptr(t) for t in dsts])
    s_ = (ctypes.c_void_p * n)(*[_ptr(t) for t in srcs])
    b = (ctypes.c_size_t * n)(*[t.numel() * t.element_size() for t in srcs])
    check(lib().rmlk_hip_memcpy_dtod_many(_stream(), n, d, s_, b), "rmlk_hip_memcpy_dtod_many")


class collected_launches:
    """Context manager: operators over tiny tensors issued inside it on the current stream are
    collected and run as one launch (rmlk_hip_batch_begin / rmlk_hip_batch_end)."""

    def __enter__(self):
        self._stream = _stream()
        check(lib().rmlk_hip_batch_begin(self._stream), "rmlk_hip_batch_begin")
        return self

    def flush(self) -> None:
        check(lib().rmlk_hip_batch_flush(self._stream), "rmlk_hip_batch_flush")

    def __exit__(self, *exc):
        check(lib().rmlk_hip_batch_end(self._stream), "rmlk_hip_batch_end")
        return False


YARDSTICK_READ, YARDSTICK_COPY = 0, 1


def stream_yardstick(kind: int, src, dst, nbytes: int, stamps=None, stream=None) -> None:
    """The minimal streaming read (kind YARDSTICK_READ) or copy (YARDSTICK_COPY) of `nbytes`, for
    benchmarks; `stamps` (int64, 2 per block) receives each block's start and end on the 100 MHz
    clock. No counterpart in the reference."""
    st = lib().rmlk_hip_stream_yardstick(_stream() if stream is None else stream, kind, nbytes, _ptr(src),
                                         _ptr(dst), _ptr(stamps))
    check(st, "rmlk_hip_stream_yardstick")


def issue_yardstick(kind: int, second_wavefront: bool, iterations: int, cycles) -> None:
    """fp32 MFMAs with something between them in wavefronts 0..3 of every block (kind 0/4/8/12/16: a
    chain with that many independent v_fma_f32 behind each MFMA; 100..103: independent MFMAs with
    nothing / a v_add_u32 / a ds_read_b128 / both, the read waiting for the add, behind every fourth)
    and (second_wavefront) a chain of dependent v_fma_f32 in wavefronts 4..7 beside them; `cycles`
    (int64, 8 per block) receives every wavefront's shader clock cycles. For benchmarks; no
    counterpart in the reference."""
    blocks = cycles.numel() // 8
    st = lib().rmlk_hip_issue_yardstick(_stream(), int(kind), int(bool(second_wavefront)), int(iterations),
                                        blocks, _ptr(cycles))
    check(st, "rmlk_hip_issue_yardstick")


def device_info(device: int = 0) -> dict:
    from ._lib import DeviceInfo
    info = DeviceInfo()
    check(lib().rmlk_hip_device_info(device, ctypes.byref(info)), "rmlk_hip_device_info")
    return {"name": info.name.decode(), "arch": info.arch.decode(),
            "compute_units": info.compute_units, "wavefront_size": info.wavefront_size,
            "lds_bytes_per_block": info.lds_bytes_per_block, "clock_khz": info.clock_khz,
            "total_mem_bytes": info.total_mem_bytes}


__all__ = [n for n in dir() if not n.startswith("_")] + ["RmlkError"]
