/*
 * rmlk_hip.h -- C ABI of librmlk_hip, the gfx950 (MI355X / CDNA4) kernel library that stands where
 * the reference's `rmlk-cuda` kernel crate stands: below the runtime's operator dispatch.
 *
 * Each entry point names the reference interface it replaces as `ref: file:line` (paths relative
 * to the reference repository root).
 *
 * Conventions (all entry points):
 *   - Returns an int32 status: 0 = ok; > 0 = a hipError_t raised by the launch; < 0 = an argument
 *     error from `rmlk_status`.
 *   - Every pointer named `a`, `b`, `in`, `out`, `data`, ... is DEVICE memory owned by the caller.
 *     `rmlk_dims` / attribute arrays are HOST memory, read before the call returns.
 *   - Work is enqueued on `stream` (a hipStream_t; NULL = the default stream). No entry point
 *     synchronises, allocates device memory or keeps a reference to host arguments after it returns
 *     (the memory helpers at the end are the exception and say so).
 *   - Tensors are dense row-major unless a stride argument says otherwise. Strides are in ELEMENTS.
 *   - A call whose output has zero elements returns 0 without launching.
 *   - Thread safety: calls on distinct streams may be made from distinct threads. The library keeps
 *     three pieces of process-wide state, each safe under that rule: a per-device note that a
 *     kernel's dynamic LDS limit has been raised (written once); the list of open batches of
 *     rmlk_hip_batch_begin / _flush / _end, guarded by a mutex and keyed by stream (two threads must
 *     not drive ONE stream while it has a batch open); and the per-device address of the fixed
 *     32 MiB scratch array of rmlk_hip_matmul_noalloc, looked up once per device — calls of THAT
 *     entry point which overlap in time on one GPU share the array and race, whatever their streams.
 */
#ifndef RMLK_HIP_H
#define RMLK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RMLK_MAX_RANK 8 /* ref: cuda/src/kernels/slice.rs:88 (rank <= 8) */

typedef void *rmlk_stream_t; /* hipStream_t */

typedef enum rmlk_status {
    RMLK_OK = 0,
    RMLK_ERR_BAD_RANK = -1,        /* rank outside 1..RMLK_MAX_RANK */
    RMLK_ERR_UNSUPPORTED = -2,     /* dtype / op combination has no kernel ("unsupported data type") */
    RMLK_ERR_NULL_POINTER = -3,    /* null pointer with a non-zero length */
    RMLK_ERR_SIZE_MISMATCH = -4,   /* shapes / lengths disagree */
    RMLK_ERR_INVALID_ARGUMENT = -5,/* bad axis, perm, step 0, negative dim ... */
    RMLK_ERR_WORKSPACE = -6,       /* workspace smaller than rmlk_hip_matmul_workspace_size says */
    RMLK_ERR_TOO_LARGE = -7,       /* more elements than the kernels index (>= 2^62) */
    RMLK_ERR_SCRATCH_LIMIT = -8    /* rmlk_hip_matmul_noalloc: the problem needs more scratch than the
                                      library's fixed array holds */
} rmlk_status;

/* Element types. Values are the ONNX TensorProto.DataType numbers the reference maps its
 * `schema::DataType` to (ref: schema/src/tensor.rs:404-430). */
typedef enum rmlk_dtype {
    RMLK_FLOAT = 1,
    RMLK_UINT8 = 2,
    RMLK_INT8 = 3,
    RMLK_UINT16 = 4,
    RMLK_INT16 = 5,
    RMLK_INT32 = 6,
    RMLK_INT64 = 7,
    RMLK_BOOL = 9, /* one byte, 0 or 1 on output; any non-zero byte is true on input */
    RMLK_FLOAT16 = 10,
    RMLK_DOUBLE = 11,
    RMLK_UINT32 = 12,
    RMLK_UINT64 = 13,
    RMLK_BFLOAT16 = 16 /* only as the storage type of constant weights (w_dtype below) */
} rmlk_dtype;

/* Shape or stride vector passed by value from the host; replaces the device `info` buffers the
 * reference uploads per call (ref: runtime/src/providers/cuda/backend/binary.rs:114-131). */
typedef struct rmlk_dims {
    int32_t rank;
    int64_t v[RMLK_MAX_RANK];
} rmlk_dims;

/* ---------------------------------------------------------------------------------------------
 * Broadcast binary ops.
 * ref: cuda/src/kernels/binary.rs:27-100 (compute / compute_with_diff_output / compute_with_types)
 *      cuda/src/ptx/headers/binary_op_macros.cuh:14-42, ptx/{add,sub,mul,div,pow,equal,greater}.cu
 * out[i] = a[ia] (op) b[ib]; `out_shape` is the broadcast shape, `a_stride` / `b_stride` hold the
 * operand's element stride per output dim with 0 on broadcast dims (the meaning of the reference's
 * info buffer, ref: runtime/src/utils/mod.rs:56-91). `out` is dense.
 *   ADD SUB MUL DIV : dtype_a == dtype_b in {FLOAT, DOUBLE, INT32, INT64}; out dtype = dtype_a.
 *                     Integer DIV truncates toward zero; x/0 yields 0 for integers (never traps).
 *   POW             : dtype_a (base) in {FLOAT, DOUBLE, INT32, INT64}, dtype_b (exponent) in
 *                     {FLOAT, DOUBLE, INT32, INT64}; out dtype = dtype_a. Float bases with exponent
 *                     2, 3, 0.5 use x*x, x*x*x, sqrt(x); integer bases round llround(pow(double)).
 *   EQUAL GREATER   : dtype_a == dtype_b in {FLOAT, DOUBLE, INT32, INT64}; out dtype = BOOL (0/1).
 */
typedef enum rmlk_binary_op {
    RMLK_ADD = 0,
    RMLK_SUB = 1,
    RMLK_MUL = 2,
    RMLK_DIV = 3,
    RMLK_POW = 4,
    RMLK_EQUAL = 5,
    RMLK_GREATER = 6
} rmlk_binary_op;

int32_t rmlk_hip_binary(rmlk_stream_t stream, int32_t op, int32_t dtype_a, int32_t dtype_b,
                        const rmlk_dims *out_shape, const rmlk_dims *a_stride,
                        const rmlk_dims *b_stride, const void *a, const void *b, void *out);

/* Where: out[i] = cond[ic] ? x[ix] : y[iy], three-way broadcast, pure move (NaN payloads kept).
 * ref: cuda/src/kernels/whereop.rs:57-101, cuda/src/ptx/headers/ternary_op_macro.cuh:1-34.
 * dtype (of x, y, out) in {FLOAT, DOUBLE, INT32, INT64, and any 1/2/4/8-byte type}; cond is BOOL. */
int32_t rmlk_hip_where(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *out_shape,
                       const rmlk_dims *x_stride, const rmlk_dims *y_stride,
                       const rmlk_dims *cond_stride, const void *x, const void *y,
                       const void *cond, void *out);

/* Contiguous unary maps.
 * ref: cuda/src/kernels/unary.rs:10-42, cuda/src/ptx/headers/unary_op_macro.cuh:1-11,
 *      ptx/{sqrt,neg,sin,cos}.cu; sigmoid replaces cuDNN (cuda/src/kernels/sigmoid.rs:7-29).
 * SQRT SIN COS SIGMOID: FLOAT, DOUBLE. NEG: FLOAT, DOUBLE, INT32, INT64 (sign flip). */
typedef enum rmlk_unary_op {
    RMLK_SQRT = 0,
    RMLK_NEG = 1,
    RMLK_SIN = 2,
    RMLK_COS = 3,
    RMLK_SIGMOID = 4
} rmlk_unary_op;

int32_t rmlk_hip_unary(rmlk_stream_t stream, int32_t op, int32_t dtype, int64_t n, const void *in,
                       void *out);

/* Cast: C static_cast semantics (float -> int truncates toward zero, NaN gives 0, values out of
 * range saturate at the limits of the 32-bit type of the target's signedness — 64-bit for a 64-bit
 * target — and an 8- or 16-bit target keeps the low bits of that, as the reference's kernels do:
 * half 32768.0 -> INT16 is -32768, cuda/src/kernels/cast.rs:524-539; to BOOL is
 * x != 0; from BOOL is 0/1). Any pair over {FLOAT, DOUBLE, FLOAT16, INT8..INT64, UINT8..UINT64,
 * BOOL}. ref: cuda/src/kernels/unary.rs:47-80, cuda/src/ptx/cast.cu:6-124. */
int32_t rmlk_hip_cast(rmlk_stream_t stream, int32_t src_dtype, int32_t dst_dtype, int64_t n,
                      const void *in, void *out);

/* ReduceMean over `axes` (normalised, distinct, 0 <= axis < rank) of a dense tensor; `out` is dense
 * over the kept dims in order (keepdims only changes the shape the host records). Accumulates in
 * double like the reference. dtype in {FLOAT, DOUBLE}.
 * ref: cuda/src/kernels/reduce_mean.rs:40-93, cuda/src/ptx/headers/aggregation_op_macros.cuh:1-49. */
int32_t rmlk_hip_reduce_mean(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                             const int64_t *axes, int32_t n_axes, const void *in, void *out);

/* Softmax along the middle axis of a dense [outer, axis_len, inner] view (inner == 1 is the
 * last-axis case; outer=N, axis_len=C, inner=H*W is the reference's rank-4 channel mode).
 * Max-subtracted: exp(x - max) / sum. dtype in {FLOAT, DOUBLE}.
 * ref: cuda/src/kernels/softmax.rs:5-37 (cuDNN), runtime/src/providers/cuda/backend/softmax.rs:121-158 */
int32_t rmlk_hip_softmax(rmlk_stream_t stream, int32_t dtype, int64_t outer, int64_t axis_len,
                         int64_t inner, const void *in, void *out);

/* Batched MatMul, row-major: C[b] = op(A[b]) . op(B[b]), op = transpose when trans_x != 0.
 * A is m x k (k x m when trans_a) with leading dimension lda, B is k x n (n x k when trans_b) with
 * ldb, C is m x n with ldc. stride_x is the element distance between batches; 0 broadcasts one
 * matrix over the batch (the reference copies the operand `batch` times instead,
 * ref: runtime/src/providers/cuda/backend/matmul.rs:48-86). fp32 in, fp32 accumulate. dtype FLOAT.
 * `workspace` is device scratch of at least rmlk_hip_matmul_workspace_size(...) bytes (may be NULL
 * when that is 0); it is only written and read inside the call's own stream order
 * (calls that share one workspace must not overlap in time); its contents on entry do not matter.
 * ref: cuda/src/kernels/gemm.rs:112-136,191-232 (cublasGemmStridedBatchedEx). */
int32_t rmlk_hip_matmul(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t m, int64_t n,
                        int64_t k, const void *a, int64_t lda, int64_t stride_a, int32_t trans_a,
                        const void *b, int64_t ldb, int64_t stride_b, int32_t trans_b, void *c,
                        int64_t ldc, int64_t stride_c, void *workspace, size_t workspace_bytes);

size_t rmlk_hip_matmul_workspace_size(int32_t dtype, int64_t batch, int64_t m, int64_t n,
                                      int64_t k);

/* Which kernel rmlk_hip_matmul picks for a row-major problem of this size, as text
 * ("mfma128x128 splitk=1", "mfma64x64 splitk=8", "gemv splitk=32"); for profiles and reports.
 * Writes at most `size` bytes including the terminator; returns the length needed. */
int32_t rmlk_hip_matmul_describe(int32_t dtype, int64_t batch, int64_t m, int64_t n, int64_t k,
                                 char *buf, int32_t size);

/* rmlk_hip_matmul for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments and results as rmlk_hip_matmul (bit for bit) without the workspace: the split-K partials
 * go to a fixed device array of RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES that is part of the library's
 * code object (every GPU the library runs on holds its copy until the process ends: 32 MiB of
 * device memory per GPU and per process that loads the library, whether or not this entry point is
 * ever called). The first call on a device looks the array's address up (hipGetSymbolAddress) and
 * must therefore be made OUTSIDE stream capture; every later call on that device does not. A problem whose
 * rmlk_hip_matmul_workspace_size exceeds that returns RMLK_ERR_SCRATCH_LIMIT and launches nothing.
 * The call allocates nothing and frees nothing. All calls on one GPU share the array: calls that may
 * overlap in time on one GPU (different streams, different threads) race on it and must be ordered
 * by the caller; calls on one stream are ordered by the stream. */
#define RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES (32 << 20)
int32_t rmlk_hip_matmul_noalloc(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t m,
                                int64_t n, int64_t k, const void *a, int64_t lda, int64_t stride_a,
                                int32_t trans_a, const void *b, int64_t ldb, int64_t stride_b,
                                int32_t trans_b, void *c, int64_t ldc, int64_t stride_c);

/* Transpose: out = permute(in, perm); out.shape[d] = in_shape[perm[d]]. Any 1/2/4/8-byte dtype.
 * ref: cuda/src/kernels/transpose.rs:38-80, cuda/src/ptx/headers/transpose_op_macros.cuh:1-25. */
int32_t rmlk_hip_transpose(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                           const int64_t *perm, const void *in, void *out);

/* Expand: broadcast-copy `in` (in_shape, right-aligned, dims of 1 repeat) to dense `out_shape`.
 * ref: cuda/src/kernels/expand.rs:35-76, cuda/src/ptx/headers/expand_op_macros.cuh:1-31. */
int32_t rmlk_hip_expand(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                        const rmlk_dims *out_shape, const void *in, void *out);

/* Slice with the ONNX clamp rules already applied by the host: for every dim d,
 * out[.., o_d, ..] = in[.., starts[d] + o_d * steps[d], ..], 0 <= o_d < out_shape[d]. steps may be
 * negative; the caller guarantees every addressed index lies in [0, in_shape[d]) (checked).
 * ref: cuda/src/kernels/slice.rs:61-122, cuda/src/ptx/headers/slice_op_macros.cuh:1-97; the clamp
 * rules the host applies are runtime/src/providers/cuda/backend/slice.rs:357-463. */
int32_t rmlk_hip_slice(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                       const rmlk_dims *starts, const rmlk_dims *steps, const rmlk_dims *out_shape,
                       const void *in, void *out);

/* Concat, one call per input: copies dense `in` (in_shape) into dense `out` (out_shape) at
 * `axis_offset` along `axis`. A zero-length input is legal and launches nothing.
 * ref: runtime/src/providers/cuda/backend/concat.rs:28-76 (a host loop of memcpy_dtod). */
int32_t rmlk_hip_concat(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                        const rmlk_dims *out_shape, int32_t axis, int64_t axis_offset,
                        const void *in, void *out);

/* Concat of all `n_inputs` dense inputs (shapes in_shapes[k], device pointers ins[k]; both arrays
 * are HOST memory) along `axis` into dense `out` (out_shape, whose extent along `axis` is the sum
 * of the inputs'). One launch for up to 8 inputs (the growing KV cache plus the new row costs one
 * launch, not two); more inputs, or very large ones, take one strided copy per input.
 * ref: runtime/src/providers/cuda/backend/concat.rs:28-76 (the whole host loop). */
int32_t rmlk_hip_concat_many(rmlk_stream_t stream, int32_t dtype, int32_t n_inputs,
                             const rmlk_dims *in_shapes, const void *const *ins,
                             const rmlk_dims *out_shape, int32_t axis, void *out);

/* Gather along `axis`: out[outer, j, inner] = data[outer, idx[j], inner], j < n_idx; negative
 * indices wrap once. idx_dtype INT32 or INT64. An index outside [-dim, dim) writes zeros for that
 * row and stores 1 to *err_flag (device int32, may be NULL); the host reads it when it chooses.
 * ref: runtime/src/providers/cuda/backend/gather.rs:199-258 (index D2H + one memcpy_dtod per
 * index), index rule runtime/src/utils/mod.rs:155-175. */
int32_t rmlk_hip_gather(rmlk_stream_t stream, int32_t dtype, int32_t idx_dtype,
                        const rmlk_dims *data_shape, int32_t axis, int64_t n_idx, const void *data,
                        const void *idx, void *out, int32_t *err_flag);

/* ScatterND. `out` must already hold a copy of `data` (or be `data` itself for an in-place
 * update); this call writes only the addressed slices. idx is INT64 [n_tuples, tuple_size],
 * updates is [n_tuples, slice_len] with slice_len = prod(data_shape[tuple_size:]). Negative
 * indices wrap once; an index outside [-dim, dim) skips the tuple and stores 1 to *err_flag.
 * NONE is plain assignment (the reference's `in + 0*out` turns Inf/NaN already in `data` into
 * NaN; ONNX does not). ADD MUL MAX MIN are atomic per element, so duplicates combine in an
 * unspecified order. dtype in {FLOAT, DOUBLE, INT32, INT64} (NONE: any 1/2/4/8-byte type).
 * ref: cuda/src/kernels/scatter_nd.rs:91-210, cuda/src/ptx/headers/scatter_op_macros.cuh:19-93. */
typedef enum rmlk_scatter_reduction {
    RMLK_SCATTER_NONE = 0,
    RMLK_SCATTER_ADD = 1,
    RMLK_SCATTER_MUL = 2,
    RMLK_SCATTER_MAX = 3,
    RMLK_SCATTER_MIN = 4
} rmlk_scatter_reduction;

int32_t rmlk_hip_scatter_nd(rmlk_stream_t stream, int32_t reduction, int32_t dtype,
                            const rmlk_dims *data_shape, int64_t n_tuples, int32_t tuple_size,
                            const int64_t *idx, const void *updates, void *out,
                            int32_t *err_flag);

/* ScatterND (reduction none) with the ONNX copy semantics in ONE pass: out = data with the
 * addressed slices taken from `updates` (`out` is written everywhere, `data` is only read; they
 * may be the same buffer). Up to 64 tuples of 16-byte aligned slices take one launch that reads
 * data and writes out once; anything else copies data to out and calls rmlk_hip_scatter_nd. When
 * several tuples address one slice, the last one wins. Index rules and *err_flag as above.
 * ref: runtime/src/providers/cuda/backend/scatter_nd.rs:128-129 (memcpy_dtod of data, then the
 * scatter kernel). */
int32_t rmlk_hip_scatter_nd_copy(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *data_shape,
                                 int64_t n_tuples, int32_t tuple_size, const int64_t *idx,
                                 const void *updates, const void *data, void *out,
                                 int32_t *err_flag);

/* Trilu on a dense [batch, rows, cols] view: keeps the upper (col >= row + k) or lower
 * (col <= row + k) triangle and WRITES ZERO elsewhere (the reference leaves those untouched).
 * ref: cuda/src/kernels/trilu.rs:36-78, cuda/src/ptx/headers/trilu_op_macros.cuh:1-43. */
int32_t rmlk_hip_trilu(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t rows,
                       int64_t cols, int32_t upper, int64_t k, const void *in, void *out);

/* ---- fused operator chains --------------------------------------------------------------------
 * The reference launches one kernel per ONNX node (runtime/src/providers/cuda/backend/<op>.rs); the
 * entry points below have no single counterpart there. Each computes, in one pass over
 * memory, the chain of nodes named in its comment, and rounds every intermediate exactly as the
 * separate kernels do, so a graph gives the same result either way. They support fp32 and return
 * RMLK_ERR_UNSUPPORTED for layouts they do not cover (the caller then runs the separate kernels).
 */

/* y[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * gamma   (reciprocal_form == 0), or
 * y[r, :] = x[r, :] * (1 / sqrt(mean(x[r, :]^2) + eps)) * gamma   (reciprocal_form != 0).
 * Chain: Pow(x, 2) -> ReduceMean(axis -1, keepdims) -> Add(eps) -> Sqrt -> Div -> Mul(gamma)
 * (ref kernels: cuda/src/kernels/binary.rs:58-100, reduce_mean.rs:40-93, unary.rs:10-42).
 * x, out dense [rows, cols]; gamma [cols]; cols % 4 == 0, cols <= 8192, 16-byte aligned. */
int32_t rmlk_hip_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows, int64_t cols,
                         const void *x, const void *gamma, float eps, int32_t reciprocal_form,
                         void *out);

/* sum_out = a + b (same dense [rows, cols] shape), out = RMSNorm(sum_out) as above, in one pass:
 * the residual Add in front of a norm, whose result the residual stream reads again.
 * Chain: Add -> the RMSNorm chain. */
int32_t rmlk_hip_add_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows, int64_t cols,
                             const void *a, const void *b, const void *gamma, float eps,
                             int32_t reciprocal_form, void *sum_out, void *out);

/* out = Softmax(x / scale + mask) (scale_is_mul == 0) or Softmax(x * scale + mask) over the last
 * axis. `shape` is x's (and out's) dense shape; `mask_stride` gives the mask's element stride per
 * dim of `shape` (0 on broadcast dims, 1 on the last dim).
 * Chain: Div|Mul(x, scalar) -> Add(mask) -> Softmax(axis -1)
 * (ref kernels: cuda/src/kernels/binary.rs:58-100, softmax.rs:5-37). */
int32_t rmlk_hip_scale_mask_softmax(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *shape,
                                    const rmlk_dims *mask_stride, int32_t scale_is_mul,
                                    float scale, const void *x, const void *mask, void *out);

/* out = (gate * sigmoid(gate)) * up over n elements.
 * Chain: Sigmoid(gate) -> Mul(gate, .) -> Mul(., up)
 * (ref kernels: cuda/src/kernels/unary.rs:10-42 via cuDNN sigmoid, binary.rs:58-100). */
int32_t rmlk_hip_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n, const void *gate,
                        const void *up, void *out);

/* ---- one-row products whose split-K combine is left to the consumer -----------------------------
 * A one-row MatMul (decode) streams its weights in K slabs and leaves one partial row per slab; these
 * entry points let the kernel that consumes the product add the slabs up itself (ascending slab
 * order), which saves the combine launch. No counterpart in the reference.
 *
 * rmlk_hip_gemv_partials: partial rows of x[k] . B[k, n] (B row-major, leading dimension ldb) into
 * `workspace` as [splits][n]; *splits_out = number of slabs (>= 1). n % 4 == 0, 16-byte aligned B.
 * rmlk_hip_gemv_partials_workspace_size: bytes the workspace must hold for that call. */
size_t rmlk_hip_gemv_partials_workspace_size(int32_t dtype, int64_t n, int64_t k);
int32_t rmlk_hip_gemv_partials(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                               const void *x, const void *b, int64_t ldb, void *workspace,
                               size_t workspace_bytes, int32_t *splits_out);
/* out[i] = swiglu(gate_i, up_i) with gate_i = sum of the slabs at element gate_offset + i and up_i
 * likewise at up_offset + i (a joint [gate | up] product): rmlk_hip_swiglu on partial slabs. */
int32_t rmlk_hip_splitk_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n, const void *partials,
                               int32_t splits, int64_t slab, int64_t gate_offset, int64_t up_offset,
                               void *out);

/* Grouped-query attention over many query rows in one kernel:
 *   out[b, h, s, :] = Softmax_l(q[b, h, s, :] . k[b, h / rep, l, :] * scale + mask[b, h, s, l]) . v[b, h / rep, :, :]
 * (scale_is_mul == 0: the scores are DIVIDED by `scale`). q and out are dense [batch, kv_heads * rep,
 * q_len, head_dim], k and v dense [batch, kv_heads, kv_len, head_dim]; `mask_stride` gives the mask's
 * element stride per dim of [batch, heads, q_len, kv_len] (0 on broadcast dims, 1 on the last).
 * Chain: MatMul(q, k^T) -> Div|Mul(scalar) -> Add(mask) -> Softmax(axis -1) -> MatMul(., v) with the
 * KV heads repeated over their query heads (ref kernels: cuda/src/kernels/gemm.rs:191-232,
 * binary.rs:58-100, softmax.rs:5-37). The softmax is accumulated chunk by chunk over the keys with a
 * running maximum, so results agree with the chain to rounding (about 1e-6 relative), not bit for bit.
 * out_seq_major != 0 writes out as [batch, q_len, heads, head_dim] instead, i.e. the
 * Transpose(perm 0,2,1,3) that leads to the output projection (ref: cuda/src/kernels/transpose.rs:38-80).
 * Covers head_dim == 64 and kv_len % 4 == 0 with 16-byte aligned operands; RMLK_ERR_UNSUPPORTED
 * otherwise (the caller then runs the separate kernels). */
int32_t rmlk_hip_attention(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                           int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                           const void *q, const void *k, const void *v, const void *mask,
                           const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                           int32_t out_seq_major, void *out);
/* The same kernel with room to skip what the mask hides: with `workspace` of at least
 * rmlk_hip_attention_workspace_size() bytes a small kernel first marks, per tile of 64 queries and
 * chunk of 64 keys (of 128 where the launch has no more blocks than compute units), whether the mask holds anything but -inf there, and the main kernel neither loads
 * nor multiplies the chunks a tile cannot see (a causal mask: about half of them). Their probabilities
 * are exact zeros, so results are those of rmlk_hip_attention bit for bit, with two exceptions: a NaN
 * or infinity in a K or V row no query of the tile can see does not reach that tile's output
 * (0 * NaN would), and a row with nothing visible anywhere is NaN as before. The size is 0 (and a
 * null workspace allowed) where skipping does not apply: q_len not a multiple of 64, fewer than 4 chunks (6 of 128), or
 * more than 128 chunks. The workspace is 16-byte aligned (one that is not, or is too small, is
 * ignored: every chunk is then visited) and belongs to the call until its kernels have run. rmlk_hip_attention is this call with a null workspace. */
size_t rmlk_hip_attention_workspace_size(int32_t dtype, int64_t batch, int64_t kv_heads, int64_t rep,
                                         int64_t q_len, int64_t kv_len, int64_t head_dim,
                                         const rmlk_dims *mask_stride);
int32_t rmlk_hip_attention_ws(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                              int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                              const void *q, const void *k, const void *v, const void *mask,
                              const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                              int32_t out_seq_major, void *workspace, size_t workspace_bytes, void *out);
/* The map of rmlk_hip_attention_ws made once and used by several launches over ONE mask (the layers
 * of a model share theirs): rmlk_hip_attention_map marks in `map` (rmlk_hip_attention_map_size()
 * bytes, 16-byte aligned) which (query tile, key chunk) pairs of `mask` hold anything but -inf;
 * rmlk_hip_attention_mapped is rmlk_hip_attention_ws over such a map, without making it again - the
 * same results bit for bit. The map belongs to the mask, its strides and the sizes it was made for;
 * between two launches that use it it must not change (each launch leaves the item counter behind
 * the map zero, as it found it), and launches that share it are ordered by one stream. Since the
 * cost of the map is shared, two chunks are enough for it to exist: the size is 0 where skipping
 * does not apply at all (q_len not a multiple of 64, fewer than 2 or more than 128 chunks), and the
 * calls then answer RMLK_ERR_UNSUPPORTED. No counterpart in the reference. */
size_t rmlk_hip_attention_map_size(int32_t dtype, int64_t batch, int64_t kv_heads, int64_t rep,
                                   int64_t q_len, int64_t kv_len, int64_t head_dim,
                                   const rmlk_dims *mask_stride);
int32_t rmlk_hip_attention_map(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                               int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                               const void *mask, const rmlk_dims *mask_stride, void *map,
                               size_t map_bytes);
int32_t rmlk_hip_attention_mapped(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                                  int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                                  const void *q, const void *k, const void *v, const void *mask,
                                  const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                                  int32_t out_seq_major, const void *map, size_t map_bytes, void *out);
/* rmlk_hip_attention_mapped with the [batch, q_len, heads, head_dim] result also stored as the three
 * bfloat16 pieces of rmlk_hip_attention_ws_pieces (same layout of `out_pieces`, same bits). */
int32_t rmlk_hip_attention_mapped_pieces(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                         int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                         int64_t head_dim, const void *q, const void *k, const void *v,
                                         const void *mask, const rmlk_dims *mask_stride,
                                         int32_t scale_is_mul, float scale, const void *map,
                                         size_t map_bytes, void *out, void *out_pieces);
/* rmlk_hip_attention_ws with a [batch, q_len, heads, head_dim] result (out_seq_major) that is also
 * stored as three bfloat16 pieces, as rmlk_hip_bf16x3_split would split the [batch * q_len, heads *
 * head_dim] matrix it is: `out_pieces` holds rmlk_hip_bf16x3_pieces_size(batch * q_len, heads *
 * head_dim) bytes. For an output projection over the pieces (rmlk_hip_matmul_bf16x3) that then needs
 * no split launch. The same values in `out`, bit for bit. */
int32_t rmlk_hip_attention_ws_pieces(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                                     int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                                     const void *q, const void *k, const void *v, const void *mask,
                                     const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                                     void *workspace, size_t workspace_bytes, void *out, void *out_pieces);

/* The same attention for a handful of query rows per KV head (rep * q_len <= 16: a decode step),
 * where there is no matrix work, only K and V to read: the keys are split over blocks in chunks of
 * 64, every block leaves a partial softmax in `workspace`, a second small kernel merges them. Any
 * kv_len; head_dim == 64; RMLK_ERR_UNSUPPORTED otherwise. */
size_t rmlk_hip_attention_few_rows_workspace_size(int32_t dtype, int64_t batch, int64_t kv_heads,
                                                  int64_t rep, int64_t q_len, int64_t kv_len,
                                                  int64_t head_dim);
int32_t rmlk_hip_attention_few_rows(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                    int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                    int64_t head_dim, const void *q, const void *k, const void *v,
                                    const void *mask, const rmlk_dims *mask_stride,
                                    int32_t scale_is_mul, float scale, int32_t out_seq_major,
                                    void *workspace, size_t workspace_bytes, void *out);
/* The same in ONE launch: the block that finishes a KV head's last chunk merges that head's partial
 * results itself. `counters` holds batch * kv_heads 32-bit counters in device memory that are zero
 * before the first call; the kernel counts finished blocks there and leaves every counter zero again,
 * so one zeroed buffer serves all later calls on the same stream (calls that overlap on the GPU need
 * buffers of their own, like the workspace). Results are those of rmlk_hip_attention_few_rows bit for
 * bit. */
int32_t rmlk_hip_attention_few_rows_one_launch(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                               int64_t kv_heads, int64_t rep, int64_t q_len,
                                               int64_t kv_len, int64_t head_dim, const void *q,
                                               const void *k, const void *v, const void *mask,
                                               const rmlk_dims *mask_stride, int32_t scale_is_mul,
                                               float scale, int32_t out_seq_major, void *workspace,
                                               size_t workspace_bytes, int32_t *counters, void *out);

/* ---- constant weights stored as 16-bit values ----------------------------------------------------
 * The products over constant weights below take the storage type of the weights as `w_dtype`:
 * RMLK_FLOAT, or RMLK_FLOAT16 / RMLK_BFLOAT16 for weights that were rounded ONCE, when they were
 * stored (rmlk_hip_store_weights), to half the bytes a token has to stream. The arithmetic stays
 * fp32: a stored value is widened exactly, products and sums are formed in float, x, gamma, the
 * residual and every output are float. A many-row product over 16-bit weights equals the fp32
 * product over the widened weights bit for bit (same kernels behind the widening); the one-row
 * products agree with it to rounding (other order of the sum). 16-bit weights must be K-contiguous
 * (trans_b), rows whole 128-bit units (k % 8 == 0, ldb % 8 == 0, 16-byte aligned base); ldb / ldw
 * and the row offsets count stored values. RMLK_ERR_UNSUPPORTED otherwise, and for any other
 * w_dtype. (ref: the f16 kernel symbols of the reference, e.g. cuda/src/ptx/add.cu:19-25, which its
 * provider cannot run: runtime/src/providers/cuda/data.rs:109-126; storage with fp32 accumulation
 * has no counterpart there.)
 *
 * rmlk_hip_store_weights: dst[i] = src[i] (float) rounded to nearest even in `w_dtype`
 * (RMLK_FLOAT16 or RMLK_BFLOAT16; NaN stays NaN, overflow gives infinity). */
int32_t rmlk_hip_store_weights(rmlk_stream_t stream, int32_t w_dtype, int64_t n, const void *src,
                               void *dst);
/* Stores 0 to *fits (device memory, set to 1 by the caller beforehand) when one of the n floats at
 * `src` would come back from `w_dtype` storage with other bits (a NaN never fits); leaves it alone
 * otherwise. Weights that fit - every checkpoint trained in bfloat16 and exported as float does -
 * can be held as 16-bit values at no loss. */
int32_t rmlk_hip_weights_fit(rmlk_stream_t stream, int32_t w_dtype, int64_t n, const void *src,
                             int32_t *fits);

/* ---- products that share their first operand (q/k/v, gate/up) ----------------------------------
 * The weights of such MatMuls (ref: one cublasGemmStridedBatchedEx each,
 * cuda/src/kernels/gemm.rs:191-232) lie side by side in one matrix B: row-major [k, sum(widths)]
 * (trans_b == 0), or K-contiguous [sum(widths), k], one row per output column (trans_b != 0), which
 * is also what the one-row products below read - one copy of the weights serves every row count.
 *
 * rmlk_hip_matmul_grouped: outs[i] (dense [m, widths[i]]) = A[m, k] . B[:, block i], block i being
 * the next widths[i] columns (rows of a K-contiguous B). One launch covers all blocks where whole tiles allow it; otherwise
 * the blocks are multiplied one after the other, with the same results as rmlk_hip_matmul on each.
 * groups <= 4. The workspace must hold rmlk_hip_matmul_grouped_workspace_size bytes. */
size_t rmlk_hip_matmul_grouped_workspace_size(int32_t dtype, int64_t m, int64_t k, int32_t groups,
                                              const int64_t *widths);
int32_t rmlk_hip_matmul_grouped(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t k,
                                const void *a, int64_t lda, int32_t w_dtype, const void *b, int64_t ldb,
                                int32_t trans_b, int32_t groups, const int64_t *widths,
                                void *const *outs, void *workspace, size_t workspace_bytes);
/* out[m, n] = swiglu(A . B[:, gate_offset .. +n], A . B[:, up_offset .. +n]) (see rmlk_hip_swiglu)
 * in one launch, the activation applied to the accumulators; with trans_b the offsets count rows of
 * the K-contiguous B. Covers n % 64 == 0, k % 32 == 0, 16-byte aligned rows and at least one
 * 128 x 64 tile per compute unit; RMLK_ERR_UNSUPPORTED otherwise (the caller then multiplies and
 * activates separately). Results do not depend on trans_b. */
int32_t rmlk_hip_matmul_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t n, int64_t k,
                               const void *a, int64_t lda, int32_t w_dtype, const void *b, int64_t ldb,
                               int32_t trans_b, int64_t gate_offset, int64_t up_offset, void *out,
                               int64_t ldc);

/* One-row product with K-CONTIGUOUS weights: y[n] = sum_k x[k] * wt[n][k] (wt row-major [n, k],
 * leading dimension ldw), i.e. rmlk_hip_matmul with m = 1 and trans_b. Every output column is
 * finished inside one wavefront: no workspace and no combine launch, at any width. k % 4 == 0,
 * 16-byte aligned operands; RMLK_ERR_UNSUPPORTED otherwise. A session stores constant weight
 * matrices K-contiguous for it (ref: cublasGemmStridedBatchedEx with
 * CUBLAS_OP_T on a transposed operand, cuda/src/kernels/gemm.rs:191-232). */
int32_t rmlk_hip_gemv_kmajor(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k, const void *x,
                        int32_t w_dtype, const void *wt, int64_t ldw, void *y);
/* y[i] = swiglu(x . wt[gate_row + i, :], x . wt[up_row + i, :]) for i < n (see rmlk_hip_swiglu): the
 * gate and the up projection of a one-row input and the activation in one launch. */
int32_t rmlk_hip_gemv_kmajor_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                               const void *x, int32_t w_dtype, const void *wt, int64_t ldw,
                               int64_t gate_row, int64_t up_row, void *y);
/* rmlk_hip_gemv_kmajor with a residual row added to the result: y = x . wt^T + residual (the Add
 * behind an output projection; ref kernels: gemm.rs:191-232, binary.rs:58-100). */
int32_t rmlk_hip_gemv_kmajor_add(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k, const void *x,
                                 int32_t w_dtype, const void *wt, int64_t ldw, const void *residual,
                                 void *y);
/* The same products over RMSNorm(x) * gamma instead of x, the normalised row never stored: every
 * wavefront works out the row's statistics with rmlk_hip_rmsnorm's arithmetic, so the results equal
 * rmlk_hip_rmsnorm followed by the product bit for bit. k <= 8192, gamma 16-byte aligned, else
 * RMLK_ERR_UNSUPPORTED. Chain: Pow, ReduceMean, Add, Sqrt, Div | Div(1,.) Mul, Mul, MatMul
 * (ref kernels: unary.rs:10-42, reduce_mean.rs:5-36, binary.rs:58-100, gemm.rs:191-232). */
int32_t rmlk_hip_gemv_kmajor_normed(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k, const void *x,
                                    const void *gamma, float eps, int32_t reciprocal_form,
                                    int32_t w_dtype, const void *wt, int64_t ldw, void *y);
int32_t rmlk_hip_gemv_kmajor_swiglu_normed(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                           const void *x, const void *gamma, float eps,
                                           int32_t reciprocal_form, int32_t w_dtype, const void *wt,
                                           int64_t ldw, int64_t gate_row, int64_t up_row, void *y);

/* ---- many-row products whose split-K combine is left to the consumer ----------------------------
 * rmlk_hip_matmul_partials: the tiled kernels of rmlk_hip_matmul for A[m, k] . B (row-major [k, n],
 * or K-contiguous [n, k] with trans_b; m > 8) without the combine: `workspace` receives *splits_out partial matrices [m, n] one after
 * the other (*splits_out >= 1; their sum in ascending order is the product rmlk_hip_matmul returns).
 * rmlk_hip_splitk_add_rmsnorm: rmlk_hip_add_rmsnorm whose first operand is that sum,
 * a = partials[0] + partials[1] + ..; `slab` = elements from one partial matrix to the next.
 * Together they save the combine launch of a projection that feeds a residual Add and a norm.
 * No counterpart in the reference. */
size_t rmlk_hip_matmul_partials_workspace_size(int32_t dtype, int64_t m, int64_t n, int64_t k);
int32_t rmlk_hip_matmul_partials(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t n, int64_t k,
                                 const void *a, int64_t lda, int32_t w_dtype, const void *b, int64_t ldb,
                                 int32_t trans_b, void *workspace, size_t workspace_bytes,
                                 int32_t *splits_out);
int32_t rmlk_hip_splitk_add_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows, int64_t cols,
                                    const void *partials, int32_t splits, int64_t slab,
                                    const void *b, const void *gamma, float eps,
                                    int32_t reciprocal_form, void *sum_out, void *out);

/* ---- many-row products over bfloat16 weights on the bf16 matrix cores ----------------------------
 * c[m, n] = a[m, k] . wt[n, k]^T with a fp32, wt bfloat16 values (K-contiguous, as
 * rmlk_hip_store_weights writes them) and fp32 results, multiplied by v_mfma_f32_32x32x16_bf16
 * without rounding a: a float is the exact sum of three bfloat16 pieces (8 + 8 + 8 significant
 * bits), a product of two bfloat16 values is exact in fp32, so three MFMAs per tile and K chunk
 * over the three pieces add up exactly the products a[i, k] * wt[j, k] - what remains is the
 * rounding of fp32 accumulation, as in any fp32 product with its sums in another order. About 2.5x
 * the rate of the fp32 MFMA kernels. No counterpart in the reference (fp32 cuBLAS,
 * cuda/src/kernels/gemm.rs:191-232).
 *
 * rmlk_hip_bf16x3_split writes the pieces of a as three planes [3][m_pad][k] of bfloat16 (m_pad = m
 * rounded up to a multiple of 128, the padding rows zero) into `pieces`, which must hold
 * rmlk_hip_bf16x3_pieces_size(m, k) bytes; k % 8 == 0, lda % 4 == 0, 16-byte aligned pointers.
 * Infinities and NaNs of a arrive in the result as they would from an fp32 product.
 * rmlk_hip_matmul_bf16x3 multiplies the pieces by wt: with splits == 1 into c (leading dimension
 * ldc); with splits > 1 slab s of K (k / splits values) goes to c + s * slab elements, for a reader
 * that adds the slabs up itself (rmlk_hip_splitk_add_rmsnorm, rmlk_hip_head_rows).
 * rmlk_hip_bf16x3_splits is the number of slabs that fills the GPU for a size (1 for wide products;
 * 0 for sizes the kernel does not take). rmlk_hip_matmul_bf16x3_swiglu is rmlk_hip_matmul_swiglu over
 * the pieces: out[m, n] = swiglu(a . wt[gate_row .. +n]^T, a . wt[up_row .. +n]^T); with out_pieces
 * (NULL: not wanted; else rmlk_hip_bf16x3_pieces_size(m, n) bytes) the same launch also stores the
 * pieces of out, as rmlk_hip_bf16x3_split would, for a product that reads it.
 * Covered: k % 32 == 0 (per slab), n % 128 == 0 (swiglu: n % 64 == 0), ldw % 8 == 0, operands below
 * 4 GiB; RMLK_ERR_UNSUPPORTED otherwise. */
size_t rmlk_hip_bf16x3_pieces_size(int64_t m, int64_t k);
int32_t rmlk_hip_bf16x3_split(rmlk_stream_t stream, int64_t m, int64_t k, const void *a, int64_t lda,
                              void *pieces);
int32_t rmlk_hip_bf16x3_splits(int64_t m, int64_t n, int64_t k);
int32_t rmlk_hip_matmul_bf16x3(rmlk_stream_t stream, int64_t m, int64_t n, int64_t k, const void *pieces,
                               const void *wt, int64_t ldw, int32_t splits, void *c, int64_t ldc,
                               int64_t slab);
int32_t rmlk_hip_matmul_bf16x3_swiglu(rmlk_stream_t stream, int64_t m, int64_t n, int64_t k,
                                      const void *pieces, const void *wt, int64_t ldw, int64_t gate_row,
                                      int64_t up_row, void *out, int64_t ldc, void *out_pieces);
/* rmlk_hip_rmsnorm / rmlk_hip_add_rmsnorm / rmlk_hip_splitk_add_rmsnorm (b NULL: no Add, sum_out
 * unused; splits == 1: `partials` is the row matrix itself) whose result goes to `out` AND, split
 * as by rmlk_hip_bf16x3_split, to `pieces` (rmlk_hip_bf16x3_pieces_size(rows, cols) bytes; the
 * padding rows are left as they are: no row of a product depends on them): a norm in front of a
 * product over the pieces needs no split launch. cols % 8 == 0. */
int32_t rmlk_hip_rmsnorm_pieces(rmlk_stream_t stream, int64_t rows, int64_t cols, const void *partials,
                                int32_t splits, int64_t slab, const void *b, const void *gamma, float eps,
                                int32_t reciprocal_form, void *sum_out, void *out, void *pieces);
/* rmlk_hip_matmul_grouped over the pieces: outs[i] (dense [m, widths[i]]) = a . (the next widths[i]
 * rows of wt)^T, one launch over the joint matrix whose 32-column blocks go to their member's
 * output. groups <= 4, every width a multiple of 32, their sum of 128. */
int32_t rmlk_hip_matmul_bf16x3_grouped(rmlk_stream_t stream, int64_t m, int64_t k, const void *pieces,
                                       const void *wt, int64_t ldw, int32_t groups, const int64_t *widths,
                                       void *const *outs);

/* Rotary position embedding, half-rotation form, over x of logical shape [B, H, S, D]:
 * out = x * cos + concat(-x[..., D/2:], x[..., :D/2]) * sin, out dense [B, H, S, D].
 * x, cos and sin are read through element strides per dim of `shape` (innermost stride 1; 0 on
 * broadcast dims), so a [B, S, H, D] projection output can be rotated and transposed in one pass.
 * Chain: Slice, Slice, Neg, Concat, Mul, Mul, Add (optionally after Transpose perm 0,2,1,3)
 * (ref kernels: cuda/src/kernels/slice.rs:61-122, unary.rs:10-42, binary.rs:58-100,
 * transpose.rs:38-80). */
int32_t rmlk_hip_rotary(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *shape,
                        const rmlk_dims *x_stride, const rmlk_dims *cos_stride,
                        const rmlk_dims *sin_stride, const void *x, const void *cos,
                        const void *sin, void *out);

/* Several streams of head rows in one launch. Stream i reads rows of D elements of x, logical
 * shape [B, H, S, D], through element strides (innermost 1), rotates them like rmlk_hip_rotary
 * when cos and sin are given (both NULL: the rows are moved unchanged, i.e. a Transpose perm
 * 0,2,1,3 read through strides) and writes them
 *   idx == NULL: densely to out [B, H, S, D];
 *   idx != NULL: to out = the data tensor of a ScatterND (reduction none) that already holds its
 *                copy of the data, shape data_shape = [.., D] of rank tuple_size + 1, row r
 *                (b, h, s order) going where the index tuple idx[r * tuple_size ..] points;
 *                negative indices wrap, an index out of range sets *err_flag and skips the row
 *                (as rmlk_hip_scatter_nd).
 * One launch covers what a decoder layer does behind its q/k/v projection (q rotated, k rotated
 * into the key cache, v moved into the value cache); the results equal the separate kernels'
 * bit for bit. At most 4 streams, all with the same D; tuple_size <= 4.
 * Chain per stream: [Transpose 0,2,1,3] [Slice Slice Neg Concat Mul Mul Add] [ScatterND]
 * (ref: cuda/src/kernels/transpose.rs:38-80, slice.rs:61-122, unary.rs:10-42, binary.rs:58-100,
 * scatter_nd.rs:11-77; runtime/src/providers/cuda/backend/scatter_nd.rs:78-225). */
typedef struct rmlk_row_stream {
    rmlk_dims shape;        /* logical [B, H, S, D] */
    rmlk_dims x_stride;     /* element strides of x over those dims */
    const void *x;
    const void *cos;        /* NULL (with sin): move */
    const void *sin;
    rmlk_dims cos_stride;   /* read only when cos / sin are given */
    rmlk_dims sin_stride;
    void *out;
    const int64_t *idx;     /* NULL: dense output */
    int32_t tuple_size;     /* read only when idx is given */
    rmlk_dims data_shape;
    int32_t partials;       /* > 1 (rmlk_hip_head_rows only): x is the sum, in ascending order, of this
                               many matrices that lie partial_stride elements apart, the first at x -
                               the partial sums of a split-K product (rmlk_hip_matmul_partials) whose
                               combine launch this saves; 0 or 1: x itself */
    int64_t partial_stride;
} rmlk_row_stream;
int32_t rmlk_hip_head_rows(rmlk_stream_t stream, int32_t dtype, int32_t n_streams,
                           const rmlk_row_stream *streams, int32_t *err_flag);

/* rmlk_hip_gemv_kmajor[_normed] and rmlk_hip_head_rows in one launch, for the q/k/v projection of
 * ONE token: the one-row product x[k] . wt[n, k]^T (over RMSNorm(x) * gamma when gamma is given;
 * gamma NULL: over x) is not stored; stream i takes its columns [first_col[i], first_col[i] +
 * H * D) as the H rows of a [1, H, 1, D] tensor (streams[i].shape; x and x_stride are ignored) and
 * rotates / moves / scatters them exactly as rmlk_hip_head_rows does (same arithmetic, same index
 * rules and *err_flag). first_col is HOST memory. RMLK_ERR_UNSUPPORTED when a stream is not one
 * token of one sequence, for more than 4 streams, or for operands the one-row products refuse.
 * No counterpart in the reference (gemm.rs:191-232 followed by the kernels listed above). */
int32_t rmlk_hip_gemv_kmajor_head_rows(rmlk_stream_t stream, int32_t dtype, int64_t k, const void *x,
                                       const void *gamma, float eps, int32_t reciprocal_form,
                                       int32_t w_dtype, const void *wt, int64_t ldw, int32_t n_streams,
                                       const rmlk_row_stream *streams, const int64_t *first_col,
                                       int32_t *err_flag);

/* ---- launches over tiny tensors collected into one ------------------------------------------------
 * Between rmlk_hip_batch_begin and rmlk_hip_batch_end on a stream, calls of rmlk_hip_binary (not
 * Pow), rmlk_hip_unary, rmlk_hip_cast, rmlk_hip_where, rmlk_hip_expand and rmlk_hip_concat_many whose
 * output has at most 1024 elements (FLOAT, DOUBLE, INT32, INT64, BOOL operands; any element size for
 * the moves) do not launch: they are recorded, and one single-block launch runs up to 24 records in
 * order with the element arithmetic of the kernels they replace (same bits). Every other call of
 * this library on the stream, rmlk_hip_batch_flush and rmlk_hip_batch_end send the recorded calls
 * out first, so effects keep the order of the calls; the operands of a recorded call must stay
 * valid until then. A caller that issues work on the stream by other means (its own kernels,
 * hipMemcpyAsync, events) calls rmlk_hip_batch_flush before it does. A decode step spends a dozen
 * launches on such tensors (a position turned into rotary tables, scatter indices, a mask).
 * rmlk_hip_batch_end returns the status of the launches the batch made. Recordable into a HIP
 * graph. No counterpart in the reference (one kernel per operator,
 * runtime/src/core/instance.rs:100-112). */
int32_t rmlk_hip_batch_begin(rmlk_stream_t stream);
int32_t rmlk_hip_batch_flush(rmlk_stream_t stream);
int32_t rmlk_hip_batch_end(rmlk_stream_t stream);
/* 1 when a call whose output iterates `shape`, its n_in (1..3) inputs walking that space with the
 * element strides strides[0 .. n_in - 1] and its output with strides[n_in], is one an open batch
 * records; 0 when it is launched as usual: more than 1024 elements, more than four dims left after
 * size-1 dims are dropped and jointly contiguous dims merged, or an operand whose farthest element
 * lies 2^31 elements or more from its first (a record's offsets are 32-bit). Host arithmetic only,
 * no GPU needed. No counterpart in the reference. */
int32_t rmlk_hip_batch_collects(const rmlk_dims *shape, int32_t n_in, const rmlk_dims *strides);

/* Fill `n` elements of `out` with the element at host address `value` (size of dtype).
 * ref: runtime/src/providers/cuda/backend/constant_of_shape.rs:59-62 (host vector + H2D). */
int32_t rmlk_hip_fill(rmlk_stream_t stream, int32_t dtype, int64_t n, const void *value,
                      void *out);

/* Range: out[i] = start + i * delta for i < n. `start` and `delta` are HOST scalars of `dtype`
 * (FLOAT, DOUBLE, INT32, INT64). ref: runtime/src/providers/cuda/backend/range.rs:103-109 (the
 * reference fills a host vector and uploads it). */
int32_t rmlk_hip_range(rmlk_stream_t stream, int32_t dtype, int64_t n, const void *start,
                       const void *delta, void *out);

/* Streaming yardsticks for benchmarks: the least a kernel can do with `bytes` on this chip, to be
 * timed next to the operators of the same traffic. READ: `bytes` of `src` are loaded (streaming
 * 128-bit loads, 32 KiB per block of 256 lanes, all requested up front, one trip) and reduced to
 * nothing; `dst` (>= 4 * bytes / 32768 bytes) is practically never written. COPY: `bytes` of `src`
 * go to `dst` (16 KiB per block, streaming loads and stores). `bytes` must be a multiple of the
 * block's share, `src` / `dst` 16-byte aligned. With `stamps` non-null (2 * number of blocks 64-bit
 * words of device memory) block b stores the constant 100 MHz clock (s_memrealtime) at its start in
 * stamps[2b] and at its end in stamps[2b + 1]: last end - first start is the time the memory system
 * needed, which a kernel trace cannot separate from dispatch. No counterpart in the reference. */
enum { RMLK_YARDSTICK_READ = 0, RMLK_YARDSTICK_COPY = 1 };
int32_t rmlk_hip_stream_yardstick(rmlk_stream_t stream, int32_t kind, size_t bytes, const void *src,
                                  void *dst, uint64_t *stamps);

/* Issue yardstick for benchmarks: what a SIMD does with other instructions beside fp32 MFMAs.
 * `blocks` blocks of eight wavefronts (two per SIMD of a compute unit): wavefronts 0..3 issue
 * 16 * iterations v_mfma_f32_32x32x2_f32 with something between them (`kind`), and with
 * `second_wavefront` non-zero wavefronts 4..7 run 64 * iterations dependent v_fma_f32 at the same
 * time. Kinds 0, 4, 8, 12, 16: one chain of MFMAs, that many independent v_fma_f32 behind each.
 * Kinds 100..103: four accumulators in turn (independent MFMAs, as in a GEMM step) and behind every
 * fourth MFMA nothing (100), one v_add_u32 (101), one ds_read_b128 (102), a v_add_u32 and the
 * ds_read_b128 that takes its result as the address (103). cycles[8 b + w] (device memory,
 * 8 * blocks 64-bit words) receives the shader clock cycles wavefront w of block b took, 0 for one
 * that had nothing to do. No counterpart in the reference. */
int32_t rmlk_hip_issue_yardstick(rmlk_stream_t stream, int32_t kind, int32_t second_wavefront,
                                 int32_t iterations, int32_t blocks, uint64_t *cycles);

/* Write up to 256 bytes from host memory `src` to device memory `dst`. The bytes travel as kernel
 * arguments: no staging copy, nothing to keep alive, recordable into a HIP graph.
 * ref: runtime/src/providers/cuda/backend/shape.rs:67-72 (host vector + H2D for tiny tensors). */
int32_t rmlk_hip_write_small(rmlk_stream_t stream, void *dst, const void *src, size_t bytes);

/* ---------------------------------------------------------------------------------------------
 * Memory and stream helpers (what the provider used cudarc for,
 * ref: runtime/src/providers/cuda/allocator.rs:96-139, data.rs:24-25, store.rs:385-416).
 * These DO call the HIP allocator / synchronise as named. */
int32_t rmlk_hip_malloc(void **ptr, size_t bytes);
int32_t rmlk_hip_free(void *ptr);
int32_t rmlk_hip_memcpy_htod(rmlk_stream_t stream, void *dst, const void *src, size_t bytes);
int32_t rmlk_hip_memcpy_dtoh(rmlk_stream_t stream, void *dst, const void *src, size_t bytes);
int32_t rmlk_hip_memcpy_dtod(rmlk_stream_t stream, void *dst, const void *src, size_t bytes);
/* n_copies device-to-device copies (dsts, srcs and bytes are HOST arrays), 32 per launch when all
 * of them have 16-byte aligned ends and lengths; one rmlk_hip_memcpy_dtod each otherwise. The cache
 * copies the layers of a decoder need when their cache inputs may not be overwritten are one launch. */
int32_t rmlk_hip_memcpy_dtod_many(rmlk_stream_t stream, int32_t n_copies, void *const *dsts,
                                  const void *const *srcs, const size_t *bytes);
int32_t rmlk_hip_memset(rmlk_stream_t stream, void *dst, int32_t byte, size_t bytes);
int32_t rmlk_hip_stream_sync(rmlk_stream_t stream);

typedef struct rmlk_device_info {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t lds_bytes_per_block;
    int32_t clock_khz;
    int64_t total_mem_bytes;
} rmlk_device_info;

int32_t rmlk_hip_device_info(int32_t device, rmlk_device_info *info);

/* Human-readable name of a status (static string). */
const char *rmlk_hip_status_string(int32_t status);

/* Library version, "major.minor.patch". */
const char *rmlk_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RMLK_HIP_H */
