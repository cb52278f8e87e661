/*
 * rmlk_runtime.h -- C ABI of the host side that sits above the kernels of rmlk_hip.h: the graph
 * builder, the operator dispatch and the sequential executor. It is the C++ stand-in for the
 * reference's Rust layers on this path (no Rust toolchain ships with this build):
 *
 *   rmlk_graph_*    <->  schema::GraphBuilder             (ref: schema/src/builder.rs:49-260)
 *   rmlk_session_*  <->  runtime::Builder / ModelInstance (ref: runtime/src/core/instance.rs:89-222)
 *   operator table  <->  CudaKernel / OperationBackend    (ref: runtime/src/providers/cuda/backend/mod.rs:82-162)
 *
 * Every function returns 0 on success or a negative rmlk_status / positive hipError_t; the text of
 * the last error of the calling thread is kept for rmlk_last_error(). Two texts are API, as in the
 * reference (ref: runtime/src/core/error.rs:6,10): an unsupported element type reports a message
 * that starts with "unsupported data type", an unsupported Cast pair one that starts with
 * "unsupported cast".
 */
#ifndef RMLK_RUNTIME_H
#define RMLK_RUNTIME_H

#include "rmlk_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rmlk_graph rmlk_graph;
typedef struct rmlk_session rmlk_session;

#define RMLK_ERR_GRAPH (-20)   /* graph construction error (duplicate / unknown name ...) */
#define RMLK_ERR_OP (-21)      /* an operator rejected its inputs (shape, attribute, dtype) */
#define RMLK_ERR_KERNEL (-22)  /* a kernel raised its device error flag (index out of range) */

const char *rmlk_last_error(void);

/* ---- graph building (ref: schema/src/builder.rs) ------------------------------------------- */
int32_t rmlk_graph_create(rmlk_graph **out);
void rmlk_graph_destroy(rmlk_graph *g);

/* Graph input. dims may hold 0 for a dim only known at run time. ref: builder.rs:66-77 */
int32_t rmlk_graph_input(rmlk_graph *g, const char *name, int32_t dtype, const int64_t *dims,
                         int32_t rank);
/* Initializer: `data` (host, dense, prod(dims) elements of dtype) is copied. ref: builder.rs:83-96 */
int32_t rmlk_graph_constant(rmlk_graph *g, const char *name, int32_t dtype, const int64_t *dims,
                            int32_t rank, const void *data);
/* Append an operator node; `op` is the ONNX operator name ("MatMul", "ScatterND", ...). Inputs
 * may be "" for an omitted optional input. Output values are declared implicitly.
 * Returns the node index (>= 0) or an error (< 0). ref: builder.rs:128-190 */
int32_t rmlk_graph_op(rmlk_graph *g, const char *op, const char *const *inputs, int32_t n_inputs,
                      const char *const *outputs, int32_t n_outputs);
/* Attributes of node `node` (ref: schema/src/attributes.rs AttributeType::{Int,Float,Ints,Floats,String,Tensor}) */
int32_t rmlk_graph_attr_int(rmlk_graph *g, int32_t node, const char *name, int64_t value);
int32_t rmlk_graph_attr_float(rmlk_graph *g, int32_t node, const char *name, float value);
int32_t rmlk_graph_attr_ints(rmlk_graph *g, int32_t node, const char *name, const int64_t *values,
                             int32_t n);
int32_t rmlk_graph_attr_floats(rmlk_graph *g, int32_t node, const char *name, const float *values,
                               int32_t n);
int32_t rmlk_graph_attr_string(rmlk_graph *g, int32_t node, const char *name, const char *value);
int32_t rmlk_graph_attr_tensor(rmlk_graph *g, int32_t node, const char *name, int32_t dtype,
                               const int64_t *dims, int32_t rank, const void *data);
/* Mark a value as graph output. ref: builder.rs:192-204 */
int32_t rmlk_graph_output(rmlk_graph *g, const char *name);

/* ---- ONNX files -------------------------------------------------------------------------------- */
/* Build a graph from the bytes of an ONNX ModelProto (protobuf wire format). Follows the
 * reference's importer: initializers first, then graph inputs (an input that shares its name with
 * an initializer is a defaulted input: the constant stays), outputs, then the nodes in stored
 * order; a symbolic or missing dim is dynamic (0); tensor payloads from raw_data, the typed
 * repeated fields, or an external file (keys location / offset / length) resolved against
 * `base_dir` (NULL or "": the working directory). Subgraph attributes, sparse and string tensors
 * and non-tensor value types are rejected.
 * ref: schema/src/onnx_import/transform.rs:76-260 (graph_from_onnx_bytes),
 *      schema/src/onnx_import/traverse.rs:33-60, schema/src/tensor.rs:149-300 */
int32_t rmlk_graph_load_onnx(const void *bytes, size_t size, const char *base_dir, rmlk_graph **out);
/* The same from a file; external data is looked up next to it.
 * ref: Builder::from_onnx_path, runtime/src/core/instance.rs:187-196 */
int32_t rmlk_graph_load_onnx_file(const char *path, rmlk_graph **out);
/* JSON text of a graph (inputs, initializers with an FNV-1a hash of their bytes, nodes with
 * attributes, outputs), for tools and tests. Writes at most `size` bytes including the
 * terminator; returns the length needed. */
int64_t rmlk_graph_describe(const rmlk_graph *g, char *buf, int64_t size);

/* ---- sessions (ref: runtime/src/core/instance.rs) ------------------------------------------- */
/* Validates the graph, uploads the initializers to `device`, creates the stream.
 * ref: Builder::build, instance.rs:198-221 and TensorStore::init, providers/cuda/store.rs:95-261 */
int32_t rmlk_session_create(const rmlk_graph *g, int32_t device, rmlk_session **out);
/* The same with option flags. By default a session replaces four chains of small nodes that
 * decoder graphs repeat per layer (decomposed RMSNorm, rotary embedding, SwiGLU, scale + mask +
 * softmax) by single nodes backed by fused kernels with identical rounding;
 * RMLK_SESSION_NO_FUSION keeps one kernel per ONNX node as the reference executes it
 * (runtime/src/core/instance.rs:25-37). rmlk_session_create passes flags = 0. */
#define RMLK_SESSION_NO_FUSION 1u
/* Constant 2-D weights that only MatMuls of fused nodes read are stored as IEEE half or bfloat16
 * values (rounded to nearest even once, while the session is built) instead of floats: half the
 * bytes per decode step, half the device memory. Activations, accumulation and every other tensor
 * stay fp32; the results are those of the same session over a graph whose weights were rounded
 * beforehand (many-row products bit for bit, one-row products to rounding). At most one of the two;
 * ignored with RMLK_SESSION_NO_FUSION. Off by default: the reference computes in fp32 only. */
#define RMLK_SESSION_WEIGHTS_F16 2u
#define RMLK_SESSION_WEIGHTS_BF16 4u
/* Without either of them a session still holds such a weight matrix as 16-bit values when that loses
 * nothing: when every one of its floats is a bfloat16 (or half) value already, as in a checkpoint
 * trained in bfloat16 and exported as float. The products then multiply exactly the numbers of the
 * graph (many-row products bit for bit as over float storage, one-row products with their sums in
 * another order) from half the bytes. RMLK_SESSION_WEIGHTS_F32 keeps float storage regardless. */
#define RMLK_SESSION_WEIGHTS_F32 8u
/* Products of many rows (64 and more) over weight matrices held as bfloat16 values run on the bf16
 * matrix cores: the fp32 first operand is split into three bfloat16 pieces whose sum it is exactly,
 * every product of a piece and a weight is exact in fp32, accumulation is fp32
 * (rmlk_hip_matmul_bf16x3). The results are fp32 products with their sums in another order - not
 * the bits of the fp32 MFMA kernels - at about 2.5x their rate. Concerns prefill over checkpoints
 * whose floats are bfloat16 values (stored in 16 bits without loss by default) or over
 * RMLK_SESSION_WEIGHTS_BF16; one-row products (decode) are unchanged. Off by default. */
#define RMLK_SESSION_BF16_PIECES 16u
int32_t rmlk_session_create_ex(const rmlk_graph *g, int32_t device, uint32_t flags,
                               rmlk_session **out);
/* Number of products the session's last run multiplied that way. */
int32_t rmlk_session_products_bf16_pieces(const rmlk_session *s);
/* Number of fused nodes the session formed while it was built. */
int32_t rmlk_session_fused_nodes(const rmlk_session *s);
/* Number of constant weight matrices the session holds as 16-bit values. */
int32_t rmlk_session_weights_16bit(const rmlk_session *s);
void rmlk_session_destroy(rmlk_session *s);

/* Feed a graph input from host memory (copied to a session-owned device buffer, H2D on the
 * session stream). ref: ExecutionState::load_value, core/execution_state.rs:117-196 */
int32_t rmlk_session_set_input(rmlk_session *s, const char *name, int32_t dtype,
                               const int64_t *dims, int32_t rank, const void *host_data);
/* Feed a graph input from device memory the caller owns (no copy; must stay valid until the run
 * has finished). With `donate` != 0 an operator may update the buffer in place (ScatterND writing
 * one row of a KV cache) instead of copying it first. */
int32_t rmlk_session_bind_input(rmlk_session *s, const char *name, int32_t dtype,
                                const int64_t *dims, int32_t rank, void *device_data,
                                int32_t donate);
/* Use output `out_name` of the previous run as input `in_name` of the next one without leaving
 * the device (the reference's example round-trips every present.* through the host,
 * ref: runtime/examples/llama.rs:96-117). */
int32_t rmlk_session_feed_output(rmlk_session *s, const char *out_name, const char *in_name);

/* Execute all nodes in stored order on the session stream; returns when everything is enqueued
 * and the kernels' error flags have been checked (one small D2H at the end of the run).
 * ref: ModelInstance::run, instance.rs:89-119 */
int32_t rmlk_session_run(rmlk_session *s);

/* Shape / dtype / device pointer of a graph output after a run. dims must hold RMLK_MAX_RANK. */
int32_t rmlk_session_output_info(rmlk_session *s, const char *name, int32_t *dtype, int64_t *dims,
                                 int32_t *rank, void **device_data);
/* Blocking copy of a graph output to host memory (`bytes` must equal the output's size).
 * ref: ExecutionState::get_value, core/execution_state.rs:201-225 */
int32_t rmlk_session_read_output(rmlk_session *s, const char *name, void *host_data,
                                 size_t bytes);

/* Record the run for the current input shapes into a HIP graph, then replay it with
 * rmlk_session_replay (inputs are re-read from the same buffers; set_input with unchanged shapes
 * refreshes them in place). Needs one plain rmlk_session_run with the same shapes first. Shapes
 * must not depend on input VALUES between replays. */
int32_t rmlk_session_capture(rmlk_session *s);
int32_t rmlk_session_replay(rmlk_session *s);
/* rmlk_session_replay in two halves, for a caller that keeps the GPU fed: _replay_enqueue launches
 * the recorded graph and returns without waiting (several may be enqueued back to back; each reads
 * the inputs as they are when it executes), _check waits for the session's stream and reports a
 * kernel failure (an index out of range) of any run or replay since the last report - the
 * kernels' error flag stays set until it has been reported. rmlk_session_replay is one of each.
 * No counterpart in the reference, whose ModelInstance::run (instance.rs:89-119) is synchronous. */
int32_t rmlk_session_replay_enqueue(rmlk_session *s);
int32_t rmlk_session_check(rmlk_session *s);

int32_t rmlk_session_sync(rmlk_session *s);
/* hipStream_t the session enqueues on */
rmlk_stream_t rmlk_session_stream(rmlk_session *s);

/* Per-node timing of the next runs with HIP events on the session stream (0 = off).
 * rmlk_session_node_count / node_info describe node i: ONNX op name, last duration in
 * microseconds (negative when not timed), bytes read + written and floating-point operations the
 * operator's definition implies for the shapes of the last run. */
int32_t rmlk_session_set_profiling(rmlk_session *s, int32_t enabled);
int32_t rmlk_session_node_count(rmlk_session *s);
int32_t rmlk_session_node_info(rmlk_session *s, int32_t node, const char **op, double *micros,
                               double *bytes, double *flops);

/* Device bytes the session's buffer pool holds, and how many times it went to the HIP
 * allocator (steady state: a run allocates nothing new). */
int32_t rmlk_session_memory_stats(rmlk_session *s, int64_t *pool_bytes, int64_t *hip_mallocs,
                                  int64_t *device_syncs);

#ifdef __cplusplus
}
#endif
#endif /* RMLK_RUNTIME_H */
