// Host-side runtime above the kernel C ABI: tensors, the device buffer pool, graphs, sessions.
// C++ stand-in for the reference's provider layer (runtime/src/providers/cuda/*.rs) and for the
// sequential executor of runtime/src/core/instance.rs.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <map>
#include <deque>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../../include/rmlk_runtime.h"

namespace rmlk {
namespace rt {

// ---- errors -----------------------------------------------------------------------------------
struct RtError : std::runtime_error {
    int32_t code;
    RtError(int32_t c, const std::string &m) : std::runtime_error(m), code(c) {}
};

// Rust `Debug` spelling of schema::DataType, used in the two error texts that are API
// (runtime/src/core/error.rs:6,10,24-28).
const char *dtype_name(int32_t dt);
size_t dtype_size(int32_t dt);
[[noreturn]] void fail_unsupported(int32_t dt);
[[noreturn]] void fail_op(const std::string &msg);
void check_status(int32_t st, const char *where);
void check_hip(hipError_t e, const char *where);

// ---- device memory ----------------------------------------------------------------------------
// Caching pool: sizes are rounded to a bucket, freed blocks are kept per bucket and handed out
// again in LIFO order, so a run with the same shapes meets the same addresses again and never
// reaches hipMalloc after the first time. (The reference bumps inside two 4 KiB arenas and falls
// back to cuMemAlloc for almost every tensor, providers/cuda/allocator.rs:96-139.)
class Pool {
public:
    ~Pool();
    void *alloc(size_t bytes);
    void release(void *p, size_t bytes);
    static size_t bucket(size_t bytes);
    int64_t pool_bytes = 0;
    int64_t hip_mallocs = 0;
    bool forbid_malloc = false;  // set while a HIP graph is being captured
    // While the launches over tiny tensors of a run are being collected, the buffers such tensors
    // give back are kept aside until let_go(): handed out again at once, a buffer would make two
    // collected operators that have nothing to do with each other look dependent (one overwrites
    // what the other read), and they could not run side by side.
    bool hold_small = false;
    static constexpr size_t kSmallBytes = 8 * 1024;   // the largest output a collected operator has
    void let_go();

private:
    std::vector<std::pair<void *, size_t>> held_;
    std::map<size_t, std::vector<void *>> free_;
    std::vector<void *> all_;
};

struct Buffer {
    void *ptr = nullptr;
    size_t bytes = 0;
    Pool *pool = nullptr;   // null: memory the session does not own (bound by the caller)
    bool owned_raw = false; // hipMalloc'ed outside the pool (initializers)
    bool donated = false;   // an operator may overwrite it in place
    ~Buffer();
};
using BufferRef = std::shared_ptr<Buffer>;

// ---- small tensors mirrored on the host ---------------------------------------------------------
// Shape arithmetic (Shape -> Gather -> Concat -> Reshape ...) runs on the device like any other
// operator; operators additionally keep the VALUES of small integer tensors on the host when all
// their inputs are known there, so that a later Reshape / Slice / Expand / Range does not have to
// stall the stream with a device-to-host read (the reference reads back every time,
// e.g. backend/reshape.rs:102-103, backend/slice.rs:262-335).
constexpr int64_t kHostMirrorMax = 64;
struct HostVal {
    bool is_float = false;
    std::vector<int64_t> i;  // integer / bool values
    std::vector<double> f;   // floating values
    size_t size() const { return is_float ? f.size() : i.size(); }
    int64_t as_int(size_t k) const { return is_float ? static_cast<int64_t>(f[k]) : i[k]; }
    double as_double(size_t k) const { return is_float ? f[k] : static_cast<double>(i[k]); }
};

struct PendingNorm;
struct PendingProduct;

struct Tensor {
    int32_t dtype = 0;
    std::vector<int64_t> shape;
    BufferRef buf;
    size_t offset = 0;  // bytes into buf
    std::shared_ptr<HostVal> host;
    // Set on the result of a one-row RMSNorm that was NOT computed: the memory holds the row before
    // the norm, and the one consumer (a one-row product, which the fusion pass has checked) applies
    // the norm while it loads the row, or computes it first if it cannot.
    std::shared_ptr<const PendingNorm> pending_norm;
    // Set on the members of a one-row product over joint K-contiguous weights that was NOT computed
    // (and on views of them): the memory is reserved but not written. The fusion pass has checked
    // that everything that reads them is one row-stream node, which either runs the product and
    // its own work as one launch or has the product computed first.
    std::shared_ptr<PendingProduct> pending_product;
    // Set on the result of a many-row norm whose one reader is a product over bfloat16 weights on the
    // bf16 matrix cores: the same rows as three bfloat16 pieces (the planes rmlk_hip_bf16x3_split would
    // write), stored by the norm kernel itself.
    std::shared_ptr<const Tensor> pieces;

    bool defined() const { return dtype != 0; }
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        return n;
    }
    size_t nbytes() const { return static_cast<size_t>(numel()) * dtype_size(dtype); }
    void *data() const { return buf ? static_cast<char *>(buf->ptr) + offset : nullptr; }
    int rank() const { return static_cast<int>(shape.size()); }
    void reset() {
        dtype = 0;
        shape.clear();
        buf.reset();
        offset = 0;
        host.reset();
        pending_norm.reset();
        pending_product.reset();
        pieces.reset();
    }
};

struct PendingNorm {
    Tensor gamma;
    float eps = 0.f;
    int32_t reciprocal = 0;
};

struct PendingProduct {
    Tensor x;                                   // the input row (before `norm`, when there is one)
    std::shared_ptr<const PendingNorm> norm;    // null: x as it is
    Tensor wt;                                  // the joint weights, K-contiguous [total, k]
    Tensor row;                                 // where the product goes when it has to be stored
    int64_t k = 0, total = 0;
    bool computed = false;                      // stored in `row`, or consumed by the fused launch
    // Many rows (m > 0): the product HAS run, but its split-K partial sums were not added up -
    // `slabs` holds `splits` matrices [m, total], `slab` elements apart; `outs` are the members'
    // (dense, still unwritten) outputs in the order of their column blocks `widths`. The row-stream
    // node reads its rows from the slabs and adds them up on the way; `x` is kept for the case
    // that the members have to be written after all.
    int64_t m = 0;
    Tensor slabs;
    int32_t splits = 0;
    int64_t slab = 0;
    std::vector<int64_t> widths;
    std::vector<Tensor> outs;
};

rmlk_dims to_dims(const std::vector<int64_t> &v);          // rank-0 becomes [1]
std::vector<int64_t> dense_strides(const std::vector<int64_t> &shape);
int64_t normalize_axis(int64_t axis, int64_t rank, const char *what);

// ---- graph ------------------------------------------------------------------------------------
struct HostTensor {
    int32_t dtype = 0;
    std::vector<int64_t> shape;
    std::vector<uint8_t> data;
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        return n;
    }
};

struct Attr {
    enum Kind { Int, Float, Ints, Floats, String, TensorK } kind = Int;
    int64_t i = 0;
    float f = 0.f;
    std::vector<int64_t> ints;
    std::vector<float> floats;
    std::string s;
    HostTensor t;
};

struct Node {
    std::string op;
    std::vector<int> inputs;   // value ids, -1 = omitted optional input
    std::vector<int> outputs;
    std::unordered_map<std::string, Attr> attrs;
    std::vector<Node> body;    // fused nodes only: the nodes this one replaced, in graph order
};

struct Value {
    std::string name;
    int32_t dtype = 0;             // declared (0 = inferred at run time)
    std::vector<int64_t> shape;    // declared
    bool is_input = false, is_initializer = false, is_output = false;
    int producer = -1;             // node index
    HostTensor init;               // initializer payload
};

}  // namespace rt
}  // namespace rmlk

struct rmlk_graph {
    std::vector<rmlk::rt::Value> values;
    std::vector<rmlk::rt::Node> nodes;
    std::unordered_map<std::string, int> by_name;
    std::vector<int> inputs, outputs;
    int value_id(const std::string &name, bool create);
};

namespace rmlk {
namespace rt {

struct Session;

// What an operator sees (ref: runtime/src/core/context.rs:41-145).
struct OpContext {
    Session &session;
    const Node &node;
    int node_index;
    std::vector<Tensor *> in;   // nullptr for an omitted optional input
    std::vector<Tensor *> out;
    hipStream_t stream;
    // Tensors an op makes to stand in for an input (`in[i]` may point here): they live as long as
    // the context, which the executor still reads after the op has returned.
    std::deque<Tensor> temps;

    int n_inputs() const { return static_cast<int>(in.size()); }
    bool has_input(int i) const { return i < n_inputs() && in[i] && in[i]->defined(); }
    const Tensor &input(int i) const;
    // Allocate output i (dense) from the pool.
    Tensor &alloc_output(int i, int32_t dtype, const std::vector<int64_t> &shape);
    // Output i shares the memory of `src` with a new shape (Reshape, Unsqueeze).
    Tensor &view_output(int i, const Tensor &src, const std::vector<int64_t> &shape);

    const Attr *attr(const char *name) const;
    int64_t attr_int(const char *name, int64_t dflt) const;
    std::vector<int64_t> attr_ints(const char *name, bool *present = nullptr) const;
    std::string attr_string(const char *name, const std::string &dflt) const;

    // Values of a small integer / float input on the host: the mirror when present, otherwise a
    // blocking device-to-host copy (counted in the session's sync statistics).
    HostVal host_values(int i) const;
    int32_t *error_flag() const;
    // The session's MatMul workspace (split-K partials): one persistent buffer, grown on demand.
    void *scratch(size_t bytes) const;
};

using OpFn = void (*)(OpContext &);
OpFn find_op(const std::string &name);

// Pattern fusion (fusion.cpp): rewrites session.graph_copy.nodes, returns the number of fused nodes.
int fuse_patterns(Session &s);
void op_fused_rmsnorm(OpContext &c);
void op_fused_swiglu(OpContext &c);
void op_fused_add_rmsnorm(OpContext &c);
void op_fused_softmax(OpContext &c);
void op_fused_rotary(OpContext &c);
void op_fused_head_rows(OpContext &c);
// ScatterND's output: the data tensor itself where it may be updated in place, else a copy of it
Tensor &scatter_destination(OpContext &c, int data_index, int out_index, bool *copy_left_to_caller = nullptr);
void op_fused_attn_matmul(OpContext &c);
void op_fused_attention(OpContext &c);
void op_fused_matmul_add_rmsnorm(OpContext &c);
void op_fused_matmul_const(OpContext &c);
void op_fused_matmul_group(OpContext &c);
void op_fused_matmul_group_swiglu(OpContext &c);

struct CapturedPlan {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<Tensor> pinned;  // every value alive at the end of the captured run
    ~CapturedPlan();
};

struct Session {
    const rmlk_graph *g = nullptr;  // copied at creation
    rmlk_graph graph_copy;
    int device = 0;
    hipStream_t stream = nullptr;
    Pool pool;
    std::vector<Tensor> values;      // by value id
    std::vector<int> last_use;       // node index of the last consumer, -1 = never read
    std::vector<BufferRef> scratch_bufs;
    void *workspace = nullptr;       // persistent MatMul workspace (raw allocation)
    size_t workspace_bytes = 0;
    int32_t *err_flag = nullptr;     // device
    // Block counters of kernels whose last block finishes the job (the decode-step attention):
    // zero when the session is built, and left zero by every kernel that uses them.
    static constexpr int64_t kBlockCounters = 1024;
    int32_t *block_counters = nullptr;
    int32_t *err_host = nullptr;     // pinned host
    // The attention kernel's map of the (query tile, key chunk) pairs a mask leaves visible, made by
    // the first attention node of a run that reads a mask and used by the later ones that read the
    // same value with the same sizes (the layers of a model share their mask); dropped when the run ends.
    struct AttentionMap {
        int mask_value = -1;           // graph value id of the mask
        int64_t sizes[6] = {0, 0, 0, 0, 0, 0};   // batch, kv heads, rep, q_len, kv_len, head dim
        rmlk_dims strides{};
        Tensor map;
    } attention_map;
    // A ScatterND destination that has to be a copy of a graph input (a cache input the caller did
    // not donate) depends on nothing the run computes: all such copies go out as ONE launch in front
    // of the first node, and the nodes find them here. `scatter_inputs` lists (node index, value id)
    // of every place where a graph input is the data of a ScatterND; found when the session is built.
    std::vector<std::pair<int, int>> scatter_inputs;
    std::multimap<std::pair<int, int>, Tensor> early_copies;
    void copy_scatter_inputs_early();
    bool capturing = false;
    bool profiling = false;
    bool fuse = true;                // form fused nodes while building
    int32_t weight_storage = RMLK_FLOAT;   // how the K-contiguous copies of constant weights are held
    bool lossless_16bit = true;            // float storage gives way to 16 bits where no value changes
    int weights_16bit = 0;                 // weight matrices held as 16-bit values
    bool bf16_pieces = false;              // many-row products over bfloat16 weights on the bf16 matrix cores
    int products_bf16_pieces = 0;          // products the last run multiplied that way
    int fused_nodes = 0;
    int folded_nodes = 0;            // constant nodes evaluated while building
    int64_t device_syncs = 0;            // blocking reads of shape-like tensors
    int64_t device_syncs_workspace = 0;  // stream syncs taken to grow the MatMul workspace
    std::unique_ptr<CapturedPlan> plan;
    struct NodeStat {
        double micros = -1.0, bytes = 0.0, flops = 0.0;
        hipEvent_t e0 = nullptr, e1 = nullptr;
    };
    std::vector<NodeStat> stats;

    ~Session();
    void build(const rmlk_graph &graph, int dev);
    void run_nodes();
    void run();
    void capture();
    void replay();
    void replay_enqueue();           // the recorded graph launched, nothing awaited
    void check_error_flag();
};

}  // namespace rt
}  // namespace rmlk

// Sets the calling thread's rmlk_last_error() text (for code outside c_api.cpp).
extern "C" void rmlk_set_last_error(const char *message);

struct rmlk_session {
    rmlk::rt::Session impl;
};
