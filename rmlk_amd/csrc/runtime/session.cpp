// Sessions: initializer upload, the sequential executor, the buffer pool and HIP-graph replay.
// Mirrors Builder::build / ModelInstance::run of the reference (runtime/src/core/instance.rs:89-222)
// and its ExecutionState / TensorStore (runtime/src/core/execution_state.rs, providers/cuda/store.rs).
#include <algorithm>
#include <cstdio>

#include "core.hpp"

namespace rmlk {
namespace rt {

// ---- small helpers ----------------------------------------------------------------------------
const char *dtype_name(int32_t dt) {
    switch (dt) {
        case RMLK_FLOAT: return "Float";
        case RMLK_UINT8: return "Uint8";
        case RMLK_INT8: return "Int8";
        case RMLK_UINT16: return "Uint16";
        case RMLK_INT16: return "Int16";
        case RMLK_INT32: return "Int32";
        case RMLK_INT64: return "Int64";
        case RMLK_BOOL: return "Bool";
        case RMLK_FLOAT16: return "Float16";
        case RMLK_DOUBLE: return "Double";
        case RMLK_UINT32: return "Uint32";
        case RMLK_UINT64: return "Uint64";
        case 8: return "String";
        default: return "Undefined";
    }
}

size_t dtype_size(int32_t dt) {
    switch (dt) {
        case RMLK_BOOL: case RMLK_UINT8: case RMLK_INT8: return 1;
        case RMLK_UINT16: case RMLK_INT16: case RMLK_FLOAT16: case RMLK_BFLOAT16: return 2;
        case RMLK_FLOAT: case RMLK_INT32: case RMLK_UINT32: return 4;
        case RMLK_DOUBLE: case RMLK_INT64: case RMLK_UINT64: return 8;
        default: return 0;
    }
}

void fail_unsupported(int32_t dt) {
    throw RtError(RMLK_ERR_UNSUPPORTED, std::string("unsupported data type: ") + dtype_name(dt));
}
void fail_op(const std::string &msg) { throw RtError(RMLK_ERR_OP, msg); }

void check_status(int32_t st, const char *where) {
    if (st == 0) return;
    if (st == RMLK_ERR_UNSUPPORTED)
        throw RtError(st, std::string("unsupported data type in ") + where);
    throw RtError(st, std::string(where) + ": " + rmlk_hip_status_string(st));
}
void check_hip(hipError_t e, const char *where) {
    if (e != hipSuccess)
        throw RtError(static_cast<int32_t>(e), std::string(where) + ": " + hipGetErrorString(e));
}

rmlk_dims to_dims(const std::vector<int64_t> &v) {
    if (v.size() > RMLK_MAX_RANK) throw RtError(RMLK_ERR_BAD_RANK, "rank above 8");
    rmlk_dims d;
    std::memset(&d, 0, sizeof(d));
    if (v.empty()) {
        d.rank = 1;
        d.v[0] = 1;
        return d;
    }
    d.rank = static_cast<int32_t>(v.size());
    for (size_t i = 0; i < v.size(); ++i) d.v[i] = v[i];
    return d;
}

std::vector<int64_t> dense_strides(const std::vector<int64_t> &shape) {
    std::vector<int64_t> st(shape.size());
    int64_t s = 1;
    for (int d = static_cast<int>(shape.size()) - 1; d >= 0; --d) {
        st[d] = s;
        s *= shape[d];
    }
    return st;
}

// ref: runtime/src/utils/mod.rs:155-175; index == size is rejected (the reference accepts it)
int64_t normalize_axis(int64_t axis, int64_t rank, const char *what) {
    int64_t a = axis < 0 ? axis + rank : axis;
    if (a < 0 || a >= rank)
        fail_op(std::string(what) + " " + std::to_string(axis) + " out of range for rank " +
                std::to_string(rank));
    return a;
}

// ---- pool -------------------------------------------------------------------------------------
size_t Pool::bucket(size_t bytes) {
    if (bytes <= 256) return 256;
    if (bytes <= (1u << 20)) {  // powers of two up to 1 MiB
        size_t b = 256;
        while (b < bytes) b <<= 1;
        return b;
    }
    const size_t q = 1u << 20;  // then multiples of 1 MiB
    return (bytes + q - 1) / q * q;
}

void *Pool::alloc(size_t bytes) {
    const size_t b = bucket(bytes);
    auto it = free_.find(b);
    if (it != free_.end() && !it->second.empty()) {
        void *p = it->second.back();
        it->second.pop_back();
        return p;
    }
    if (forbid_malloc)
        throw RtError(RMLK_ERR_OP, "buffer pool miss while recording a HIP graph");
    void *p = nullptr;
    check_hip(hipMalloc(&p, b), "hipMalloc");
    all_.push_back(p);
    pool_bytes += static_cast<int64_t>(b);
    ++hip_mallocs;
    return p;
}

void Pool::release(void *p, size_t bytes) {
    const size_t b = bucket(bytes);
    if (hold_small && b <= kSmallBytes) held_.emplace_back(p, b);
    else free_[b].push_back(p);
}

void Pool::let_go() {
    for (const auto &h : held_) free_[h.second].push_back(h.first);
    held_.clear();
}

Pool::~Pool() {
    for (void *p : all_) (void)hipFree(p);
}

Buffer::~Buffer() {
    if (!ptr) return;
    if (pool) pool->release(ptr, bytes);
    else if (owned_raw) (void)hipFree(ptr);
}

CapturedPlan::~CapturedPlan() {
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
}

// ---- operator context -------------------------------------------------------------------------
const Tensor &OpContext::input(int i) const {
    if (!has_input(i)) fail_op(node.op + ": missing input " + std::to_string(i));
    return *in[i];
}

Tensor &OpContext::alloc_output(int i, int32_t dtype, const std::vector<int64_t> &shape) {
    if (i >= static_cast<int>(out.size()) || !out[i]) fail_op(node.op + ": missing output");
    if (shape.size() > RMLK_MAX_RANK) throw RtError(RMLK_ERR_BAD_RANK, "rank above 8");
    Tensor &t = *out[i];
    t.reset();
    t.dtype = dtype;
    t.shape = shape;
    for (int64_t d : shape)
        if (d < 0) fail_op(node.op + ": negative output dim");
    size_t bytes = t.nbytes();
    auto b = std::make_shared<Buffer>();
    b->bytes = bytes ? bytes : 1;
    b->pool = &session.pool;
    b->ptr = session.pool.alloc(b->bytes);
    t.buf = b;
    return t;
}

Tensor &OpContext::view_output(int i, const Tensor &src, const std::vector<int64_t> &shape) {
    if (i >= static_cast<int>(out.size()) || !out[i]) fail_op(node.op + ": missing output");
    Tensor v;
    v.dtype = src.dtype;
    v.shape = shape;
    v.buf = src.buf;
    v.offset = src.offset;
    v.pending_product = src.pending_product;   // a view of a product not computed yet is not computed either
    v.pieces = src.pieces;                     // (the same dense elements in the same order)
    *out[i] = v;
    return *out[i];
}

const Attr *OpContext::attr(const char *name) const {
    auto it = node.attrs.find(name);
    return it == node.attrs.end() ? nullptr : &it->second;
}
int64_t OpContext::attr_int(const char *name, int64_t dflt) const {
    const Attr *a = attr(name);
    return a ? a->i : dflt;
}
std::vector<int64_t> OpContext::attr_ints(const char *name, bool *present) const {
    const Attr *a = attr(name);
    if (present) *present = a != nullptr;
    return a ? a->ints : std::vector<int64_t>();
}
std::string OpContext::attr_string(const char *name, const std::string &dflt) const {
    const Attr *a = attr(name);
    return a ? a->s : dflt;
}

// Element types decode_host reads (integers, bool, float, double): only those get host mirrors.
static bool host_decodable(int32_t dtype) {
    switch (dtype) {
        case RMLK_FLOAT: case RMLK_DOUBLE: case RMLK_INT64: case RMLK_UINT64: case RMLK_INT32:
        case RMLK_UINT32: case RMLK_INT16: case RMLK_UINT16: case RMLK_INT8: case RMLK_UINT8:
        case RMLK_BOOL: return true;
        default: return false;
    }
}

static HostVal decode_host(int32_t dtype, const uint8_t *p, size_t n) {
    HostVal h;
    switch (dtype) {
        case RMLK_FLOAT: h.is_float = true; for (size_t k = 0; k < n; ++k) { float v; std::memcpy(&v, p + 4 * k, 4); h.f.push_back(v); } break;
        case RMLK_DOUBLE: h.is_float = true; for (size_t k = 0; k < n; ++k) { double v; std::memcpy(&v, p + 8 * k, 8); h.f.push_back(v); } break;
        case RMLK_INT64: case RMLK_UINT64: for (size_t k = 0; k < n; ++k) { int64_t v; std::memcpy(&v, p + 8 * k, 8); h.i.push_back(v); } break;
        case RMLK_INT32: for (size_t k = 0; k < n; ++k) { int32_t v; std::memcpy(&v, p + 4 * k, 4); h.i.push_back(v); } break;
        case RMLK_UINT32: for (size_t k = 0; k < n; ++k) { uint32_t v; std::memcpy(&v, p + 4 * k, 4); h.i.push_back(v); } break;
        case RMLK_INT16: for (size_t k = 0; k < n; ++k) { int16_t v; std::memcpy(&v, p + 2 * k, 2); h.i.push_back(v); } break;
        case RMLK_UINT16: for (size_t k = 0; k < n; ++k) { uint16_t v; std::memcpy(&v, p + 2 * k, 2); h.i.push_back(v); } break;
        case RMLK_INT8: for (size_t k = 0; k < n; ++k) h.i.push_back(static_cast<int8_t>(p[k])); break;
        case RMLK_UINT8: for (size_t k = 0; k < n; ++k) h.i.push_back(p[k]); break;
        case RMLK_BOOL: for (size_t k = 0; k < n; ++k) h.i.push_back(p[k] != 0); break;
        default: fail_unsupported(dtype);
    }
    return h;
}

HostVal OpContext::host_values(int i) const {
    const Tensor &t = input(i);
    if (t.host) return *t.host;
    // the reference's path: blocking device-to-host read (e.g. backend/slice.rs:262-335)
    if (session.capturing)
        fail_op(node.op + ": input " + std::to_string(i) +
                " must be known on the host to record a HIP graph (it depends on input values)");
    const size_t n = static_cast<size_t>(t.numel());
    if (n > (1u << 20)) fail_op(node.op + ": shape-like input is too large");
    std::vector<uint8_t> tmp(t.nbytes());
    if (!tmp.empty()) {
        check_status(rmlk_hip_batch_flush(stream), "collected launches");   // (what wrote t may still be collected)
        check_hip(hipMemcpyAsync(tmp.data(), t.data(), tmp.size(), hipMemcpyDeviceToHost, stream),
                  "hipMemcpyAsync D2H");
        check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
        ++session.device_syncs;
    }
    return decode_host(t.dtype, tmp.data(), n);
}

int32_t *OpContext::error_flag() const { return session.err_flag; }

void *OpContext::scratch(size_t bytes) const {
    Session &ss = session;
    if (bytes <= ss.workspace_bytes) return ss.workspace;
    if (ss.capturing)
        throw RtError(RMLK_ERR_OP, "MatMul workspace would grow while recording a HIP graph");
    // grow: nothing that uses the old buffer is still queued behind this point of the stream
    // once it is synchronised
    check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    ++ss.device_syncs_workspace;
    if (ss.workspace) check_hip(hipFree(ss.workspace), "hipFree");
    ss.workspace = nullptr;
    size_t want = bytes + bytes / 4;
    check_hip(hipMalloc(&ss.workspace, want), "hipMalloc (workspace)");
    ss.workspace_bytes = want;
    ++ss.pool.hip_mallocs;
    return ss.workspace;
}

// ---- session ----------------------------------------------------------------------------------
Session::~Session() {
    plan.reset();
    for (auto &st : stats) {
        if (st.e0) (void)hipEventDestroy(st.e0);
        if (st.e1) (void)hipEventDestroy(st.e1);
    }
    values.clear();
    scratch_bufs.clear();
    if (workspace) (void)hipFree(workspace);
    if (err_flag) (void)hipFree(err_flag);
    if (block_counters) (void)hipFree(block_counters);
    if (err_host) (void)hipHostFree(err_host);
    if (stream) (void)hipStreamDestroy(stream);
}

static Tensor upload_initializer(const HostTensor &ht, hipStream_t stream) {
    Tensor t;
    t.dtype = ht.dtype;
    t.shape = ht.shape;
    auto b = std::make_shared<Buffer>();
    b->bytes = ht.data.size() ? ht.data.size() : 1;
    b->owned_raw = true;
    check_hip(hipMalloc(&b->ptr, b->bytes), "hipMalloc (initializer)");
    if (!ht.data.empty())
        check_hip(hipMemcpyAsync(b->ptr, ht.data.data(), ht.data.size(), hipMemcpyHostToDevice,
                                 stream),
                  "hipMemcpyAsync H2D (initializer)");
    t.buf = b;
    if (ht.numel() <= kHostMirrorMax && host_decodable(ht.dtype))
        t.host = std::make_shared<HostVal>(
            decode_host(ht.dtype, ht.data.data(), static_cast<size_t>(ht.numel())));
    return t;
}

// Evaluate, once, the nodes whose inputs are all initializers (exported graphs compute Expand /
// Reshape targets and masks from constants through ConstantOfShape, Mul, Equal, Where ...): their
// outputs become initializers, with host mirrors where small, and the nodes leave the list. Nodes
// that produce a graph output, more than 1 MiB, or an error now are left for run time.
static int fold_constants(Session &s) {
    rmlk_graph &g = s.graph_copy;
    std::vector<bool> drop(g.nodes.size(), false);
    int folded = 0;
    for (size_t n = 0; n < g.nodes.size(); ++n) {
        const Node &node = g.nodes[n];
        if (node.op == "Constant") {   // already materialised by build()
            drop[n] = true;
            continue;
        }
        // Gather / ScatterND report bad indices through the device flag of a run: not folded
        if (node.op == "Gather" || node.op == "ScatterND") continue;
        bool constant = false;
        for (int v : node.inputs) {
            if (v < 0) continue;
            constant = g.values[v].is_initializer && s.values[v].defined();
            if (!constant) break;
        }
        for (int v : node.outputs)
            if (g.values[v].is_output) constant = false;
        if (!constant) continue;
        OpContext ctx{s, node, static_cast<int>(n), {}, {}, s.stream};
        for (int v : node.inputs) ctx.in.push_back(v < 0 ? nullptr : &s.values[v]);
        std::vector<Tensor> outs(node.outputs.size());
        for (size_t o = 0; o < outs.size(); ++o) ctx.out.push_back(&outs[o]);
        try {
            find_op(node.op)(ctx);
        } catch (const RtError &) {
            continue;
        }
        bool small = true;
        for (const Tensor &t : outs)
            if (!t.defined() || t.nbytes() > (1u << 20)) small = false;
        if (!small) continue;
        for (size_t o = 0; o < outs.size(); ++o) {
            s.values[node.outputs[o]] = outs[o];
            g.values[node.outputs[o]].is_initializer = true;
        }
        drop[n] = true;
        ++folded;
    }
    check_hip(hipStreamSynchronize(s.stream), "hipStreamSynchronize");
    s.scratch_bufs.clear();
    std::vector<Node> kept;
    for (size_t n = 0; n < g.nodes.size(); ++n)
        if (!drop[n]) kept.push_back(std::move(g.nodes[n]));
    g.nodes = std::move(kept);
    for (Value &v : g.values) v.producer = -1;
    for (size_t n = 0; n < g.nodes.size(); ++n)
        for (int v : g.nodes[n].outputs) g.values[v].producer = static_cast<int>(n);
    return folded;
}

void Session::build(const rmlk_graph &graph, int dev) {
    graph_copy = graph;
    g = &graph_copy;
    device = dev;
    check_hip(hipSetDevice(dev), "hipSetDevice");
    check_hip(hipStreamCreate(&stream), "hipStreamCreate");  // default priority
    check_hip(hipMalloc(reinterpret_cast<void **>(&err_flag), sizeof(int32_t)), "hipMalloc");
    check_hip(hipMemset(err_flag, 0, sizeof(int32_t)), "hipMemset");
    check_hip(hipHostMalloc(reinterpret_cast<void **>(&err_host), sizeof(int32_t)), "hipHostMalloc");
    *err_host = 0;
    check_hip(hipMalloc(reinterpret_cast<void **>(&block_counters), kBlockCounters * sizeof(int32_t)), "hipMalloc");
    check_hip(hipMemset(block_counters, 0, kBlockCounters * sizeof(int32_t)), "hipMemset");
    if (g->outputs.empty()) throw RtError(RMLK_ERR_GRAPH, "graph has no outputs");
    values.assign(g->values.size(), Tensor());
    for (size_t n = 0; n < g->nodes.size(); ++n) {
        const Node &node = g->nodes[n];
        if (!find_op(node.op) || node.op.rfind("rmlk.", 0) == 0)
            throw RtError(RMLK_ERR_OP, "unsupported operator `" + node.op + "`");
        for (int v : node.inputs) {
            if (v < 0) continue;
            const Value &val = g->values[v];
            if (!val.is_input && !val.is_initializer && (val.producer < 0 || val.producer >= static_cast<int>(n)))
                throw RtError(RMLK_ERR_GRAPH, "node " + std::to_string(n) + " (" + node.op +
                                                  ") reads `" + val.name +
                                                  "` before anything produces it");
        }
    }
    for (int o : g->outputs) {
        const Value &val = g->values[o];
        if (!val.is_input && !val.is_initializer && val.producer < 0)
            throw RtError(RMLK_ERR_GRAPH, "output `" + val.name + "` is not produced by any op");
    }
    // initializers, and the outputs of Constant nodes, live on the device for the session's life
    // (ref: TensorStore::init, providers/cuda/store.rs:95-261)
    for (size_t v = 0; v < g->values.size(); ++v)
        if (g->values[v].is_initializer) values[v] = upload_initializer(g->values[v].init, stream);
    check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    // the host copies of large initializers are not needed once they are on the device
    for (size_t v = 0; v < graph_copy.values.size(); ++v)
        if (graph_copy.values[v].is_initializer && graph_copy.values[v].init.data.size() > 4096)
            std::vector<uint8_t>().swap(graph_copy.values[v].init.data);
    for (size_t n = 0; n < g->nodes.size(); ++n) {
        const Node &node = g->nodes[n];
        if (node.op != "Constant") continue;
        // value / value_float(s) / value_int(s) forms, ref: backend/constant.rs
        HostTensor ht;
        auto put = [&](int32_t dt, std::vector<int64_t> shape, const void *p, size_t bytes) {
            ht.dtype = dt;
            ht.shape = std::move(shape);
            ht.data.assign(static_cast<const uint8_t *>(p), static_cast<const uint8_t *>(p) + bytes);
        };
        auto it = node.attrs.find("value");
        if (it != node.attrs.end() && it->second.kind == Attr::TensorK) {
            ht = it->second.t;
        } else if ((it = node.attrs.find("value_float")) != node.attrs.end()) {
            put(RMLK_FLOAT, {}, &it->second.f, 4);
        } else if ((it = node.attrs.find("value_floats")) != node.attrs.end()) {
            put(RMLK_FLOAT, {static_cast<int64_t>(it->second.floats.size())},
                it->second.floats.data(), it->second.floats.size() * 4);
        } else if ((it = node.attrs.find("value_int")) != node.attrs.end()) {
            put(RMLK_INT64, {}, &it->second.i, 8);
        } else if ((it = node.attrs.find("value_ints")) != node.attrs.end()) {
            put(RMLK_INT64, {static_cast<int64_t>(it->second.ints.size())}, it->second.ints.data(),
                it->second.ints.size() * 8);
        } else {
            throw RtError(RMLK_ERR_OP, "Constant needs a value attribute");
        }
        if (node.outputs.size() != 1) throw RtError(RMLK_ERR_GRAPH, "Constant has one output");
        graph_copy.values[node.outputs[0]].is_initializer = true;
        values[node.outputs[0]] = upload_initializer(ht, stream);
    }
    check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    if (fuse) {
        folded_nodes = fold_constants(*this);
        fused_nodes = fuse_patterns(*this);
    }
    // liveness over the final node list
    last_use.assign(g->values.size(), -1);
    stats.assign(g->nodes.size(), NodeStat());
    for (size_t n = 0; n < g->nodes.size(); ++n)
        for (int v : g->nodes[n].inputs)
            if (v >= 0) last_use[v] = static_cast<int>(n);
    // where a graph input is the data of a ScatterND (alone, or as a stream of a row-stream node)
    scatter_inputs.clear();
    for (size_t n = 0; n < g->nodes.size(); ++n) {
        const Node &node = g->nodes[n];
        auto note = [&](size_t i) {
            if (i >= node.inputs.size() || node.inputs[i] < 0) return;
            const Value &val = g->values[node.inputs[i]];
            if (val.is_input && !val.is_initializer) scatter_inputs.emplace_back(static_cast<int>(n), node.inputs[i]);
        };
        if (node.op == "ScatterND") {
            note(0);
        } else if (node.op == "rmlk.HeadRows") {
            auto kinds = node.attrs.find("kinds");
            if (kinds == node.attrs.end()) continue;
            size_t at = 0;
            for (int64_t kind : kinds->second.ints) {   // (input lists by kind: op_fused_head_rows)
                if (kind == 1) note(at + 3);
                else if (kind == 2) note(at + 1);
                at += kind == 1 ? 5 : 3;
            }
        }
    }
}

// The copies of graph inputs that ScatterND nodes of this run will need as their destinations, all
// in one launch (the reference copies data -> output in front of every scatter,
// backend/scatter_nd.rs:128-129). Only inputs the caller did not donate: a donated one is
// updated in place, or copied by its node when something else still reads it.
void Session::copy_scatter_inputs_early() {
    early_copies.clear();
    if (!fuse || scatter_inputs.empty()) return;
    std::vector<void *> dsts;
    std::vector<const void *> srcs;
    std::vector<size_t> sizes;
    for (const std::pair<int, int> &site : scatter_inputs) {
        const Tensor &data = values[site.second];
        if (!data.defined() || !data.buf || data.buf->donated || data.nbytes() == 0) continue;
        Tensor y;
        y.dtype = data.dtype;
        y.shape = data.shape;
        auto b = std::make_shared<Buffer>();
        b->bytes = data.nbytes();
        b->pool = &pool;
        b->ptr = pool.alloc(b->bytes);
        y.buf = b;
        dsts.push_back(y.data());
        srcs.push_back(data.data());
        sizes.push_back(data.nbytes());
        early_copies.emplace(site, std::move(y));
    }
    if (!dsts.empty())
        check_status(rmlk_hip_memcpy_dtod_many(stream, static_cast<int32_t>(dsts.size()), dsts.data(), srcs.data(),
                                               sizes.data()),
                     "ScatterND copies");
}

void Session::run_nodes() {
    const rmlk_graph &gr = graph_copy;
    products_bf16_pieces = 0;
    attention_map.map.reset();   // (a run that ended in an error may have left one)
    attention_map.mask_value = -1;
    // Operators over tiny tensors (the per-step set-up of a decoder graph: tables, indices, masks) are
    // collected by the kernel library and go out as one launch in front of the next larger one. Not
    // with one kernel per node (no fusion), and not while nodes are timed one by one.
    struct Collecting {
        rmlk_stream_t stream;
        Pool &pool;
        bool on = false;
        void stop() {
            on = false;
            pool.hold_small = false;
            pool.let_go();
        }
        ~Collecting() {
            if (!on) return;
            (void)rmlk_hip_batch_end(stream);   // (an exception is on its way)
            stop();
        }
    } collecting{stream, pool};
    copy_scatter_inputs_early();
    if (fuse && !profiling) {
        check_status(rmlk_hip_batch_begin(stream), "collected launches");
        collecting.on = true;
        pool.hold_small = true;
    }
    for (size_t n = 0; n < gr.nodes.size(); ++n) {
        const Node &node = gr.nodes[n];
        if (node.op == "Constant") continue;
        OpContext ctx{*this, node, static_cast<int>(n), {}, {}, stream};
        for (int v : node.inputs) {
            if (v < 0) {
                ctx.in.push_back(nullptr);
                continue;
            }
            if (!values[v].defined())
                throw RtError(RMLK_ERR_OP, "input `" + gr.values[v].name + "` of node " +
                                               std::to_string(n) + " (" + node.op +
                                               ") has no value (graph input not fed?)");
            ctx.in.push_back(&values[v]);
        }
        std::vector<Tensor> outs(node.outputs.size());
        for (size_t o = 0; o < node.outputs.size(); ++o) ctx.out.push_back(&outs[o]);
        NodeStat &st = stats[n];
        const bool timed = profiling && !capturing;
        if (timed) {
            if (!st.e0) {
                check_hip(hipEventCreate(&st.e0), "hipEventCreate");
                check_hip(hipEventCreate(&st.e1), "hipEventCreate");
            }
            check_hip(hipEventRecord(st.e0, stream), "hipEventRecord");
        }
        try {
            find_op(node.op)(ctx);
        } catch (RtError &e) {
            throw RtError(e.code, std::string(e.what()) + " [node " + std::to_string(n) + " " +
                                      node.op + "]");
        }
        if (timed) check_hip(hipEventRecord(st.e1, stream), "hipEventRecord");
        // cost model: every distinct input read once, every output written once; views move nothing
        double bytes = 0.0, flops = 0.0;
        std::vector<const void *> seen;
        bool any_new = false;
        for (size_t o = 0; o < outs.size(); ++o) {
            bool is_view = false;
            for (Tensor *ti : ctx.in)
                if (ti && ti->buf && outs[o].buf == ti->buf) is_view = true;
            if (!is_view) {
                bytes += static_cast<double>(outs[o].nbytes());
                any_new = true;
            }
        }
        if (any_new || node.op == "ScatterND") {
            for (Tensor *ti : ctx.in) {
                if (!ti) continue;
                if (std::find(seen.begin(), seen.end(), ti->data()) != seen.end()) continue;
                seen.push_back(ti->data());
                if (node.op == "Gather" && ti == ctx.in[0]) {
                    bytes += static_cast<double>(outs[0].nbytes());  // only the gathered rows
                } else if (node.op == "ScatterND" && ti == ctx.in[0] && !any_new) {
                    continue;  // in place: only indices and updates move
                } else if (node.op == "rmlk.HeadRows" && ti->buf &&
                           std::any_of(outs.begin(), outs.end(),
                                       [&](const Tensor &o) { return o.buf == ti->buf; })) {
                    continue;  // a cache updated in place: only its new rows move (counted as read)
                } else {
                    bytes += static_cast<double>(ti->nbytes());
                }
            }
            if (node.op == "ScatterND" && !any_new) bytes += static_cast<double>(ctx.in[2]->nbytes());
        }
        if ((node.op == "MatMul" || node.op == "rmlk.AttnMatMul" || node.op == "rmlk.MatMulGroup" ||
             node.op == "rmlk.MatMulConst") &&
            ctx.in[0] && !ctx.in[0]->shape.empty()) {
            double out_elems = 0.0;
            for (const Tensor &t : outs) out_elems += static_cast<double>(t.numel());
            flops = 2.0 * out_elems * static_cast<double>(ctx.in[0]->shape.back());
        } else if (node.op == "rmlk.MatMulAddRMSNorm" && ctx.in[0] && ctx.in[1] && ctx.in[1]->rank() == 2) {
            // (weights of fused nodes are stored [n, k])
            flops = 2.0 * static_cast<double>(ctx.in[0]->numel()) * static_cast<double>(ctx.in[1]->shape[0]);
        } else if (node.op == "rmlk.Attention" && ctx.in[0] && ctx.in[1] && ctx.in[0]->rank() == 4 &&
                   ctx.in[1]->rank() == 4) {
            // scores and context: 2 * [B, H, S, L, D] multiply-adds
            flops = 4.0 * static_cast<double>(ctx.in[0]->numel()) * static_cast<double>(ctx.in[1]->shape[2]);
        } else if (node.op == "rmlk.MatMulGroupSwiGLU" &&
                   ctx.in[0] && ctx.in[1] && ctx.in[1]->rank() == 2 && ctx.in[1]->shape[1] > 0) {
            // rows of a times the whole weight matrix
            flops = 2.0 * static_cast<double>(ctx.in[0]->numel()) / static_cast<double>(ctx.in[1]->shape[1]) *
                    static_cast<double>(ctx.in[1]->numel());
        }
        st.bytes = bytes;
        st.flops = flops;
        for (size_t o = 0; o < node.outputs.size(); ++o) values[node.outputs[o]] = outs[o];
        // release what nobody reads any more (graph inputs stay unless they were donated)
        for (int v : node.inputs) {
            if (v < 0 || last_use[v] != static_cast<int>(n)) continue;
            const Value &val = gr.values[v];
            if (val.is_initializer || val.is_output) continue;
            if (val.is_input && !(values[v].buf && values[v].buf->donated)) continue;
            values[v].reset();
        }
        for (size_t o = 0; o < node.outputs.size(); ++o) {
            int v = node.outputs[o];
            if (last_use[v] < 0 && !gr.values[v].is_output) values[v].reset();
        }
    }
    if (collecting.on) {
        collecting.stop();
        check_status(rmlk_hip_batch_end(stream), "collected launches");
    }
    scratch_bufs.clear();
    early_copies.clear();
    attention_map.map.reset();
    attention_map.mask_value = -1;
}

// The error flag of the kernels is zero when the session is built and is put back to zero when it
// has been reported (or when a run has failed for another reason). A run that succeeds leaves it
// untouched, so it stays set across the replays that are enqueued without a wait in between
// (replay_enqueue) until check_error_flag reports it, and no run spends a launch on clearing it.
static void clear_flag(Session &s) {
    int32_t zero = 0;
    (void)rmlk_hip_write_small(s.stream, s.err_flag, &zero, sizeof(zero));
}

void Session::check_error_flag() {
    check_hip(hipSetDevice(device), "hipSetDevice");
    check_hip(hipMemcpyAsync(err_host, err_flag, sizeof(int32_t), hipMemcpyDeviceToHost, stream),
              "hipMemcpyAsync D2H (error flag)");
    check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    if (*err_host != 0) {
        int32_t code = *err_host;
        *err_host = 0;
        clear_flag(*this);
        throw RtError(RMLK_ERR_KERNEL,
                      "kernel failed: index out of range (code " + std::to_string(code) + ")");
    }
}

// The one-launch decode attention counts the blocks that have finished a KV head in
// `block_counters` and expects them zero on entry; it leaves them zero when it completes. A run that
// fails between launches may not have completed one: put the zeros back (a fill kernel, best effort
// — the error that is being reported wins) so that later runs of the session still merge.
static void rezero_block_counters(Session &s) {
    if (s.block_counters)
        (void)rmlk_hip_memset(s.stream, s.block_counters, 0, Session::kBlockCounters * sizeof(int32_t));
}

void Session::run() {
    check_hip(hipSetDevice(device), "hipSetDevice");
    plan.reset();  // an eager run with (possibly) other shapes invalidates a recorded graph
    // drop results of the previous run
    for (size_t v = 0; v < values.size(); ++v) {
        const Value &val = graph_copy.values[v];
        if (!val.is_initializer && !val.is_input) values[v].reset();
    }
    try {
        run_nodes();
    } catch (...) {
        rezero_block_counters(*this);
        clear_flag(*this);
        throw;
    }
    check_error_flag();
    if (profiling) {
        for (auto &st : stats) {
            st.micros = -1.0;
            if (st.e0 && st.e1) {
                float ms = 0.f;
                if (hipEventElapsedTime(&ms, st.e0, st.e1) == hipSuccess) st.micros = ms * 1e3;
            }
        }
    }
}

void Session::capture() {
    check_hip(hipSetDevice(device), "hipSetDevice");
    // Warm run: fills the pool so that the recorded run never reaches hipMalloc. Extra references
    // to the graph inputs are held meanwhile, so no operator may update a donated input in place:
    // the warm run leaves every input untouched and its results are dropped.
    std::vector<Tensor> saved_inputs(values.size());
    for (size_t v = 0; v < values.size(); ++v)
        if (graph_copy.values[v].is_input) saved_inputs[v] = values[v];
    run();
    for (size_t v = 0; v < values.size(); ++v) {
        const Value &val = graph_copy.values[v];
        if (val.is_input) values[v] = std::move(saved_inputs[v]);  // sole owner again
        else if (!val.is_initializer) values[v].reset();
    }
    saved_inputs.clear();
    auto p = std::make_unique<CapturedPlan>();
    capturing = true;
    pool.forbid_malloc = true;
    hipError_t e = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) {
        capturing = false;
        pool.forbid_malloc = false;
        check_hip(e, "hipStreamBeginCapture");
    }
    try {
        run_nodes();
    } catch (...) {
        hipGraph_t dead = nullptr;
        (void)hipStreamEndCapture(stream, &dead);
        if (dead) (void)hipGraphDestroy(dead);
        capturing = false;
        pool.forbid_malloc = false;
        rezero_block_counters(*this);
        throw;
    }
    capturing = false;
    pool.forbid_malloc = false;
    check_hip(hipStreamEndCapture(stream, &p->graph), "hipStreamEndCapture");
    check_hip(hipGraphInstantiate(&p->exec, p->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    // Every buffer the recorded kernels touch that is still referenced now (inputs, outputs and
    // in-place aliases of donated inputs) stays out of the pool's hands while the plan lives.
    // Intermediates went back to the pool: replays and eager runs never overlap on one stream.
    for (size_t v = 0; v < values.size(); ++v)
        if (values[v].defined()) p->pinned.push_back(values[v]);
    plan = std::move(p);
}

void Session::replay_enqueue() {
    if (!plan) throw RtError(RMLK_ERR_OP, "no recorded graph: call rmlk_session_capture first");
    check_hip(hipSetDevice(device), "hipSetDevice");
    check_hip(hipGraphLaunch(plan->exec, stream), "hipGraphLaunch");
}

void Session::replay() {
    replay_enqueue();
    check_error_flag();
}

}  // namespace rt
}  // namespace rmlk
