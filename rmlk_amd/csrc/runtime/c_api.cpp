// extern "C" surface of the host runtime (include/rmlk_runtime.h): exceptions become status
// codes plus a per-thread message.
#include "core.hpp"

using namespace rmlk::rt;

namespace {
thread_local std::string g_last_error;

template <typename Fn>
int32_t guarded(Fn &&fn) {
    try {
        fn();
        return 0;
    } catch (const RtError &e) {
        g_last_error = e.what();
        return e.code ? e.code : RMLK_ERR_OP;
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return RMLK_ERR_OP;
    }
}

std::vector<int64_t> dims_vec(const int64_t *dims, int32_t rank) {
    if (rank < 0 || rank > RMLK_MAX_RANK) throw RtError(RMLK_ERR_BAD_RANK, "rank outside 0..8");
    if (rank > 0 && !dims) throw RtError(RMLK_ERR_NULL_POINTER, "null dims");
    return std::vector<int64_t>(dims, dims + rank);
}

HostTensor host_tensor(int32_t dtype, const int64_t *dims, int32_t rank, const void *data) {
    HostTensor t;
    t.dtype = dtype;
    t.shape = dims_vec(dims, rank);
    const size_t es = dtype_size(dtype);
    if (!es) fail_unsupported(dtype);
    for (int64_t d : t.shape)
        if (d < 0) throw RtError(RMLK_ERR_INVALID_ARGUMENT, "negative dim");
    const size_t bytes = static_cast<size_t>(t.numel()) * es;
    if (bytes && !data) throw RtError(RMLK_ERR_NULL_POINTER, "null tensor data");
    t.data.assign(static_cast<const uint8_t *>(data), static_cast<const uint8_t *>(data) + bytes);
    return t;
}

Node &node_of(rmlk_graph *g, int32_t node) {
    if (!g) throw RtError(RMLK_ERR_NULL_POINTER, "null graph");
    if (node < 0 || node >= static_cast<int32_t>(g->nodes.size()))
        throw RtError(RMLK_ERR_GRAPH, "node index out of range");
    return g->nodes[node];
}

int input_id(rmlk_session *s, const char *name) {
    if (!s || !name) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
    auto it = s->impl.graph_copy.by_name.find(name);
    if (it == s->impl.graph_copy.by_name.end() || !s->impl.graph_copy.values[it->second].is_input)
        throw RtError(RMLK_ERR_GRAPH, std::string("unknown graph input `") + name + "`");
    return it->second;
}

int output_id(rmlk_session *s, const char *name) {
    if (!s || !name) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
    auto it = s->impl.graph_copy.by_name.find(name);
    if (it == s->impl.graph_copy.by_name.end() || !s->impl.graph_copy.values[it->second].is_output)
        throw RtError(RMLK_ERR_GRAPH, std::string("unknown graph output `") + name + "`");
    return it->second;
}

// Declared shape check of the reference: rank must match, a declared dim of 0 is dynamic
// (ref: runtime/src/utils/mod.rs:19-38 compare_shapes).
void check_declared(const Value &v, int32_t dtype, const std::vector<int64_t> &shape) {
    if (v.dtype && v.dtype != dtype)
        throw RtError(RMLK_ERR_OP, "input `" + v.name + "`: element type " + dtype_name(dtype) +
                                       " does not match the declared " + dtype_name(v.dtype));
    if (v.shape.size() != shape.size())
        throw RtError(RMLK_ERR_OP, "input `" + v.name + "`: rank mismatch");
    for (size_t d = 0; d < shape.size(); ++d)
        if (v.shape[d] != 0 && v.shape[d] != shape[d])
            throw RtError(RMLK_ERR_OP, "input `" + v.name + "`: dimensions mismatch");
}
}  // namespace

int rmlk_graph::value_id(const std::string &name, bool create) {
    auto it = by_name.find(name);
    if (it != by_name.end()) return it->second;
    if (!create) return -1;
    Value v;
    v.name = name;
    values.push_back(v);
    by_name[name] = static_cast<int>(values.size()) - 1;
    return static_cast<int>(values.size()) - 1;
}

extern "C" {

const char *rmlk_last_error(void) { return g_last_error.c_str(); }
void rmlk_set_last_error(const char *message) { g_last_error = message ? message : ""; }

int32_t rmlk_graph_create(rmlk_graph **out) {
    return guarded([&] {
        if (!out) throw RtError(RMLK_ERR_NULL_POINTER, "null out");
        *out = new rmlk_graph();
    });
}

void rmlk_graph_destroy(rmlk_graph *g) { delete g; }

int32_t rmlk_graph_input(rmlk_graph *g, const char *name, int32_t dtype, const int64_t *dims,
                         int32_t rank) {
    return guarded([&] {
        if (!g || !name) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        if (g->by_name.count(name))
            throw RtError(RMLK_ERR_GRAPH, std::string("duplicate node name `") + name + "`");
        int id = g->value_id(name, true);
        Value &v = g->values[id];
        v.dtype = dtype;
        v.shape = dims_vec(dims, rank);
        v.is_input = true;
        g->inputs.push_back(id);
    });
}

int32_t rmlk_graph_constant(rmlk_graph *g, const char *name, int32_t dtype, const int64_t *dims,
                            int32_t rank, const void *data) {
    return guarded([&] {
        if (!g || !name) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        if (g->by_name.count(name))
            throw RtError(RMLK_ERR_GRAPH, std::string("duplicate node name `") + name + "`");
        HostTensor t = host_tensor(dtype, dims, rank, data);
        int id = g->value_id(name, true);
        Value &v = g->values[id];
        v.dtype = dtype;
        v.shape = t.shape;
        v.is_initializer = true;
        v.init = std::move(t);
    });
}

int32_t rmlk_graph_op(rmlk_graph *g, const char *op, const char *const *inputs, int32_t n_inputs,
                      const char *const *outputs, int32_t n_outputs) {
    int32_t index = -1;
    int32_t st = guarded([&] {
        if (!g || !op) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        if (n_outputs < 1) throw RtError(RMLK_ERR_GRAPH, "op must declare at least one output");
        if (!find_op(op))
            throw RtError(RMLK_ERR_GRAPH, std::string("invalid op for the graph builder: ") + op);
        Node node;
        node.op = op;
        for (int32_t i = 0; i < n_inputs; ++i) {
            if (!inputs[i] || !inputs[i][0]) {
                node.inputs.push_back(-1);
                continue;
            }
            int id = g->value_id(inputs[i], false);
            if (id < 0)
                throw RtError(RMLK_ERR_GRAPH, std::string("unknown name `") + inputs[i] + "`");
            node.inputs.push_back(id);
        }
        for (int32_t i = 0; i < n_outputs; ++i) {
            if (!outputs[i] || !outputs[i][0]) throw RtError(RMLK_ERR_GRAPH, "empty output name");
            int existing = g->value_id(outputs[i], false);
            if (existing >= 0 && (g->values[existing].is_input || g->values[existing].is_initializer ||
                                  g->values[existing].producer >= 0))
                throw RtError(RMLK_ERR_GRAPH,
                              std::string("duplicate node name `") + outputs[i] + "`");
            int id = g->value_id(outputs[i], true);
            g->values[id].producer = static_cast<int>(g->nodes.size());
            node.outputs.push_back(id);
        }
        g->nodes.push_back(std::move(node));
        index = static_cast<int32_t>(g->nodes.size()) - 1;
    });
    return st ? st : index;
}

int32_t rmlk_graph_attr_int(rmlk_graph *g, int32_t node, const char *name, int64_t value) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::Int;
        a.i = value;
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_attr_float(rmlk_graph *g, int32_t node, const char *name, float value) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::Float;
        a.f = value;
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_attr_ints(rmlk_graph *g, int32_t node, const char *name, const int64_t *values,
                             int32_t n) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::Ints;
        if (n > 0 && !values) throw RtError(RMLK_ERR_NULL_POINTER, "null ints");
        a.ints.assign(values, values + (n > 0 ? n : 0));
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_attr_floats(rmlk_graph *g, int32_t node, const char *name, const float *values,
                               int32_t n) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::Floats;
        if (n > 0 && !values) throw RtError(RMLK_ERR_NULL_POINTER, "null floats");
        a.floats.assign(values, values + (n > 0 ? n : 0));
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_attr_string(rmlk_graph *g, int32_t node, const char *name, const char *value) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::String;
        a.s = value ? value : "";
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_attr_tensor(rmlk_graph *g, int32_t node, const char *name, int32_t dtype,
                               const int64_t *dims, int32_t rank, const void *data) {
    return guarded([&] {
        Attr a;
        a.kind = Attr::TensorK;
        a.t = host_tensor(dtype, dims, rank, data);
        node_of(g, node).attrs[name] = a;
    });
}

int32_t rmlk_graph_output(rmlk_graph *g, const char *name) {
    return guarded([&] {
        if (!g || !name) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        int id = g->value_id(name, false);
        if (id < 0) throw RtError(RMLK_ERR_GRAPH, std::string("unknown name `") + name + "`");
        g->values[id].is_output = true;
        g->outputs.push_back(id);
    });
}

int32_t rmlk_session_create(const rmlk_graph *g, int32_t device, rmlk_session **out) {
    return guarded([&] {
        if (!g || !out) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        auto s = std::make_unique<rmlk_session>();
        s->impl.build(*g, device);
        *out = s.release();
    });
}

int32_t rmlk_session_create_ex(const rmlk_graph *g, int32_t device, uint32_t flags,
                               rmlk_session **out) {
    return guarded([&] {
        if (!g || !out) throw RtError(RMLK_ERR_NULL_POINTER, "null argument");
        auto s = std::make_unique<rmlk_session>();
        s->impl.fuse = (flags & RMLK_SESSION_NO_FUSION) == 0;
        if ((flags & RMLK_SESSION_WEIGHTS_F16) && (flags & RMLK_SESSION_WEIGHTS_BF16))
            throw RtError(RMLK_ERR_INVALID_ARGUMENT, "one storage type for the weights at most");
        if (flags & RMLK_SESSION_WEIGHTS_F16) s->impl.weight_storage = RMLK_FLOAT16;
        if (flags & RMLK_SESSION_WEIGHTS_BF16) s->impl.weight_storage = RMLK_BFLOAT16;
        if (flags & RMLK_SESSION_WEIGHTS_F32) {
            if (s->impl.weight_storage != RMLK_FLOAT)
                throw RtError(RMLK_ERR_INVALID_ARGUMENT, "one storage type for the weights at most");
            s->impl.lossless_16bit = false;
        }
        s->impl.bf16_pieces = (flags & RMLK_SESSION_BF16_PIECES) != 0;
        s->impl.build(*g, device);
        *out = s.release();
    });
}

int32_t rmlk_session_fused_nodes(const rmlk_session *s) { return s ? s->impl.fused_nodes : 0; }
int32_t rmlk_session_weights_16bit(const rmlk_session *s) { return s ? s->impl.weights_16bit : 0; }
int32_t rmlk_session_products_bf16_pieces(const rmlk_session *s) { return s ? s->impl.products_bf16_pieces : 0; }

void rmlk_session_destroy(rmlk_session *s) {
    if (!s) return;
    (void)hipSetDevice(s->impl.device);
    if (s->impl.stream) (void)hipStreamSynchronize(s->impl.stream);
    delete s;
}

int32_t rmlk_session_set_input(rmlk_session *s, const char *name, int32_t dtype,
                               const int64_t *dims, int32_t rank, const void *host_data) {
    return guarded([&] {
        int id = input_id(s, name);
        Session &ss = s->impl;
        check_hip(hipSetDevice(ss.device), "hipSetDevice");
        std::vector<int64_t> shape = dims_vec(dims, rank);
        check_declared(ss.graph_copy.values[id], dtype, shape);
        if (!dtype_size(dtype)) fail_unsupported(dtype);
        Tensor &t = ss.values[id];
        size_t bytes = dtype_size(dtype);
        for (int64_t d : shape) {
            if (d < 0) throw RtError(RMLK_ERR_INVALID_ARGUMENT, "negative dim");
            bytes *= static_cast<size_t>(d);
        }
        // same shape as before and a buffer of the session's own: refresh it in place, so that a
        // recorded HIP graph keeps reading the address it knows
        // only when every owner of the buffer is accounted for. Without a recorded graph that is
        // the input slot alone: a view of the input that the last run left among the values (a
        // Reshape of an input as a graph output) must keep the old bytes, so a fresh buffer is
        // taken. With a recorded graph the owners are the session's values that share the buffer
        // and the plan's pins of them; the recorded kernels read this address, so it is refreshed
        // in place (outputs of the last replay that are views of the input then show the new bytes
        // until the next replay rewrites them). Any other owner drops the plan.
        bool reuse = t.defined() && t.dtype == dtype && t.shape == shape && t.buf &&
                     t.buf->pool == &ss.pool && !t.buf->donated;
        if (reuse) {
            long expected = 1;
            if (ss.plan) {
                expected = 0;
                for (const Tensor &v : ss.values)
                    if (v.buf == t.buf) ++expected;
                for (const Tensor &v : ss.plan->pinned)
                    if (v.buf == t.buf) ++expected;
            }
            reuse = t.buf.use_count() == expected;
        }
        if (!reuse) {
            if (ss.plan) ss.plan.reset();
            t.reset();
            t.dtype = dtype;
            t.shape = shape;
            auto b = std::make_shared<Buffer>();
            b->bytes = bytes ? bytes : 1;
            b->pool = &ss.pool;
            b->ptr = ss.pool.alloc(b->bytes);
            t.buf = b;
        }
        if (bytes) {
            if (!host_data) throw RtError(RMLK_ERR_NULL_POINTER, "null input data");
            check_hip(hipMemcpyAsync(t.data(), host_data, bytes, hipMemcpyHostToDevice, ss.stream),
                      "hipMemcpyAsync H2D");
            // the host buffer belongs to the caller: finish the copy before returning
            check_hip(hipStreamSynchronize(ss.stream), "hipStreamSynchronize");
        }
    });
}

int32_t rmlk_session_bind_input(rmlk_session *s, const char *name, int32_t dtype,
                                const int64_t *dims, int32_t rank, void *device_data,
                                int32_t donate) {
    return guarded([&] {
        int id = input_id(s, name);
        Session &ss = s->impl;
        std::vector<int64_t> shape = dims_vec(dims, rank);
        check_declared(ss.graph_copy.values[id], dtype, shape);
        if (!dtype_size(dtype)) fail_unsupported(dtype);
        if (ss.plan) ss.plan.reset();
        Tensor &t = ss.values[id];
        t.reset();
        t.dtype = dtype;
        t.shape = shape;
        if (t.numel() > 0 && !device_data) throw RtError(RMLK_ERR_NULL_POINTER, "null device data");
        auto b = std::make_shared<Buffer>();
        b->ptr = device_data;
        b->bytes = t.nbytes();
        b->donated = donate != 0;
        t.buf = b;
    });
}

int32_t rmlk_session_feed_output(rmlk_session *s, const char *out_name, const char *in_name) {
    return guarded([&] {
        int oid = output_id(s, out_name);
        int iid = input_id(s, in_name);
        Session &ss = s->impl;
        Tensor &o = ss.values[oid];
        if (!o.defined())
            throw RtError(RMLK_ERR_OP, std::string("output `") + out_name + "` has no value yet");
        check_declared(ss.graph_copy.values[iid], o.dtype, o.shape);
        if (ss.plan) ss.plan.reset();
        Tensor t = o;
        o.reset();
        t.host.reset();
        // the tensor now belongs to the input slot alone: an operator may update it in place
        if (t.buf && t.buf.use_count() == 1 && (t.buf->pool || t.buf->donated)) t.buf->donated = true;
        ss.values[iid] = t;
    });
}

int32_t rmlk_session_run(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.run();
    });
}

int32_t rmlk_session_output_info(rmlk_session *s, const char *name, int32_t *dtype, int64_t *dims,
                                 int32_t *rank, void **device_data) {
    return guarded([&] {
        int id = output_id(s, name);
        const Tensor &t = s->impl.values[id];
        if (!t.defined())
            throw RtError(RMLK_ERR_OP, std::string("output `") + name + "` has no value yet");
        if (dtype) *dtype = t.dtype;
        if (rank) *rank = t.rank();
        if (dims)
            for (int d = 0; d < t.rank(); ++d) dims[d] = t.shape[d];
        if (device_data) *device_data = t.data();
    });
}

int32_t rmlk_session_read_output(rmlk_session *s, const char *name, void *host_data,
                                 size_t bytes) {
    return guarded([&] {
        int id = output_id(s, name);
        Session &ss = s->impl;
        const Tensor &t = ss.values[id];
        if (!t.defined())
            throw RtError(RMLK_ERR_OP, std::string("output `") + name + "` has no value yet");
        if (bytes != t.nbytes()) throw RtError(RMLK_ERR_SIZE_MISMATCH, "output size mismatch");
        if (!bytes) return;
        if (!host_data) throw RtError(RMLK_ERR_NULL_POINTER, "null host buffer");
        check_hip(hipSetDevice(ss.device), "hipSetDevice");
        check_hip(hipMemcpyAsync(host_data, t.data(), bytes, hipMemcpyDeviceToHost, ss.stream),
                  "hipMemcpyAsync D2H");
        check_hip(hipStreamSynchronize(ss.stream), "hipStreamSynchronize");
    });
}

int32_t rmlk_session_capture(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.capture();
    });
}

int32_t rmlk_session_replay(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.replay();
    });
}

int32_t rmlk_session_replay_enqueue(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.replay_enqueue();
    });
}

int32_t rmlk_session_check(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.check_error_flag();
    });
}

int32_t rmlk_session_sync(rmlk_session *s) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        check_hip(hipSetDevice(s->impl.device), "hipSetDevice");
        check_hip(hipStreamSynchronize(s->impl.stream), "hipStreamSynchronize");
    });
}

rmlk_stream_t rmlk_session_stream(rmlk_session *s) { return s ? s->impl.stream : nullptr; }

int32_t rmlk_session_set_profiling(rmlk_session *s, int32_t enabled) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        s->impl.profiling = enabled != 0;
    });
}

int32_t rmlk_session_node_count(rmlk_session *s) {
    return s ? static_cast<int32_t>(s->impl.graph_copy.nodes.size()) : 0;
}

int32_t rmlk_session_node_info(rmlk_session *s, int32_t node, const char **op, double *micros,
                               double *bytes, double *flops) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        Session &ss = s->impl;
        if (node < 0 || node >= static_cast<int32_t>(ss.graph_copy.nodes.size()))
            throw RtError(RMLK_ERR_GRAPH, "node index out of range");
        if (op) *op = ss.graph_copy.nodes[node].op.c_str();
        if (micros) *micros = ss.stats[node].micros;
        if (bytes) *bytes = ss.stats[node].bytes;
        if (flops) *flops = ss.stats[node].flops;
    });
}

int32_t rmlk_session_memory_stats(rmlk_session *s, int64_t *pool_bytes, int64_t *hip_mallocs,
                                  int64_t *device_syncs) {
    return guarded([&] {
        if (!s) throw RtError(RMLK_ERR_NULL_POINTER, "null session");
        if (pool_bytes) *pool_bytes = s->impl.pool.pool_bytes;
        if (hip_mallocs) *hip_mallocs = s->impl.pool.hip_mallocs;
        if (device_syncs) *device_syncs = s->impl.device_syncs;
    });
}

}  // extern "C"
