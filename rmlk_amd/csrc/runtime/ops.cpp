// Operator backends: ONNX shape inference + dtype dispatch + one call into the kernel C ABI each.
// The C++ counterpart of runtime/src/providers/cuda/backend/*.rs of the reference; each function
// names the backend it mirrors. Element types an operator accepts follow the reference's dispatch
// arms; Float16 arithmetic is rejected (the reference's f16 path cannot run: its device buffers
// have no Drop for f16, providers/cuda/data.rs:109-126).
#include <algorithm>
#include <cmath>
#include <functional>

#include "core.hpp"

namespace rmlk {
namespace rt {

namespace {

bool in_set(int32_t dt, std::initializer_list<int32_t> set) {
    for (int32_t s : set)
        if (s == dt) return true;
    return false;
}

void require_dtype(int32_t dt, std::initializer_list<int32_t> set) {
    if (!in_set(dt, set)) fail_unsupported(dt);
}

std::vector<int64_t> broadcast_shape(const std::vector<int64_t> &a, const std::vector<int64_t> &b) {
    // ref: runtime/src/utils/mod.rs:114-143
    size_t n = std::max(a.size(), b.size());
    std::vector<int64_t> out(n);
    for (size_t i = 0; i < n; ++i) {
        int64_t da = i + a.size() >= n ? a[i + a.size() - n] : 1;
        int64_t db = i + b.size() >= n ? b[i + b.size() - n] : 1;
        if (da != db && da != 1 && db != 1) fail_op("incompatible shapes for broadcasting");
        out[i] = da == 1 ? db : da;
    }
    return out;
}

// Element stride of `shape` along every dim of `out`, 0 where it is broadcast.
// ref: runtime/src/utils/mod.rs:56-112
rmlk_dims bcast_strides(const std::vector<int64_t> &shape, const std::vector<int64_t> &out) {
    std::vector<int64_t> dense = dense_strides(shape);
    std::vector<int64_t> st(out.size(), 0);
    for (size_t i = 0; i < out.size(); ++i) {
        if (i + shape.size() < out.size()) continue;
        size_t j = i + shape.size() - out.size();
        if (shape[j] == out[i] && shape[j] != 1) st[i] = dense[j];
    }
    return to_dims(st);
}

std::shared_ptr<HostVal> make_host_ints(const std::vector<int64_t> &v) {
    auto h = std::make_shared<HostVal>();
    h->i = v;
    return h;
}

bool all_hosted(const OpContext &c) {
    for (Tensor *t : c.in)
        if (t && t->defined() && !t->host) return false;
    return true;
}

int64_t wrap_to(int32_t dt, int64_t v) {
    switch (dt) {
        case RMLK_INT32: return static_cast<int32_t>(v);
        case RMLK_BOOL: return v != 0;
        case RMLK_INT8: return static_cast<int8_t>(v);
        case RMLK_UINT8: return static_cast<uint8_t>(v);
        case RMLK_INT16: return static_cast<int16_t>(v);
        case RMLK_UINT16: return static_cast<uint16_t>(v);
        case RMLK_UINT32: return static_cast<uint32_t>(v);
        default: return v;
    }
}

// index of output element `lin` of shape `out` into a broadcast operand of shape `shape`
size_t bcast_index(size_t lin, const std::vector<int64_t> &out, const std::vector<int64_t> &shape) {
    std::vector<int64_t> dense = dense_strides(shape);
    size_t idx = 0;
    for (int d = static_cast<int>(out.size()) - 1; d >= 0; --d) {
        int64_t i = out[d] ? static_cast<int64_t>(lin % out[d]) : 0;
        if (out[d]) lin /= out[d];
        int j = d - static_cast<int>(out.size() - shape.size());
        if (j >= 0 && shape[j] != 1) idx += static_cast<size_t>(i * dense[j]);
    }
    return idx;
}

bool is_int_like(int32_t dt) {
    return in_set(dt, {RMLK_INT32, RMLK_INT64, RMLK_BOOL, RMLK_INT8, RMLK_UINT8, RMLK_INT16,
                       RMLK_UINT16, RMLK_UINT32});
}

// ---- broadcast binary ops ---------------------------------------------------------------------
// ref: backend/binary.rs:18-112 (shared), backend/{add,sub,mul,div,equal,greater,pow}.rs
void binary_op(OpContext &c, int op) {
    const Tensor &a = c.input(0);
    const Tensor &b = c.input(1);
    if (op == RMLK_POW) {
        // the nine pairs the reference enables, backend/pow.rs:123-132
        if (!in_set(a.dtype, {RMLK_FLOAT, RMLK_INT32, RMLK_INT64})) fail_unsupported(a.dtype);
        if (!in_set(b.dtype, {RMLK_FLOAT, RMLK_INT32, RMLK_INT64})) fail_unsupported(b.dtype);
    } else {
        require_dtype(a.dtype, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
        if (b.dtype != a.dtype) fail_op("binary operands must have the same element type");
    }
    std::vector<int64_t> out_shape = broadcast_shape(a.shape, b.shape);
    const bool compare = op == RMLK_EQUAL || op == RMLK_GREATER;
    Tensor &y = c.alloc_output(0, compare ? RMLK_BOOL : a.dtype, out_shape);
    rmlk_dims od = to_dims(out_shape);
    std::vector<int64_t> oshape(od.v, od.v + od.rank);
    rmlk_dims as = bcast_strides(a.shape, oshape), bs = bcast_strides(b.shape, oshape);
    check_status(rmlk_hip_binary(c.stream, op, a.dtype, b.dtype, &od, &as, &bs, a.data(), b.data(),
                                 y.data()),
                 c.node.op.c_str());
    // host mirror for integer shape arithmetic
    if (a.host && b.host && is_int_like(a.dtype) && is_int_like(b.dtype) && op != RMLK_POW &&
        y.numel() <= kHostMirrorMax) {
        auto h = std::make_shared<HostVal>();
        size_t n = static_cast<size_t>(y.numel());
        h->i.resize(n);
        for (size_t k = 0; k < n; ++k) {
            int64_t x = a.host->as_int(bcast_index(k, out_shape, a.shape));
            int64_t z = b.host->as_int(bcast_index(k, out_shape, b.shape));
            int64_t r = 0;
            switch (op) {
                case RMLK_ADD: r = static_cast<int64_t>(static_cast<uint64_t>(x) + static_cast<uint64_t>(z)); break;
                case RMLK_SUB: r = static_cast<int64_t>(static_cast<uint64_t>(x) - static_cast<uint64_t>(z)); break;
                case RMLK_MUL: r = static_cast<int64_t>(static_cast<uint64_t>(x) * static_cast<uint64_t>(z)); break;
                case RMLK_DIV: r = z == 0 ? 0 : (z == -1 ? static_cast<int64_t>(0 - static_cast<uint64_t>(x)) : x / z); break;
                case RMLK_EQUAL: r = x == z; break;
                case RMLK_GREATER: r = x > z; break;
            }
            h->i[k] = wrap_to(y.dtype, r);
        }
        y.host = h;
    }
}
void op_add(OpContext &c) { binary_op(c, RMLK_ADD); }
void op_sub(OpContext &c) { binary_op(c, RMLK_SUB); }
void op_mul(OpContext &c) { binary_op(c, RMLK_MUL); }
void op_div(OpContext &c) { binary_op(c, RMLK_DIV); }
void op_pow(OpContext &c) { binary_op(c, RMLK_POW); }
void op_equal(OpContext &c) { binary_op(c, RMLK_EQUAL); }
void op_greater(OpContext &c) { binary_op(c, RMLK_GREATER); }

// ref: backend/whereop.rs:43-194 (ONNX order: condition, X, Y)
void op_where(OpContext &c) {
    const Tensor &cond = c.input(0);
    const Tensor &x = c.input(1);
    const Tensor &y = c.input(2);
    if (cond.dtype != RMLK_BOOL) fail_op("Where condition must be bool");
    require_dtype(x.dtype, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    if (y.dtype != x.dtype) fail_op("Where branches must have the same element type");
    std::vector<int64_t> out_shape = broadcast_shape(broadcast_shape(cond.shape, x.shape), y.shape);
    Tensor &o = c.alloc_output(0, x.dtype, out_shape);
    rmlk_dims od = to_dims(out_shape);
    std::vector<int64_t> oshape(od.v, od.v + od.rank);
    rmlk_dims xs = bcast_strides(x.shape, oshape), ys = bcast_strides(y.shape, oshape),
              cs = bcast_strides(cond.shape, oshape);
    check_status(rmlk_hip_where(c.stream, x.dtype, &od, &xs, &ys, &cs, x.data(), y.data(),
                                cond.data(), o.data()),
                 "Where");
    if (cond.host && x.host && y.host && is_int_like(x.dtype) && o.numel() <= kHostMirrorMax) {
        auto h = std::make_shared<HostVal>();
        size_t n = static_cast<size_t>(o.numel());
        h->i.resize(n);
        for (size_t k = 0; k < n; ++k)
            h->i[k] = cond.host->as_int(bcast_index(k, out_shape, cond.shape))
                          ? x.host->as_int(bcast_index(k, out_shape, x.shape))
                          : y.host->as_int(bcast_index(k, out_shape, y.shape));
        o.host = h;
    }
}

// ---- unary ------------------------------------------------------------------------------------
// ref: backend/unary.rs:12-50, backend/{sqrt,neg,sin,cos,sigmoid}.rs
void unary_op(OpContext &c, int op, std::initializer_list<int32_t> dtypes) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, dtypes);
    Tensor &y = c.alloc_output(0, x.dtype, x.shape);
    check_status(rmlk_hip_unary(c.stream, op, x.dtype, x.numel(), x.data(), y.data()),
                 c.node.op.c_str());
    if (op == RMLK_NEG && x.host && is_int_like(x.dtype)) {
        auto h = std::make_shared<HostVal>();
        for (int64_t v : x.host->i) h->i.push_back(wrap_to(x.dtype, -v));
        y.host = h;
    }
}
void op_sqrt(OpContext &c) { unary_op(c, RMLK_SQRT, {RMLK_FLOAT, RMLK_DOUBLE}); }
void op_sin(OpContext &c) { unary_op(c, RMLK_SIN, {RMLK_FLOAT, RMLK_DOUBLE}); }
// backend/cos.rs:65-67 lists Float/Int32/Int64 but only float kernels exist (cos.rs:28-35)
void op_cos(OpContext &c) { unary_op(c, RMLK_COS, {RMLK_FLOAT, RMLK_DOUBLE}); }
void op_sigmoid(OpContext &c) { unary_op(c, RMLK_SIGMOID, {RMLK_FLOAT, RMLK_DOUBLE}); }
// backend/neg.rs:67-71 dispatches Int64 without a kernel behind it (neg.rs:29-36); here it runs.
void op_neg(OpContext &c) {
    unary_op(c, RMLK_NEG, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
}

// ref: backend/cast.rs:29-179
void op_cast(OpContext &c) {
    const Tensor &x = c.input(0);
    const Attr *to = c.attr("to");
    if (!to) fail_op("missing `to` cast attribute");
    const int32_t dst = static_cast<int32_t>(to->i);
    static const int32_t pairs[][2] = {
        {RMLK_FLOAT16, RMLK_FLOAT}, {RMLK_FLOAT16, RMLK_DOUBLE}, {RMLK_FLOAT16, RMLK_INT32},
        {RMLK_FLOAT16, RMLK_UINT32}, {RMLK_FLOAT16, RMLK_INT64}, {RMLK_FLOAT16, RMLK_UINT64},
        {RMLK_FLOAT, RMLK_FLOAT16}, {RMLK_FLOAT, RMLK_DOUBLE}, {RMLK_FLOAT, RMLK_INT32},
        {RMLK_FLOAT, RMLK_UINT32}, {RMLK_FLOAT, RMLK_INT64}, {RMLK_FLOAT, RMLK_UINT64},
        {RMLK_DOUBLE, RMLK_FLOAT16}, {RMLK_DOUBLE, RMLK_FLOAT}, {RMLK_DOUBLE, RMLK_INT32},
        {RMLK_DOUBLE, RMLK_UINT32}, {RMLK_DOUBLE, RMLK_INT64}, {RMLK_DOUBLE, RMLK_UINT64},
        {RMLK_INT32, RMLK_FLOAT16}, {RMLK_INT32, RMLK_FLOAT}, {RMLK_INT32, RMLK_DOUBLE},
        {RMLK_INT32, RMLK_INT64}, {RMLK_UINT32, RMLK_FLOAT16}, {RMLK_UINT32, RMLK_FLOAT},
        {RMLK_UINT32, RMLK_DOUBLE}, {RMLK_UINT32, RMLK_UINT64}, {RMLK_INT64, RMLK_FLOAT16},
        {RMLK_INT64, RMLK_FLOAT}, {RMLK_INT64, RMLK_DOUBLE}, {RMLK_INT64, RMLK_INT32},
        {RMLK_UINT64, RMLK_FLOAT16}, {RMLK_UINT64, RMLK_FLOAT}, {RMLK_UINT64, RMLK_DOUBLE},
        {RMLK_UINT64, RMLK_UINT32}, {RMLK_BOOL, RMLK_FLOAT},
        // identity casts of the supported numeric types cost nothing to allow
        {RMLK_FLOAT, RMLK_FLOAT}, {RMLK_INT64, RMLK_INT64}, {RMLK_INT32, RMLK_INT32},
        {RMLK_DOUBLE, RMLK_DOUBLE},
    };
    bool ok = false;
    for (auto &p : pairs)
        if (p[0] == x.dtype && p[1] == dst) ok = true;
    if (!ok)
        throw RtError(RMLK_ERR_UNSUPPORTED, std::string("unsupported cast ") + dtype_name(x.dtype) +
                                                " to " + dtype_name(dst));
    Tensor &y = c.alloc_output(0, dst, x.shape);
    check_status(rmlk_hip_cast(c.stream, x.dtype, dst, x.numel(), x.data(), y.data()), "Cast");
    if (x.host) {
        auto h = std::make_shared<HostVal>();
        const bool dst_float = in_set(dst, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_FLOAT16});
        h->is_float = dst_float;
        for (size_t k = 0; k < x.host->size(); ++k) {
            if (dst_float) {
                double v = x.host->as_double(k);
                h->f.push_back(dst == RMLK_FLOAT ? static_cast<double>(static_cast<float>(v)) : v);
            } else {
                h->i.push_back(wrap_to(dst, x.host->is_float
                                                ? static_cast<int64_t>(std::trunc(x.host->f[k]))
                                                : x.host->i[k]));
            }
        }
        y.host = h;
    }
}

// ---- reductions -------------------------------------------------------------------------------
// ref: backend/reduce_mean.rs:47-232
void op_reduce_mean(OpContext &c) {
    const Tensor &x = c.input(0);
    // Int32 / Int64 arms of the reference run u32 / u64 kernels (kernels/reduce_mean.rs:19-29);
    // integer means are not on the Llama path and are rejected here.
    require_dtype(x.dtype, {RMLK_FLOAT, RMLK_DOUBLE});
    const int rank = std::max(x.rank(), 1);
    const bool keepdims = c.attr_int("keepdims", 1) > 0;
    const bool noop = c.attr_int("noop_with_empty_axes", 0) > 0;
    std::vector<int64_t> axes;
    bool have_axes = false;
    if (c.has_input(1)) {
        if (c.input(1).numel() > 0) {
            HostVal hv = c.host_values(1);
            for (size_t k = 0; k < hv.size(); ++k) axes.push_back(hv.as_int(k));
            have_axes = true;
        }
    } else {
        bool present = false;
        std::vector<int64_t> a = c.attr_ints("axes", &present);
        if (present && !a.empty()) {
            axes = a;
            have_axes = true;
        } else if (!present) {
            for (int d = 0; d < rank; ++d) axes.push_back(d);
            have_axes = true;
        }
    }
    if (!have_axes) {
        if (noop) {  // identity
            Tensor &y = c.alloc_output(0, x.dtype, x.shape);
            check_status(rmlk_hip_memcpy_dtod(c.stream, y.data(), x.data(), x.nbytes()),
                         "ReduceMean");
            return;
        }
        for (int d = 0; d < rank; ++d) axes.push_back(d);
    }
    std::vector<bool> red(rank, false);
    std::vector<int64_t> norm;
    for (int64_t a : axes) {
        int64_t n = normalize_axis(a, rank, "ReduceMean axis");
        if (!red[n]) norm.push_back(n);
        red[n] = true;
    }
    std::vector<int64_t> in_shape = x.shape;
    if (in_shape.empty()) in_shape.push_back(1);
    std::vector<int64_t> out_shape;
    for (int d = 0; d < rank; ++d) {
        if (!red[d]) out_shape.push_back(in_shape[d]);
        else if (keepdims) out_shape.push_back(1);
    }
    if (x.rank() == 0) out_shape.clear();
    Tensor &y = c.alloc_output(0, x.dtype, out_shape);
    rmlk_dims id = to_dims(in_shape);
    check_status(rmlk_hip_reduce_mean(c.stream, x.dtype, &id, norm.data(),
                                      static_cast<int32_t>(norm.size()), x.data(), y.data()),
                 "ReduceMean");
}

// ref: backend/softmax.rs:31-158. The reference accepts axis == -1, or axis == 1 on rank 4; any
// axis is accepted here (ONNX opset 13 semantics: softmax along that one axis).
void op_softmax(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT});
    if (x.rank() == 0) fail_op("Softmax needs rank >= 1");
    const int64_t axis = normalize_axis(c.attr_int("axis", -1), x.rank(), "Softmax axis");
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < axis; ++d) outer *= x.shape[d];
    for (int d = static_cast<int>(axis) + 1; d < x.rank(); ++d) inner *= x.shape[d];
    Tensor &y = c.alloc_output(0, x.dtype, x.shape);
    check_status(rmlk_hip_softmax(c.stream, x.dtype, outer, x.shape[axis], inner, x.data(),
                                  y.data()),
                 "Softmax");
}

// ref: backend/matmul.rs:47-356 (prepare_gemm_params, compute_output_shape). Output shape follows
// numpy / ONNX (the reference folds all leading dims into one, matmul.rs:323-330).
void op_matmul(OpContext &c) {
    const Tensor &a = c.input(0);
    const Tensor &b = c.input(1);
    require_dtype(a.dtype, {RMLK_FLOAT});
    if (b.dtype != a.dtype) fail_op("MatMul operands must have the same element type");
    if (a.rank() == 0 || b.rank() == 0) fail_op("ZeroRank");
    std::vector<int64_t> as = a.shape, bs = b.shape;
    const bool pa = as.size() == 1, pb = bs.size() == 1;
    if (pa) as.insert(as.begin(), 1);
    if (pb) bs.push_back(1);
    const int64_t m = as[as.size() - 2], k = as[as.size() - 1];
    const int64_t kb = bs[bs.size() - 2], n = bs[bs.size() - 1];
    if (k != kb) fail_op("IncompatibleDimForMul");
    std::vector<int64_t> abatch(as.begin(), as.end() - 2), bbatch(bs.begin(), bs.end() - 2);
    std::vector<int64_t> obatch;
    try {
        obatch = broadcast_shape(abatch, bbatch);
    } catch (const RtError &) {
        fail_op("IncompatibleDimForBroadcast");
    }
    int64_t batch = 1, na = 1, nb = 1;
    for (int64_t d : obatch) batch *= d;
    for (int64_t d : abatch) na *= d;
    for (int64_t d : bbatch) nb *= d;
    std::vector<int64_t> out_shape = obatch;
    if (!pa) out_shape.push_back(m);
    if (!pb) out_shape.push_back(n);
    Tensor &y = c.alloc_output(0, a.dtype, out_shape);
    if (y.numel() == 0) return;
    auto run = [&](int64_t bt, const void *pa_, int64_t sa, const void *pb_, int64_t sb, void *pc) {
        size_t ws_bytes = rmlk_hip_matmul_workspace_size(a.dtype, bt, m, n, k);
        void *ws = ws_bytes ? c.scratch(ws_bytes) : nullptr;
        check_status(rmlk_hip_matmul(c.stream, a.dtype, bt, m, n, k, pa_, k, sa, 0, pb_, n, sb, 0,
                                     pc, n, m * n, ws, ws_bytes),
                     "MatMul");
    };
    const bool a_full = na == batch, b_full = nb == batch;
    if ((a_full || na == 1) && (b_full || nb == 1)) {
        run(batch, a.data(), a_full && batch > 1 ? m * k : 0, b.data(),
            b_full && batch > 1 ? k * n : 0, y.data());
        return;
    }
    // mixed broadcast over several leading dims: one launch per output matrix
    const size_t es = dtype_size(a.dtype);
    for (int64_t o = 0; o < batch; ++o) {
        size_t ia = bcast_index(static_cast<size_t>(o), obatch, abatch);
        size_t ib = bcast_index(static_cast<size_t>(o), obatch, bbatch);
        run(1, static_cast<const char *>(a.data()) + ia * m * k * es, 0,
            static_cast<const char *>(b.data()) + ib * k * n * es, 0,
            static_cast<char *>(y.data()) + static_cast<size_t>(o) * m * n * es);
    }
}

// ---- data movement ----------------------------------------------------------------------------
const std::initializer_list<int32_t> kMoveTypes = {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE,
                                                   RMLK_INT32,   RMLK_UINT32, RMLK_INT64,
                                                   RMLK_UINT64};

// ref: backend/transpose.rs:44-131
void op_transpose(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    bool present = false;
    std::vector<int64_t> perm = c.attr_ints("perm", &present);
    if (!present)
        for (int d = x.rank() - 1; d >= 0; --d) perm.push_back(d);
    if (static_cast<int>(perm.size()) != x.rank()) fail_op("Transpose perm length must equal rank");
    std::vector<int64_t> out_shape(perm.size());
    for (size_t d = 0; d < perm.size(); ++d) {
        perm[d] = normalize_axis(perm[d], x.rank(), "Transpose perm");
        out_shape[d] = x.shape[perm[d]];
    }
    // A permutation that only moves size-1 dims leaves the element order unchanged: the output
    // is a view of the input (decode-time [1,1,H,D] <-> [1,H,1,D] head splits).
    bool same_order = true;
    int64_t prev = -1;
    for (size_t d = 0; d < perm.size(); ++d) {
        if (x.shape[perm[d]] == 1) continue;
        if (perm[d] < prev) same_order = false;
        prev = perm[d];
    }
    if (same_order) {
        c.view_output(0, x, out_shape);
        return;
    }
    Tensor &y = c.alloc_output(0, x.dtype, out_shape);
    rmlk_dims id = to_dims(x.shape);
    check_status(rmlk_hip_transpose(c.stream, x.dtype, &id, perm.data(), x.data(), y.data()),
                 "Transpose");
}

// ref: backend/expand.rs:49-156
void op_expand(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, kMoveTypes);
    HostVal shp = c.host_values(1);
    std::vector<int64_t> target;
    for (size_t k = 0; k < shp.size(); ++k) target.push_back(shp.as_int(k));
    std::vector<int64_t> out_shape = broadcast_shape(x.shape, target);
    Tensor &y = c.alloc_output(0, x.dtype, out_shape);
    rmlk_dims id = to_dims(x.shape), od = to_dims(out_shape);
    check_status(rmlk_hip_expand(c.stream, x.dtype, &id, &od, x.data(), y.data()), "Expand");
    if (x.host && y.numel() <= kHostMirrorMax) {
        auto h = std::make_shared<HostVal>();
        h->is_float = x.host->is_float;
        for (size_t k = 0; k < static_cast<size_t>(y.numel()); ++k) {
            size_t j = bcast_index(k, out_shape, x.shape);
            if (h->is_float) h->f.push_back(x.host->f[j]);
            else h->i.push_back(x.host->i[j]);
        }
        y.host = h;
    }
}

// ONNX Slice clamp rules as the reference's host side applies them, backend/slice.rs:357-463.
void op_slice(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    if (x.rank() > RMLK_MAX_RANK) fail_op("Slice supports rank <= 8");
    HostVal starts = c.host_values(1), ends = c.host_values(2);
    if (starts.size() != ends.size()) fail_op("Slice starts and ends must have the same length");
    if (x.rank() == 0) {
        // nothing to slice along: the scalar itself (cuda/src/kernels/slice.rs:200-222)
        if (starts.size() != 0) fail_op("AxisOutOfRange");
        c.view_output(0, x, {});
        return;
    }
    const int rank = x.rank();
    std::vector<int64_t> axes, steps;
    if (c.has_input(3)) {
        HostVal a = c.host_values(3);
        for (size_t k = 0; k < a.size(); ++k) axes.push_back(a.as_int(k));
    } else {
        for (size_t k = 0; k < starts.size(); ++k) axes.push_back(static_cast<int64_t>(k));
    }
    if (c.has_input(4)) {
        HostVal s = c.host_values(4);
        for (size_t k = 0; k < s.size(); ++k) steps.push_back(s.as_int(k));
        if (steps.size() != axes.size()) fail_op("StepsAndAxesLengthMismatch");
    } else {
        steps.assign(axes.size(), 1);
    }
    if (axes.size() != starts.size()) fail_op("Slice axes and starts must have the same length");
    std::vector<int64_t> st(rank, 0), sp(rank, 1), out_shape = x.shape;
    for (size_t k = 0; k < axes.size(); ++k) {
        int64_t axis = axes[k] < 0 ? axes[k] + rank : axes[k];
        if (axis < 0 || axis >= rank) fail_op("AxisOutOfRange");
        const int64_t step = steps[k];
        if (step == 0) fail_op("ZeroStep");
        const int64_t dim = x.shape[axis];
        int64_t start = starts.as_int(k);
        if (start < 0) start += dim;
        if (start < 0) start = 0;
        if (step > 0 && start > dim) start = dim;
        else if (step < 0 && start >= dim) start = dim - 1;
        int64_t end = ends.as_int(k);
        if (end < 0) end += dim;
        if (end < -1) end = -1;
        if (step > 0 && end > dim) end = dim;
        else if (step < 0 && end >= dim) end = dim - 1;
        int64_t count;
        if ((step < 0 && start < end) || (step > 0 && start >= end)) count = 0;
        else if (step > 0) count = (end - start + step - 1) / step;
        else count = (start - end + (-step) - 1) / (-step);
        st[axis] = count ? start : 0;
        sp[axis] = step;
        out_shape[axis] = count;
    }
    Tensor &y = c.alloc_output(0, x.dtype, out_shape);
    rmlk_dims id = to_dims(x.shape), sd = to_dims(st), pd = to_dims(sp), od = to_dims(out_shape);
    check_status(rmlk_hip_slice(c.stream, x.dtype, &id, &sd, &pd, &od, x.data(), y.data()),
                 "Slice");
    if (x.host && rank == 1) {
        auto h = std::make_shared<HostVal>();
        h->is_float = x.host->is_float;
        for (int64_t k = 0; k < out_shape[0]; ++k) {
            size_t j = static_cast<size_t>(st[0] + k * sp[0]);
            if (h->is_float) h->f.push_back(x.host->f[j]);
            else h->i.push_back(x.host->i[j]);
        }
        y.host = h;
    }
}

// ref: backend/concat.rs:28-199
void op_concat(OpContext &c) {
    const Tensor &first = c.input(0);
    require_dtype(first.dtype, kMoveTypes);
    if (first.rank() == 0) fail_op("scalars are not allowed");
    const Attr *ax = c.attr("axis");
    if (!ax) fail_op("`axis` is missing");
    const int64_t axis = normalize_axis(ax->i, first.rank(), "Concat axis");
    std::vector<int64_t> out_shape = first.shape;
    int64_t total = 0;
    for (int i = 0; i < c.n_inputs(); ++i) {
        const Tensor &t = c.input(i);
        if (t.dtype != first.dtype) fail_op("Concat inputs must have the same element type");
        if (t.rank() != first.rank()) fail_op("shape mismatch: ranks differ");
        for (int d = 0; d < t.rank(); ++d)
            if (d != axis && t.shape[d] != first.shape[d]) fail_op("dimension mismatch");
        total += t.shape[axis];
    }
    out_shape[axis] = total;
    Tensor &y = c.alloc_output(0, first.dtype, out_shape);
    rmlk_dims od = to_dims(out_shape);
    bool hosted = all_hosted(c) && first.rank() == 1 && total <= kHostMirrorMax;
    auto h = std::make_shared<HostVal>();
    std::vector<rmlk_dims> in_dims;
    std::vector<const void *> in_ptrs;
    for (int i = 0; i < c.n_inputs(); ++i) {
        const Tensor &t = c.input(i);
        in_dims.push_back(to_dims(t.shape));
        in_ptrs.push_back(t.numel() ? t.data() : nullptr);
        if (hosted) {
            h->is_float = t.host->is_float;
            for (size_t k = 0; k < t.host->size(); ++k) {
                if (h->is_float) h->f.push_back(t.host->f[k]);
                else h->i.push_back(t.host->i[k]);
            }
        }
    }
    check_status(rmlk_hip_concat_many(c.stream, first.dtype, c.n_inputs(), in_dims.data(), in_ptrs.data(),
                                      &od, static_cast<int32_t>(axis), y.data()),
                 "Concat");
    if (hosted) y.host = h;
}

// ref: backend/gather.rs:28-258
void op_gather(OpContext &c) {
    const Tensor &data = c.input(0);
    const Tensor &idx = c.input(1);
    require_dtype(data.dtype, kMoveTypes);
    if (idx.dtype != RMLK_INT32 && idx.dtype != RMLK_INT64) fail_unsupported(idx.dtype);
    if (data.rank() == 0) fail_op("scalar input data not allowed");
    const int64_t axis = normalize_axis(c.attr_int("axis", 0), data.rank(), "Gather axis");
    std::vector<int64_t> out_shape(data.shape.begin(), data.shape.begin() + axis);
    out_shape.insert(out_shape.end(), idx.shape.begin(), idx.shape.end());
    out_shape.insert(out_shape.end(), data.shape.begin() + axis + 1, data.shape.end());
    Tensor &y = c.alloc_output(0, data.dtype, out_shape);
    rmlk_dims dd = to_dims(data.shape);
    check_status(rmlk_hip_gather(c.stream, data.dtype, idx.dtype, &dd, static_cast<int32_t>(axis),
                                 idx.numel(), data.data(), idx.data(), y.data(), c.error_flag()),
                 "Gather");
    if (data.host && idx.host && data.rank() == 1) {
        auto h = std::make_shared<HostVal>();
        h->is_float = data.host->is_float;
        for (size_t k = 0; k < idx.host->size(); ++k) {
            int64_t j = idx.host->as_int(k);
            if (j < 0) j += data.shape[0];
            if (j < 0 || j >= data.shape[0]) fail_op("Gather index out of range");
            if (h->is_float) h->f.push_back(data.host->f[j]);
            else h->i.push_back(data.host->i[j]);
        }
        y.host = h;
    }
}

}  // namespace

// Output `out_index` as the destination of a ScatterND over input `data_index`: the data tensor
// itself when it may be updated in place (see op_scatter_nd), else a fresh copy of it.
Tensor &scatter_destination(OpContext &c, int data_index, int out_index, bool *copy_left_to_caller) {
    if (copy_left_to_caller) *copy_left_to_caller = false;
    const Tensor &data = c.input(data_index);
    const int vid = c.node.inputs[data_index];
    const Value &v = c.session.graph_copy.values[vid];
    const bool last_reader = c.session.last_use[vid] == c.node_index;
    const bool sole_owner = data.buf && data.buf.use_count() == 1;
    const bool may_overwrite = data.buf && (v.is_input ? data.buf->donated
                                                       : (data.buf->pool != nullptr));
    // the same value read through another input of this node (as updates, or by another row stream
    // of the launch) must keep its contents
    bool read_elsewhere = false;
    for (size_t i = 0; i < c.node.inputs.size(); ++i)
        if (static_cast<int>(i) != data_index && c.node.inputs[i] == vid) read_elsewhere = true;
    if (last_reader && sole_owner && may_overwrite && !read_elsewhere && !v.is_output && !v.is_initializer)
        return c.view_output(out_index, data, data.shape);
    // a copy of a graph input made in front of the first node of the run
    auto early = c.session.early_copies.find(std::make_pair(c.node_index, vid));
    if (early != c.session.early_copies.end() && early->second.dtype == data.dtype &&
        early->second.shape == data.shape) {
        if (out_index >= static_cast<int>(c.out.size()) || !c.out[out_index]) fail_op(c.node.op + ": missing output");
        *c.out[out_index] = std::move(early->second);
        c.session.early_copies.erase(early);
        return *c.out[out_index];
    }
    Tensor &y = c.alloc_output(out_index, data.dtype, data.shape);
    if (copy_left_to_caller) {
        *copy_left_to_caller = true;     // the caller's kernel copies while it scatters
        return y;
    }
    check_status(rmlk_hip_memcpy_dtod(c.stream, y.data(), data.data(), data.nbytes()),
                 "ScatterND copy");
    return y;
}

namespace {

// ref: backend/scatter_nd.rs:78-225. The reference always copies data -> output first
// (scatter_nd.rs:128-129). Here the copy is skipped and the update is done in place when nothing
// else can observe the data tensor afterwards: this node is its last reader, no view shares its
// buffer, it is not a graph output, and it is either an intermediate of this run or an input the
// caller donated (a KV cache fed back from the previous run).
void op_scatter_nd(OpContext &c) {
    const Tensor &data = c.input(0);
    const Tensor &idx = c.input(1);
    const Tensor &upd = c.input(2);
    require_dtype(data.dtype, kMoveTypes);
    if (idx.dtype != RMLK_INT64) fail_unsupported(idx.dtype);
    if (upd.dtype != data.dtype) fail_op("ScatterND updates must have the element type of data");
    if (data.rank() == 0 || idx.rank() == 0) fail_op("ScatterND needs rank >= 1 operands");
    const int64_t t = idx.shape.back();
    if (t > data.rank()) fail_op("ScatterND index tuple longer than data rank");
    std::vector<int64_t> expect(idx.shape.begin(), idx.shape.end() - 1);
    expect.insert(expect.end(), data.shape.begin() + t, data.shape.end());
    if (upd.shape != expect) fail_op("ScatterND updates shape mismatch");
    const std::string red = c.attr_string("reduction", "none");
    int32_t rcode;
    if (red == "none") rcode = RMLK_SCATTER_NONE;
    else if (red == "add") rcode = RMLK_SCATTER_ADD;
    else if (red == "mul") rcode = RMLK_SCATTER_MUL;
    else if (red == "max") rcode = RMLK_SCATTER_MAX;
    else if (red == "min") rcode = RMLK_SCATTER_MIN;
    else fail_op("ScatterND: unknown reduction " + red);
    if (rcode != RMLK_SCATTER_NONE)
        require_dtype(data.dtype, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    int64_t n_tuples = 1;
    for (size_t d = 0; d + 1 < idx.shape.size(); ++d) n_tuples *= idx.shape[d];

    bool fresh = false;
    Tensor *y = &scatter_destination(c, 0, 0, rcode == RMLK_SCATTER_NONE ? &fresh : nullptr);
    rmlk_dims dd = to_dims(data.shape);
    if (fresh) {
        // a fresh output: the copy of data and the assignment of the slices in one pass
        check_status(rmlk_hip_scatter_nd_copy(c.stream, data.dtype, &dd, n_tuples, static_cast<int32_t>(t),
                                              static_cast<const int64_t *>(idx.data()), upd.data(),
                                              c.input(0).data(), y->data(), c.error_flag()),
                     "ScatterND");
        return;
    }
    check_status(rmlk_hip_scatter_nd(c.stream, rcode, data.dtype, &dd, n_tuples,
                                     static_cast<int32_t>(t),
                                     static_cast<const int64_t *>(idx.data()), upd.data(),
                                     y->data(), c.error_flag()),
                 "ScatterND");
}

// ref: backend/trilu.rs:48-159
void op_trilu(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    if (x.rank() < 2) fail_op("Trilu needs rank >= 2");
    const bool upper = c.attr_int("upper", 1) != 0;
    int64_t k = 0;
    if (c.has_input(1)) {
        if (c.input(1).numel() != 1) fail_op("InvalidKTensor");
        k = c.host_values(1).as_int(0);
    }
    int64_t batch = 1;
    for (int d = 0; d < x.rank() - 2; ++d) batch *= x.shape[d];
    Tensor &y = c.alloc_output(0, x.dtype, x.shape);
    check_status(rmlk_hip_trilu(c.stream, x.dtype, batch, x.shape[x.rank() - 2],
                                x.shape[x.rank() - 1], upper, k, x.data(), y.data()),
                 "Trilu");
}

// ---- metadata ops -----------------------------------------------------------------------------
// ref: backend/reshape.rs:44-130 (the reference copies the payload; here the output is a view)
void op_reshape(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    HostVal shp = c.host_values(1);
    const bool allowzero = c.attr_int("allowzero", 0) != 0;
    std::vector<int64_t> out;
    int infer = -1;
    int64_t known = 1;
    for (size_t k = 0; k < shp.size(); ++k) {
        int64_t d = shp.as_int(k);
        if (d == 0 && !allowzero) {
            if (static_cast<int>(k) >= x.rank()) fail_op("Reshape: 0 dim beyond input rank");
            d = x.shape[k];
        }
        if (d == -1) {
            if (infer >= 0) fail_op("Reshape: more than one -1");
            infer = static_cast<int>(k);
            out.push_back(1);
            continue;
        }
        if (d < 0) fail_op("Reshape: negative dim");
        known *= d;
        out.push_back(d);
    }
    const int64_t n = x.numel();
    if (infer >= 0) {
        if (known == 0 || n % known) fail_op("Reshape: cannot infer dim");
        out[infer] = n / known;
    } else if (known != n) {
        fail_op("Reshape: element count mismatch");
    }
    Tensor &y = c.view_output(0, x, out);
    y.host = x.host;
}

// ref: backend/unsqueeze.rs:39-120 (axes input of opset 13, or the attribute of older opsets)
void op_unsqueeze(OpContext &c) {
    const Tensor &x = c.input(0);
    require_dtype(x.dtype, {RMLK_FLOAT16, RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    std::vector<int64_t> axes;
    if (c.has_input(1)) {
        HostVal a = c.host_values(1);
        for (size_t k = 0; k < a.size(); ++k) axes.push_back(a.as_int(k));
    } else {
        bool present = false;
        axes = c.attr_ints("axes", &present);
        if (!present) fail_op("Unsqueeze needs axes");
    }
    const int64_t out_rank = x.rank() + static_cast<int64_t>(axes.size());
    std::vector<bool> is_new(out_rank, false);
    for (int64_t a : axes) {
        int64_t n = normalize_axis(a, out_rank, "Unsqueeze axis");
        if (is_new[n]) fail_op("Unsqueeze: duplicate axis");
        is_new[n] = true;
    }
    std::vector<int64_t> out;
    int src = 0;
    for (int64_t d = 0; d < out_rank; ++d) out.push_back(is_new[d] ? 1 : x.shape[src++]);
    Tensor &y = c.view_output(0, x, out);
    y.host = x.host;
}

// ref: backend/shape.rs:29-92
void op_shape(OpContext &c) {
    const Tensor &x = c.input(0);
    const int64_t rank = x.rank();
    int64_t s = c.attr_int("start", 0), e = c.attr("end") ? c.attr("end")->i : rank;
    if (s < 0) s += rank;
    if (e < 0) e += rank;
    s = std::min(std::max<int64_t>(s, 0), rank);
    e = std::min(std::max<int64_t>(e, 0), rank);
    std::vector<int64_t> vals;
    for (int64_t d = s; d < e; ++d) vals.push_back(x.shape[d]);
    Tensor &y = c.alloc_output(0, RMLK_INT64, {static_cast<int64_t>(vals.size())});
    if (!vals.empty())
        check_status(rmlk_hip_write_small(c.stream, y.data(), vals.data(), vals.size() * 8),
                     "Shape");
    y.host = make_host_ints(vals);
}

// ref: backend/range.rs:56-151. Element count follows ONNX: max(ceil((limit - start) / delta), 0).
void op_range(OpContext &c) {
    const Tensor &st = c.input(0);
    require_dtype(st.dtype, {RMLK_FLOAT, RMLK_DOUBLE, RMLK_INT32, RMLK_INT64});
    if (c.input(1).dtype != st.dtype || c.input(2).dtype != st.dtype)
        fail_op("Range inputs must have the same element type");
    HostVal s = c.host_values(0), l = c.host_values(1), d = c.host_values(2);
    if (s.size() != 1 || l.size() != 1 || d.size() != 1) fail_op("Range inputs must be scalars");
    int64_t n;
    if (st.dtype == RMLK_INT32 || st.dtype == RMLK_INT64) {
        const int64_t a = s.as_int(0), b = l.as_int(0), step = d.as_int(0);
        if (step == 0) fail_op("Range delta must not be zero");
        const int64_t span = b - a;
        n = (span > 0) == (step > 0) ? (std::llabs(span) + std::llabs(step) - 1) / std::llabs(step) : 0;
        if (span == 0) n = 0;
        Tensor &y = c.alloc_output(0, st.dtype, {n});
        if (st.dtype == RMLK_INT32) {
            int32_t a32 = static_cast<int32_t>(a), d32 = static_cast<int32_t>(step);
            check_status(rmlk_hip_range(c.stream, st.dtype, n, &a32, &d32, y.data()), "Range");
        } else {
            check_status(rmlk_hip_range(c.stream, st.dtype, n, &a, &step, y.data()), "Range");
        }
        if (n <= kHostMirrorMax) {
            std::vector<int64_t> v;
            for (int64_t k = 0; k < n; ++k) v.push_back(wrap_to(st.dtype, a + k * step));
            y.host = make_host_ints(v);
        }
        return;
    }
    const double a = s.as_double(0), b = l.as_double(0), step = d.as_double(0);
    if (step == 0.0) fail_op("Range delta must not be zero");
    n = std::max<int64_t>(static_cast<int64_t>(std::ceil((b - a) / step)), 0);
    Tensor &y = c.alloc_output(0, st.dtype, {n});
    if (st.dtype == RMLK_FLOAT) {
        float af = static_cast<float>(a), df = static_cast<float>(step);
        check_status(rmlk_hip_range(c.stream, st.dtype, n, &af, &df, y.data()), "Range");
    } else {
        check_status(rmlk_hip_range(c.stream, st.dtype, n, &a, &step, y.data()), "Range");
    }
}

// ref: backend/constant_of_shape.rs:29-70
void op_constant_of_shape(OpContext &c) {
    HostVal shp = c.host_values(0);
    std::vector<int64_t> out;
    for (size_t k = 0; k < shp.size(); ++k) {
        if (shp.as_int(k) < 0) fail_op("ConstantOfShape: negative dim");
        out.push_back(shp.as_int(k));
    }
    int32_t dt = RMLK_FLOAT;
    uint8_t value[8] = {0};
    const Attr *v = c.attr("value");
    if (v) {
        if (v->t.numel() != 1) fail_op("ConstantOfShape value must hold one element");
        dt = v->t.dtype;
        std::memcpy(value, v->t.data.data(), dtype_size(dt));
    }
    Tensor &y = c.alloc_output(0, dt, out);
    check_status(rmlk_hip_fill(c.stream, dt, y.numel(), value, y.data()), "ConstantOfShape");
    if (y.numel() <= kHostMirrorMax && is_int_like(dt)) {
        int64_t iv = 0;
        std::memcpy(&iv, value, dtype_size(dt));
        if (dt == RMLK_INT32) iv = static_cast<int32_t>(iv);
        y.host = make_host_ints(std::vector<int64_t>(static_cast<size_t>(y.numel()), iv));
    }
}

// Constant nodes are materialised when the session is built (their output value is an
// initializer); running one is a no-op. ref: backend/constant.rs
void op_constant(OpContext &) {}

const std::unordered_map<std::string, OpFn> &registry() {
    // the operator table of CudaKernel for the Llama path (backend/mod.rs:82-162)
    static const std::unordered_map<std::string, OpFn> table = {
        {"Add", op_add},         {"Sub", op_sub},
        {"Mul", op_mul},         {"Div", op_div},
        {"Pow", op_pow},         {"Equal", op_equal},
        {"Greater", op_greater}, {"Where", op_where},
        {"Sqrt", op_sqrt},       {"Neg", op_neg},
        {"Sin", op_sin},         {"Cos", op_cos},
        {"Sigmoid", op_sigmoid}, {"Cast", op_cast},
        {"ReduceMean", op_reduce_mean},
        {"Softmax", op_softmax}, {"MatMul", op_matmul},
        {"Transpose", op_transpose},
        {"Expand", op_expand},   {"Slice", op_slice},
        {"Concat", op_concat},   {"Gather", op_gather},
        {"ScatterND", op_scatter_nd},
        {"Trilu", op_trilu},     {"Reshape", op_reshape},
        {"Unsqueeze", op_unsqueeze},
        {"Shape", op_shape},     {"Range", op_range},
        {"ConstantOfShape", op_constant_of_shape},
        {"Constant", op_constant},
        {"rmlk.RMSNorm", op_fused_rmsnorm},
        {"rmlk.SwiGLU", op_fused_swiglu},
        {"rmlk.AddRMSNorm", op_fused_add_rmsnorm},
        {"rmlk.ScaleMaskSoftmax", op_fused_softmax},
        {"rmlk.Rotary", op_fused_rotary},
        {"rmlk.HeadRows", op_fused_head_rows},
        {"rmlk.AttnMatMul", op_fused_attn_matmul},
        {"rmlk.Attention", op_fused_attention},
        {"rmlk.MatMulAddRMSNorm", op_fused_matmul_add_rmsnorm},
        {"rmlk.MatMulConst", op_fused_matmul_const},
        {"rmlk.MatMulGroup", op_fused_matmul_group},
        {"rmlk.MatMulGroupSwiGLU", op_fused_matmul_group_swiglu},
    };
    return table;
}
}  // namespace

OpFn find_op(const std::string &name) {
    auto it = registry().find(name);
    return it == registry().end() ? nullptr : it->second;
}

}  // namespace rt
}  // namespace rmlk
