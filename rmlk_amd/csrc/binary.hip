// Broadcast binary ops: Add Sub Mul Div Pow Equal Greater.
// Replaces cuda/src/ptx/{add,sub,mul,div,pow,equal,greater}.cu of the reference, whose kernels
// decode a `size_t` info buffer with one div/mod pair per dim per element
// (cuda/src/ptx/headers/binary_op_macros.cuh:14-42).
#include <type_traits>

#include "batch.hpp"
#include "elementwise.hpp"
#include "functors.hpp"

namespace rmlk {
namespace {

template <template <typename> class F, typename T, typename TO>
int32_t run_same(hipStream_t s, int rank, const int64_t *shape, const int64_t (*st)[kMaxRank],
                 const void *a, const void *b, void *out) {
    return for_each_piece<3>(rank, shape, st,
                             [&](int r, const int64_t *shp, const int64_t (*str)[kMaxRank],
                                 const int64_t *offs) {
                                 return launch_binary_typed<F<T>, T, T, TO>(
                                     s, r, shp, str, static_cast<const T *>(a) + offs[0],
                                     static_cast<const T *>(b) + offs[1],
                                     static_cast<TO *>(out) + offs[2]);
                             });
}

template <template <typename> class F, bool kCompare>
int32_t dispatch_same(hipStream_t s, int32_t dt, int rank, const int64_t *shape,
                      const int64_t (*st)[kMaxRank], const void *a, const void *b, void *out) {
    switch (dt) {
        case RMLK_FLOAT:
            return run_same<F, float, typename std::conditional<kCompare, uint8_t, float>::type>(
                s, rank, shape, st, a, b, out);
        case RMLK_DOUBLE:
            return run_same<F, double, typename std::conditional<kCompare, uint8_t, double>::type>(
                s, rank, shape, st, a, b, out);
        case RMLK_INT32:
            return run_same<F, int32_t,
                            typename std::conditional<kCompare, uint8_t, int32_t>::type>(
                s, rank, shape, st, a, b, out);
        case RMLK_INT64:
            return run_same<F, int64_t,
                            typename std::conditional<kCompare, uint8_t, int64_t>::type>(
                s, rank, shape, st, a, b, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

template <typename TX, typename TY>
int32_t run_pow(hipStream_t s, int rank, const int64_t *shape, const int64_t (*st)[kMaxRank],
                const void *a, const void *b, void *out) {
    return for_each_piece<3>(rank, shape, st,
                             [&](int r, const int64_t *shp, const int64_t (*str)[kMaxRank],
                                 const int64_t *offs) {
                                 return launch_binary_typed<PowF<TX, TY>, TX, TY, TX>(
                                     s, r, shp, str, static_cast<const TX *>(a) + offs[0],
                                     static_cast<const TY *>(b) + offs[1],
                                     static_cast<TX *>(out) + offs[2]);
                             });
}

template <typename TX>
int32_t dispatch_pow_exp(hipStream_t s, int32_t dt_b, int rank, const int64_t *shape,
                         const int64_t (*st)[kMaxRank], const void *a, const void *b, void *out) {
    switch (dt_b) {
        case RMLK_FLOAT: return run_pow<TX, float>(s, rank, shape, st, a, b, out);
        case RMLK_DOUBLE: return run_pow<TX, double>(s, rank, shape, st, a, b, out);
        case RMLK_INT32: return run_pow<TX, int32_t>(s, rank, shape, st, a, b, out);
        case RMLK_INT64: return run_pow<TX, int64_t>(s, rank, shape, st, a, b, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_binary(rmlk_stream_t stream, int32_t op, int32_t dtype_a,
                                   int32_t dtype_b, const rmlk_dims *out_shape,
                                   const rmlk_dims *a_stride, const rmlk_dims *b_stride,
                                   const void *a, const void *b, void *out) {
    if (!dims_ok(out_shape) || !dims_ok(a_stride) || !dims_ok(b_stride)) return RMLK_ERR_BAD_RANK;
    if (a_stride->rank != out_shape->rank || b_stride->rank != out_shape->rank)
        return RMLK_ERR_SIZE_MISMATCH;
    int64_t numel = dims_numel(out_shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!a || !b || !out) return RMLK_ERR_NULL_POINTER;
    const int rank = out_shape->rank;
    int64_t st[3][kMaxRank];
    for (int d = 0; d < rank; ++d) {
        if (a_stride->v[d] < 0 || b_stride->v[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        st[0][d] = a_stride->v[d];
        st[1][d] = b_stride->v[d];
    }
    dense_strides(rank, out_shape->v, st[2]);
    if (op != RMLK_POW && dtype_a != dtype_b) return RMLK_ERR_UNSUPPORTED;
    // a tiny operator on a stream that is collecting its launches: handed over as a record
    if (numel <= kBatchMaxElems && batch_collecting() && op >= RMLK_ADD && op <= RMLK_GREATER && op != RMLK_POW &&
        (dtype_a == RMLK_FLOAT || dtype_a == RMLK_DOUBLE || dtype_a == RMLK_INT32 || dtype_a == RMLK_INT64)) {
        SmallOp so{};
        so.kind = kSmallBinary;
        so.op = op;
        so.dt = dtype_a;
        so.in[0] = a;
        so.in[1] = b;
        so.out = out;
        if (small_op_layout(so, rank, out_shape->v, 2, st) && batch_take(as_stream_collecting(stream), so))
            return RMLK_OK;
    }
    hipStream_t s = as_stream(stream);
    switch (op) {
        case RMLK_ADD: return dispatch_same<AddF, false>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_SUB: return dispatch_same<SubF, false>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_MUL: return dispatch_same<MulF, false>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_DIV: return dispatch_same<DivF, false>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_EQUAL:
            return dispatch_same<EqualF, true>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_GREATER:
            return dispatch_same<GreaterF, true>(s, dtype_a, rank, out_shape->v, st, a, b, out);
        case RMLK_POW:
            switch (dtype_a) {
                case RMLK_FLOAT:
                    return dispatch_pow_exp<float>(s, dtype_b, rank, out_shape->v, st, a, b, out);
                case RMLK_DOUBLE:
                    return dispatch_pow_exp<double>(s, dtype_b, rank, out_shape->v, st, a, b, out);
                case RMLK_INT32:
                    return dispatch_pow_exp<int32_t>(s, dtype_b, rank, out_shape->v, st, a, b, out);
                case RMLK_INT64:
                    return dispatch_pow_exp<int64_t>(s, dtype_b, rank, out_shape->v, st, a, b, out);
                default: return RMLK_ERR_UNSUPPORTED;
            }
        default: return RMLK_ERR_INVALID_ARGUMENT;
    }
}
