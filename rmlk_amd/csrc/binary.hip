// Broadcast binary ops: Add Sub Mul Div Pow Equal Greater.
// Replaces cuda/src/ptx/{add,sub,mul,div,pow,equal,greater}.cu of the reference, whose kernels
// decode a `size_t` info buffer with one div/mod pair per dim per element
// (cuda/src/ptx/headers/binary_op_macros.cuh:14-42).
#include <type_traits>

#include "elementwise.hpp"

namespace rmlk {
namespace {

template <typename T>
struct AddF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) + static_cast<U>(y));
        } else {
            return x + y;
        }
    }
};
template <typename T>
struct SubF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) - static_cast<U>(y));
        } else {
            return x - y;
        }
    }
};
template <typename T>
struct MulF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) * static_cast<U>(y));
        } else {
            return x * y;
        }
    }
};
// Integer division truncates toward zero (cuda/src/ptx/div.cu:9-12). The reference leaves x/0 and
// MIN/-1 undefined; here x/0 = 0 and MIN/-1 wraps to MIN so that no input can trap.
template <typename T>
struct DivF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            if (y == 0) return 0;
            if (y == static_cast<T>(-1)) return static_cast<T>(U(0) - static_cast<U>(x));
            return x / y;
        } else {
            return x / y;
        }
    }
};
template <typename T>
struct EqualF {
    static __device__ __forceinline__ uint8_t apply(T x, T y) { return x == y ? 1 : 0; }
};
template <typename T>
struct GreaterF {
    static __device__ __forceinline__ uint8_t apply(T x, T y) { return x > y ? 1 : 0; }
};

// Pow (cuda/src/ptx/pow.cu:18-65): float base -> powf(x, (float)y); double base -> pow; integer
// base -> llround(pow((double)x, (double)y)). Exponents 2, 3 and 0.5 take the product / sqrt
// forms, which are the correctly rounded results the CPU oracle produces for them.
template <typename TX, typename TY>
struct PowF {
    static __device__ __forceinline__ TX apply(TX x, TY y) {
        if constexpr (std::is_same<TX, float>::value) {
            float e = static_cast<float>(y);
            if (e == 2.0f) return x * x;
            if (e == 3.0f) return x * x * x;
            if (e == 0.5f) return sqrtf(x);
            return powf(x, e);
        } else if constexpr (std::is_same<TX, double>::value) {
            double e = static_cast<double>(y);
            if (e == 2.0) return x * x;
            if (e == 3.0) return x * x * x;
            if (e == 0.5) return sqrt(x);
            return pow(x, e);
        } else {
            double r = pow(static_cast<double>(x), static_cast<double>(y));
            return static_cast<TX>(llround(r));
        }
    }
};

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
    hipStream_t s = as_stream(stream);
    if (op != RMLK_POW && dtype_a != dtype_b) return RMLK_ERR_UNSUPPORTED;
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
