// Contiguous maps: Sqrt Neg Sin Cos Sigmoid, Cast, Fill.
// Replaces cuda/src/ptx/{sqrt,neg,sin,cos,cast}.cu (cuda/src/ptx/headers/unary_op_macro.cuh:1-11,
// cast_op_macro.cuh:1-11) and the cuDNN sigmoid call (cuda/src/kernels/activation.rs:6-39).
#include <cstring>
#include <limits>
#include <type_traits>

#include "batch.hpp"
#include "elementwise.hpp"
#include "functors.hpp"

namespace rmlk {
namespace {

template <typename F, typename TI, typename TO, int VEC>
__global__ __launch_bounds__(kEwBlock) void map_flat_kernel(const TI *__restrict__ in,
                                                            TO *__restrict__ out, uint32_t n) {
    if constexpr (VEC == 1) {
        const uint32_t step = gridDim.x * kEwBlock;
        for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n; i += step) out[i] = F::apply(in[i]);
    } else {
        const uint32_t n_vec = n / kEwVec;
        for (uint32_t base = blockIdx.x * kEwChunk; base < n_vec; base += gridDim.x * kEwChunk) {
            const uint32_t i0 = base + threadIdx.x;
            if (base + kEwChunk <= n_vec) {
                TI ri[kEwUnroll][kEwVec];
#pragma unroll
                for (int u = 0; u < kEwUnroll; ++u)
                    load_op<kEwDense, true>(in + static_cast<size_t>(i0 + u * kEwBlock) * kEwVec, ri[u]);
#pragma unroll
                for (int u = 0; u < kEwUnroll; ++u) {
                    TO ro[kEwVec];
#pragma unroll
                    for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ri[u][j]);
                    store_vec(out + static_cast<size_t>(i0 + u * kEwBlock) * kEwVec, ro);
                }
            } else {
                for (uint32_t i = i0; i < n_vec; i += kEwBlock) {
                    TI ri[kEwVec];
                    TO ro[kEwVec];
                    load_op<kEwDense, true>(in + static_cast<size_t>(i) * kEwVec, ri);
#pragma unroll
                    for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ri[j]);
                    store_vec(out + static_cast<size_t>(i) * kEwVec, ro);
                }
            }
        }
        if (blockIdx.x == 0 && threadIdx.x < (n - n_vec * kEwVec)) {
            uint32_t t = n_vec * kEwVec + threadIdx.x;
            out[t] = F::apply(in[t]);
        }
    }
}

template <typename F, typename TI, typename TO>
int32_t launch_map(hipStream_t s, int64_t n, const void *in, void *out) {
    constexpr int64_t kPiece = (int64_t)1 << 30;
    for (int64_t off = 0; off < n; off += kPiece) {
        const TI *pi = static_cast<const TI *>(in) + off;
        TO *po = static_cast<TO *>(out) + off;
        uint32_t m = static_cast<uint32_t>(n - off < kPiece ? n - off : kPiece);
        size_t ai = sizeof(TI) * kEwVec > 16 ? 16 : sizeof(TI) * kEwVec;
        size_t ao = sizeof(TO) * kEwVec > 16 ? 16 : sizeof(TO) * kEwVec;
        bool aligned = reinterpret_cast<uintptr_t>(pi) % ai == 0 &&
                       reinterpret_cast<uintptr_t>(po) % ao == 0;
        if (aligned) {
            unsigned grid = chunk_grid(m / kEwVec, kEwChunk);
            map_flat_kernel<F, TI, TO, kEwVec><<<grid, kEwBlock, 0, s>>>(pi, po, m);
        } else {
            unsigned grid = grid_for(m, kEwBlock, 16);
            map_flat_kernel<F, TI, TO, 1><<<grid, kEwBlock, 0, s>>>(pi, po, m);
        }
        int32_t st = launch_status();
        if (st) return st;
    }
    return RMLK_OK;
}

template <template <typename> class F>
int32_t dispatch_float(hipStream_t s, int32_t dt, int64_t n, const void *in, void *out) {
    switch (dt) {
        case RMLK_FLOAT: return launch_map<F<float>, float, float>(s, n, in, out);
        case RMLK_DOUBLE: return launch_map<F<double>, double, double>(s, n, in, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

// ---- cast ------------------------------------------------------------------------------------
template <typename TI>
int32_t dispatch_cast_dst(hipStream_t s, int32_t dst, int64_t n, const void *in, void *out) {
    switch (dst) {
        case RMLK_FLOAT: return launch_map<CastF<TI, float>, TI, float>(s, n, in, out);
        case RMLK_DOUBLE: return launch_map<CastF<TI, double>, TI, double>(s, n, in, out);
        case RMLK_FLOAT16: return launch_map<CastF<TI, _Float16>, TI, _Float16>(s, n, in, out);
        case RMLK_INT8: return launch_map<CastF<TI, int8_t>, TI, int8_t>(s, n, in, out);
        case RMLK_INT16: return launch_map<CastF<TI, int16_t>, TI, int16_t>(s, n, in, out);
        case RMLK_INT32: return launch_map<CastF<TI, int32_t>, TI, int32_t>(s, n, in, out);
        case RMLK_INT64: return launch_map<CastF<TI, int64_t>, TI, int64_t>(s, n, in, out);
        case RMLK_UINT8: return launch_map<CastF<TI, uint8_t>, TI, uint8_t>(s, n, in, out);
        case RMLK_UINT16: return launch_map<CastF<TI, uint16_t>, TI, uint16_t>(s, n, in, out);
        case RMLK_UINT32: return launch_map<CastF<TI, uint32_t>, TI, uint32_t>(s, n, in, out);
        case RMLK_UINT64: return launch_map<CastF<TI, uint64_t>, TI, uint64_t>(s, n, in, out);
        case RMLK_BOOL: return launch_map<CastF<TI, BoolTag>, TI, BoolTag>(s, n, in, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

template <typename T>
__global__ __launch_bounds__(kEwBlock) void fill_kernel(T *__restrict__ out, T value, uint64_t n) {
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kEwBlock;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += step)
        out[i] = value;
}

template <typename T>
__global__ __launch_bounds__(kEwBlock) void range_kernel(T *__restrict__ out, T start, T delta,
                                                         uint64_t n) {
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kEwBlock;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kEwBlock + threadIdx.x; i < n; i += step) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            out[i] = static_cast<T>(static_cast<U>(start) + static_cast<U>(i) * static_cast<U>(delta));
        } else {
            out[i] = static_cast<T>(static_cast<double>(start) +
                                    static_cast<double>(i) * static_cast<double>(delta));
        }
    }
}

struct SmallPayload {
    uint32_t w[64];
};

__global__ void write_small_kernel(uint8_t *__restrict__ dst, SmallPayload p, uint32_t bytes) {
    const uint8_t *src = reinterpret_cast<const uint8_t *>(p.w);
    for (uint32_t i = threadIdx.x; i < bytes; i += blockDim.x) dst[i] = src[i];
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_range(rmlk_stream_t stream, int32_t dtype, int64_t n,
                                  const void *start, const void *delta, void *out) {
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    if (dtype != RMLK_FLOAT && dtype != RMLK_DOUBLE && dtype != RMLK_INT32 && dtype != RMLK_INT64)
        return RMLK_ERR_UNSUPPORTED;
    if (n == 0) return RMLK_OK;
    if (!start || !delta || !out) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    unsigned grid = grid_for(n, kEwBlock, 16);
    switch (dtype) {
        case RMLK_FLOAT: range_kernel<float><<<grid, kEwBlock, 0, s>>>(static_cast<float *>(out), *static_cast<const float *>(start), *static_cast<const float *>(delta), n); break;
        case RMLK_DOUBLE: range_kernel<double><<<grid, kEwBlock, 0, s>>>(static_cast<double *>(out), *static_cast<const double *>(start), *static_cast<const double *>(delta), n); break;
        case RMLK_INT32: range_kernel<int32_t><<<grid, kEwBlock, 0, s>>>(static_cast<int32_t *>(out), *static_cast<const int32_t *>(start), *static_cast<const int32_t *>(delta), n); break;
        default: range_kernel<int64_t><<<grid, kEwBlock, 0, s>>>(static_cast<int64_t *>(out), *static_cast<const int64_t *>(start), *static_cast<const int64_t *>(delta), n); break;
    }
    return launch_status();
}

extern "C" int32_t rmlk_hip_write_small(rmlk_stream_t stream, void *dst, const void *src,
                                        size_t bytes) {
    if (bytes == 0) return RMLK_OK;
    if (bytes > sizeof(SmallPayload)) return RMLK_ERR_INVALID_ARGUMENT;
    if (!dst || !src) return RMLK_ERR_NULL_POINTER;
    SmallPayload p;
    std::memset(&p, 0, sizeof(p));
    std::memcpy(&p, src, bytes);
    write_small_kernel<<<1, 64, 0, as_stream(stream)>>>(static_cast<uint8_t *>(dst), p,
                                                        static_cast<uint32_t>(bytes));
    return launch_status();
}

extern "C" int32_t rmlk_hip_unary(rmlk_stream_t stream, int32_t op, int32_t dtype, int64_t n,
                                  const void *in, void *out) {
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    if (op < RMLK_SQRT || op > RMLK_SIGMOID) return RMLK_ERR_INVALID_ARGUMENT;
    if (dtype_size(dtype) == 0) return RMLK_ERR_UNSUPPORTED;
    bool is_float = dtype == RMLK_FLOAT || dtype == RMLK_DOUBLE;
    bool neg_int = op == RMLK_NEG && (dtype == RMLK_INT32 || dtype == RMLK_INT64);
    if (!is_float && !neg_int) return RMLK_ERR_UNSUPPORTED;
    if (n == 0) return RMLK_OK;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    if (n <= kBatchMaxElems && batch_collecting() && is_float) {
        // (a tiny map on a stream that is collecting its launches)
        SmallOp so{};
        so.kind = kSmallUnary;
        so.op = op;
        so.dt = dtype;
        so.in[0] = in;
        so.out = out;
        const int64_t flat[2][kMaxRank] = {{1}, {1}};
        if (small_op_layout(so, 1, &n, 1, flat) && batch_take(as_stream_collecting(stream), so)) return RMLK_OK;
    }
    hipStream_t s = as_stream(stream);
    switch (op) {
        case RMLK_SQRT: return dispatch_float<SqrtF>(s, dtype, n, in, out);
        case RMLK_SIN: return dispatch_float<SinF>(s, dtype, n, in, out);
        case RMLK_COS: return dispatch_float<CosF>(s, dtype, n, in, out);
        case RMLK_SIGMOID: return dispatch_float<SigmoidF>(s, dtype, n, in, out);
        case RMLK_NEG:
            if (dtype == RMLK_INT32) return launch_map<NegF<int32_t>, int32_t, int32_t>(s, n, in, out);
            if (dtype == RMLK_INT64) return launch_map<NegF<int64_t>, int64_t, int64_t>(s, n, in, out);
            return dispatch_float<NegF>(s, dtype, n, in, out);
        default: return RMLK_ERR_INVALID_ARGUMENT;
    }
}

extern "C" int32_t rmlk_hip_cast(rmlk_stream_t stream, int32_t src, int32_t dst, int64_t n,
                                 const void *in, void *out) {
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    if (dtype_size(src) == 0 || dtype_size(dst) == 0) return RMLK_ERR_UNSUPPORTED;
    if (n == 0) return RMLK_OK;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    auto collectable = [](int32_t dt) {
        return dt == RMLK_FLOAT || dt == RMLK_DOUBLE || dt == RMLK_INT32 || dt == RMLK_INT64 || dt == RMLK_BOOL;
    };
    if (n <= kBatchMaxElems && batch_collecting() && collectable(src) && collectable(dst)) {
        SmallOp so{};
        so.kind = kSmallCast;
        so.dt = src;
        so.dt2 = dst;
        so.in[0] = in;
        so.out = out;
        const int64_t flat[2][kMaxRank] = {{1}, {1}};
        if (small_op_layout(so, 1, &n, 1, flat) && batch_take(as_stream_collecting(stream), so)) return RMLK_OK;
    }
    hipStream_t s = as_stream(stream);
    switch (src) {
        case RMLK_FLOAT: return dispatch_cast_dst<float>(s, dst, n, in, out);
        case RMLK_DOUBLE: return dispatch_cast_dst<double>(s, dst, n, in, out);
        case RMLK_FLOAT16: return dispatch_cast_dst<_Float16>(s, dst, n, in, out);
        case RMLK_INT8: return dispatch_cast_dst<int8_t>(s, dst, n, in, out);
        case RMLK_INT16: return dispatch_cast_dst<int16_t>(s, dst, n, in, out);
        case RMLK_INT32: return dispatch_cast_dst<int32_t>(s, dst, n, in, out);
        case RMLK_INT64: return dispatch_cast_dst<int64_t>(s, dst, n, in, out);
        case RMLK_UINT8: return dispatch_cast_dst<uint8_t>(s, dst, n, in, out);
        case RMLK_UINT16: return dispatch_cast_dst<uint16_t>(s, dst, n, in, out);
        case RMLK_UINT32: return dispatch_cast_dst<uint32_t>(s, dst, n, in, out);
        case RMLK_UINT64: return dispatch_cast_dst<uint64_t>(s, dst, n, in, out);
        case RMLK_BOOL: return dispatch_cast_dst<BoolTag>(s, dst, n, in, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

extern "C" int32_t rmlk_hip_fill(rmlk_stream_t stream, int32_t dtype, int64_t n,
                                 const void *value, void *out) {
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    int es = dtype_size(dtype);
    if (es == 0) return RMLK_ERR_UNSUPPORTED;
    if (n == 0) return RMLK_OK;
    if (!value || !out) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    unsigned grid = grid_for(n, kEwBlock, 16);
    switch (es) {
        case 1: fill_kernel<uint8_t><<<grid, kEwBlock, 0, s>>>(static_cast<uint8_t *>(out), *static_cast<const uint8_t *>(value), n); break;
        case 2: fill_kernel<uint16_t><<<grid, kEwBlock, 0, s>>>(static_cast<uint16_t *>(out), *static_cast<const uint16_t *>(value), n); break;
        case 4: fill_kernel<uint32_t><<<grid, kEwBlock, 0, s>>>(static_cast<uint32_t *>(out), *static_cast<const uint32_t *>(value), n); break;
        default: fill_kernel<uint64_t><<<grid, kEwBlock, 0, s>>>(static_cast<uint64_t *>(out), *static_cast<const uint64_t *>(value), n); break;
    }
    return launch_status();
}
