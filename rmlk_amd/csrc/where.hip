// Where: out = cond ? x : y with three-way broadcast. A pure move, so it is instantiated per
// element size, not per dtype. Replaces cuda/src/ptx/where.cu:4-12
// (cuda/src/ptx/headers/ternary_op_macro.cuh:1-34).
#include "batch.hpp"
#include "elementwise.hpp"

namespace rmlk {
namespace {

template <typename T>
__device__ __forceinline__ void select_store(T *dst, const T (&x)[kEwVec], const T (&y)[kEwVec],
                                             const uint8_t (&c)[kEwVec]) {
    T ro[kEwVec];
#pragma unroll
    for (int j = 0; j < kEwVec; ++j) ro[j] = c[j] ? x[j] : y[j];
    store_vec(dst, ro);
}

// XM / YM: how x and y walk the output (kEwDense, or kEwRepeat: one element for all of it); the
// condition is dense. Other combinations take the nd<1> kernel.
template <typename T, int XM, int YM>
__global__ __launch_bounds__(kEwBlock) void where_flat_kernel(const T *__restrict__ x,
                                                              const T *__restrict__ y,
                                                              const uint8_t *__restrict__ c,
                                                              T *__restrict__ out, uint32_t n) {
    const uint32_t n_vec = n / kEwVec;
    for (uint32_t base = blockIdx.x * kEwChunk; base < n_vec; base += gridDim.x * kEwChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kEwChunk <= n_vec) {
            T rx[kEwUnroll][kEwVec], ry[kEwUnroll][kEwVec];
            uint8_t rc[kEwUnroll][kEwVec];
#pragma unroll
            for (int u = 0; u < kEwUnroll; ++u) {
                const size_t e = static_cast<size_t>(i0 + u * kEwBlock) * kEwVec;
                load_op<XM, true>(XM == kEwRepeat ? x : x + e, rx[u]);
                load_op<YM, true>(YM == kEwRepeat ? y : y + e, ry[u]);
                load_op<kEwDense, true>(c + e, rc[u]);
            }
#pragma unroll
            for (int u = 0; u < kEwUnroll; ++u)
                select_store(out + static_cast<size_t>(i0 + u * kEwBlock) * kEwVec, rx[u], ry[u], rc[u]);
        } else {
            for (uint32_t i = i0; i < n_vec; i += kEwBlock) {
                T rx[kEwVec], ry[kEwVec];
                uint8_t rc[kEwVec];
                const size_t e = static_cast<size_t>(i) * kEwVec;
                load_op<XM, true>(XM == kEwRepeat ? x : x + e, rx);
                load_op<YM, true>(YM == kEwRepeat ? y : y + e, ry);
                load_op<kEwDense, true>(c + e, rc);
                select_store(out + e, rx, ry, rc);
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n - n_vec * kEwVec)) {
        uint32_t t = n_vec * kEwVec + threadIdx.x;
        out[t] = c[t] ? x[XM == kEwRepeat ? 0 : t] : y[YM == kEwRepeat ? 0 : t];
    }
}

// plan operands: 0 = x, 1 = y, 2 = cond, 3 = out. XM / YM: how x and y walk the innermost run
// (VEC == 4 only; the condition walks it densely).
template <typename T, int VEC, int UNR, int XM, int YM>
__global__ __launch_bounds__(kEwBlock) void where_nd_kernel(EwIndexArg<4, VEC> pl, EwUnrollDim<4> ud,
                                                            const T *__restrict__ x,
                                                            const T *__restrict__ y,
                                                            const uint8_t *__restrict__ c,
                                                            T *__restrict__ out, uint32_t n_items) {
    if constexpr (VEC == 1) {
        const uint32_t step = gridDim.x * kEwBlock;
        for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_items; i += step) {
            int64_t offs[4];
            nd_offsets<4>(pl, i, offs);
            out[offs[3]] = c[offs[2]] ? x[offs[0]] : y[offs[1]];
        }
    } else {
        // one trip: the grid covers n_items; lanes past the end work on item 0 and do not store
        const uint32_t i_raw = blockIdx.x * kEwBlock + threadIdx.x;
        const bool live = i_raw < n_items;
        const uint32_t i = live ? i_raw : 0;
        int32_t offs[4];
        nd4_offsets<4>(pl, i, offs);
        T rx[UNR][kEwVec], ry[UNR][kEwVec];
        uint8_t rc[UNR][kEwVec];
        // An operand that does not change along the lane's UNR positions is loaded once: thousands
        // of wavefronts asking for the same few lines of a small broadcast operand are a queue of
        // their own in the L2 (see binary_nd_kernel).
        if (UNR > 1 && ud.stride[1] == 0) {
            load_op<YM, false>(y + offs[1], ry[0]);
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                load_op<XM, true>(x + (offs[0] + u * ud.stride[0]), rx[u]);
                load_op<kEwDense, true>(c + (offs[2] + u * ud.stride[2]), rc[u]);
            }
#pragma unroll
            for (int u = 1; u < UNR; ++u)
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) ry[u][j] = ry[0][j];
        } else if (UNR > 1 && ud.stride[0] == 0) {
            load_op<XM, false>(x + offs[0], rx[0]);
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                load_op<YM, true>(y + (offs[1] + u * ud.stride[1]), ry[u]);
                load_op<kEwDense, true>(c + (offs[2] + u * ud.stride[2]), rc[u]);
            }
#pragma unroll
            for (int u = 1; u < UNR; ++u)
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) rx[u][j] = rx[0][j];
        } else {
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                load_op<XM, true>(x + (offs[0] + u * ud.stride[0]), rx[u]);
                load_op<YM, true>(y + (offs[1] + u * ud.stride[1]), ry[u]);
                load_op<kEwDense, true>(c + (offs[2] + u * ud.stride[2]), rc[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u)
            if (live) select_store(out + (offs[3] + u * ud.stride[3]), rx[u], ry[u], rc[u]);
    }
}

// bit 0: x repeats one element along the innermost run, bit 1: y does (the condition never)
constexpr uint32_t kWhereModes = (1u << 0) | (1u << 1) | (1u << 2) | (1u << 3);

template <typename T, int XM, int YM>
void launch_where_mode(hipStream_t stream, const EwDecision<4> &dec, const T *x, const T *y,
                       const uint8_t *c, T *out) {
    if (dec.shape == EwShape::Flat) {
        where_flat_kernel<T, XM, YM><<<chunk_grid(dec.n_items / kEwVec, kEwChunk), kEwBlock, 0, stream>>>(
            x, y, c, out, dec.n_items);
    } else {
        const unsigned grid = (dec.n_items + kEwBlock - 1) / kEwBlock;      // one trip
        if (dec.unrolled)
            where_nd_kernel<T, kEwVec, kEwUnroll, XM, YM><<<grid, kEwBlock, 0, stream>>>(
                dec.index, dec.udim, x, y, c, out, dec.n_items);
        else
            where_nd_kernel<T, kEwVec, 1, XM, YM><<<grid, kEwBlock, 0, stream>>>(
                dec.index, dec.udim, x, y, c, out, dec.n_items);
    }
}

template <typename T>
int32_t launch_where(hipStream_t stream, int rank, const int64_t *shape,
                     const int64_t (*strides)[kMaxRank], const T *x, const T *y, const uint8_t *c,
                     T *out) {
    EwDecision<4> dec;
    const void *ptrs[4] = {x, y, c, out};
    const int sizes[4] = {static_cast<int>(sizeof(T)), static_cast<int>(sizeof(T)), 1,
                          static_cast<int>(sizeof(T))};
    if (!ew_decide<4>(dec, rank, shape, strides, ptrs, sizes, kWhereModes)) return RMLK_OK;
    if (dec.shape == EwShape::Nd1) {
        where_nd_kernel<T, 1, 1, kEwDense, kEwDense><<<grid_for(dec.n_items, kEwBlock, 16), kEwBlock, 0, stream>>>(
            dec.plan, dec.udim, x, y, c, out, dec.n_items);
    } else {
        switch (dec.mode_bits) {
            case 0: launch_where_mode<T, kEwDense, kEwDense>(stream, dec, x, y, c, out); break;
            case 1: launch_where_mode<T, kEwRepeat, kEwDense>(stream, dec, x, y, c, out); break;
            case 2: launch_where_mode<T, kEwDense, kEwRepeat>(stream, dec, x, y, c, out); break;
            default: launch_where_mode<T, kEwRepeat, kEwRepeat>(stream, dec, x, y, c, out); break;
        }
    }
    return launch_status();
}

template <typename T>
int32_t run_where(hipStream_t s, int rank, const int64_t *shape, const int64_t (*st)[kMaxRank],
                  const void *x, const void *y, const void *c, void *out) {
    return for_each_piece<4>(
        rank, shape, st,
        [&](int r, const int64_t *shp, const int64_t (*str)[kMaxRank], const int64_t *offs) {
            return launch_where<T>(s, r, shp, str, static_cast<const T *>(x) + offs[0],
                                   static_cast<const T *>(y) + offs[1],
                                   static_cast<const uint8_t *>(c) + offs[2],
                                   static_cast<T *>(out) + offs[3]);
        });
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_where(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *out_shape,
                                  const rmlk_dims *x_stride, const rmlk_dims *y_stride,
                                  const rmlk_dims *cond_stride, const void *x, const void *y,
                                  const void *cond, void *out) {
    if (!dims_ok(out_shape) || !dims_ok(x_stride) || !dims_ok(y_stride) || !dims_ok(cond_stride))
        return RMLK_ERR_BAD_RANK;
    const int rank = out_shape->rank;
    if (x_stride->rank != rank || y_stride->rank != rank || cond_stride->rank != rank)
        return RMLK_ERR_SIZE_MISMATCH;
    int64_t numel = dims_numel(out_shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!x || !y || !cond || !out) return RMLK_ERR_NULL_POINTER;
    int64_t st[4][kMaxRank];
    for (int d = 0; d < rank; ++d) {
        if (x_stride->v[d] < 0 || y_stride->v[d] < 0 || cond_stride->v[d] < 0)
            return RMLK_ERR_INVALID_ARGUMENT;
        st[0][d] = x_stride->v[d];
        st[1][d] = y_stride->v[d];
        st[2][d] = cond_stride->v[d];
    }
    dense_strides(rank, out_shape->v, st[3]);
    if (numel <= kBatchMaxElems && batch_collecting() && dtype_size(dtype) != 0) {
        // (a tiny select on a stream that is collecting its launches)
        SmallOp so{};
        so.kind = kSmallWhere;
        so.dt = dtype_size(dtype);
        so.in[0] = x;
        so.in[1] = y;
        so.in[2] = cond;
        so.out = out;
        if (small_op_layout(so, rank, out_shape->v, 3, st) && batch_take(as_stream_collecting(stream), so))
            return RMLK_OK;
    }
    hipStream_t s = as_stream(stream);
    switch (dtype_size(dtype)) {
        case 1: return run_where<uint8_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 2: return run_where<uint16_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 4: return run_where<uint32_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 8: return run_where<uint64_t>(s, rank, out_shape->v, st, x, y, cond, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}
