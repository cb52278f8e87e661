// Where: out = cond ? x : y with three-way broadcast. A pure move, so it is instantiated per
// element size, not per dtype. Replaces cuda/src/ptx/where.cu:4-12
// (cuda/src/ptx/headers/ternary_op_macro.cuh:1-34).
#include "elementwise.hpp"

namespace rmlk {
namespace {

template <typename T>
__global__ __launch_bounds__(kEwBlock) void where_flat_kernel(const T *__restrict__ x,
                                                              const T *__restrict__ y,
                                                              const uint8_t *__restrict__ c,
                                                              T *__restrict__ out, uint32_t n,
                                                              int x_b, int y_b, int c_b) {
    const uint32_t n_vec = n / kEwVec;
    const uint32_t step = gridDim.x * kEwBlock;
    for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_vec; i += step) {
        T rx[kEwVec], ry[kEwVec], ro[kEwVec];
        uint8_t rc[kEwVec];
        size_t e = static_cast<size_t>(i) * kEwVec;
        load_vec(x_b ? x : x + e, x_b != 0, rx);
        load_vec(y_b ? y : y + e, y_b != 0, ry);
        load_vec(c_b ? c : c + e, c_b != 0, rc);
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) ro[j] = rc[j] ? rx[j] : ry[j];
        store_vec(out + e, ro);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n - n_vec * kEwVec)) {
        uint32_t i = n_vec * kEwVec + threadIdx.x;
        out[i] = c[c_b ? 0 : i] ? x[x_b ? 0 : i] : y[y_b ? 0 : i];
    }
}

// plan operands: 0 = x, 1 = y, 2 = cond, 3 = out
template <typename T, int VEC>
__global__ __launch_bounds__(kEwBlock) void where_nd_kernel(NdPlan<4> pl, const T *__restrict__ x,
                                                            const T *__restrict__ y,
                                                            const uint8_t *__restrict__ c,
                                                            T *__restrict__ out, uint32_t n_items,
                                                            int x0, int y0, int c0) {
    const uint32_t step = gridDim.x * kEwBlock;
    for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_items; i += step) {
        int64_t offs[4];
        nd_offsets<4>(pl, i, offs);
        if constexpr (VEC == 1) {
            out[offs[3]] = c[offs[2]] ? x[offs[0]] : y[offs[1]];
        } else {
            T rx[kEwVec], ry[kEwVec], ro[kEwVec];
            uint8_t rc[kEwVec];
            load_vec(x + offs[0], x0 != 0, rx);
            load_vec(y + offs[1], y0 != 0, ry);
            load_vec(c + offs[2], c0 != 0, rc);
#pragma unroll
            for (int j = 0; j < kEwVec; ++j) ro[j] = rc[j] ? rx[j] : ry[j];
            store_vec(out + offs[3], ro);
        }
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
    if (!ew_decide<4>(dec, rank, shape, strides, ptrs, sizes)) return RMLK_OK;
    unsigned grid;
    switch (dec.shape) {
        case EwShape::Flat:
            grid = grid_for(dec.n_items / kEwVec + 1, kEwBlock, 16);
            where_flat_kernel<T><<<grid, kEwBlock, 0, stream>>>(x, y, c, out, dec.n_items,
                                                                dec.inner0[0], dec.inner0[1],
                                                                dec.inner0[2]);
            break;
        case EwShape::Nd4:
            grid = grid_for(dec.n_items, kEwBlock, 16);
            where_nd_kernel<T, kEwVec><<<grid, kEwBlock, 0, stream>>>(
                dec.plan, x, y, c, out, dec.n_items, dec.inner0[0], dec.inner0[1], dec.inner0[2]);
            break;
        case EwShape::Nd1:
            grid = grid_for(dec.n_items, kEwBlock, 16);
            where_nd_kernel<T, 1><<<grid, kEwBlock, 0, stream>>>(dec.plan, x, y, c, out,
                                                                 dec.n_items, 0, 0, 0);
            break;
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
    hipStream_t s = as_stream(stream);
    switch (dtype_size(dtype)) {
        case 1: return run_where<uint8_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 2: return run_where<uint16_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 4: return run_where<uint32_t>(s, rank, out_shape->v, st, x, y, cond, out);
        case 8: return run_where<uint64_t>(s, rank, out_shape->v, st, x, y, cond, out);
        default: return RMLK_ERR_UNSUPPORTED;
    }
}
