// Broadcast element-wise engine shared by the binary, compare, pow and where kernels.
//
// Three kernel shapes per (functor, types):
//   flat   : every operand is dense or a broadcast scalar and 16-byte aligned; 4 elements per
//            lane per step as one 128-bit access, scalar tail.
//   nd<4>  : coalesced rank > 1 whose innermost run is a multiple of 4 and is walked with stride
//            0 or 1 by every operand; 128-bit accesses, outer coordinates through FastDiv.
//   nd<1>  : anything else (odd inner runs, unaligned pointers, strided inner dims).
#pragma once

#include "nd_index.hpp"

namespace rmlk {

constexpr int kEwBlock = 256;
constexpr int kEwVec = 4;

template <typename T>
struct VecOf {
    using type = Vec<T, kEwVec>;
};

template <typename T>
__device__ __forceinline__ void load_vec(const T *p, bool bcast, T (&r)[kEwVec]) {
    if (bcast) {
        T s = *p;
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) r[j] = s;
    } else {
        using V = Vec<T, kEwVec>;
        V v = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) r[j] = v.v[j];
    }
}

template <typename T>
__device__ __forceinline__ void store_vec(T *p, const T (&r)[kEwVec]) {
    using V = Vec<T, kEwVec>;
    V v;
#pragma unroll
    for (int j = 0; j < kEwVec; ++j) v.v[j] = r[j];
    *reinterpret_cast<V *>(p) = v;
}

// ---- two inputs ------------------------------------------------------------------------------
template <typename F, typename TA, typename TB, typename TO>
__global__ __launch_bounds__(kEwBlock) void binary_flat_kernel(const TA *__restrict__ a,
                                                               const TB *__restrict__ b,
                                                               TO *__restrict__ out, uint32_t n,
                                                               int a_bcast, int b_bcast) {
    const uint32_t n_vec = n / kEwVec;
    const uint32_t step = gridDim.x * kEwBlock;
    for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_vec; i += step) {
        TA ra[kEwVec];
        TB rb[kEwVec];
        TO ro[kEwVec];
        load_vec(a_bcast ? a : a + static_cast<size_t>(i) * kEwVec, a_bcast != 0, ra);
        load_vec(b_bcast ? b : b + static_cast<size_t>(i) * kEwVec, b_bcast != 0, rb);
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[j], rb[j]);
        store_vec(out + static_cast<size_t>(i) * kEwVec, ro);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n - n_vec * kEwVec)) {
        uint32_t i = n_vec * kEwVec + threadIdx.x;
        out[i] = F::apply(a[a_bcast ? 0 : i], b[b_bcast ? 0 : i]);
    }
}

// plan operands: 0 = a, 1 = b, 2 = out. For VEC == 4 the host has divided the innermost dim by 4
// and multiplied the innermost strides by 4; a_inner0 / b_inner0 say the operand repeats one
// element along the innermost run.
template <typename F, typename TA, typename TB, typename TO, int VEC>
__global__ __launch_bounds__(kEwBlock) void binary_nd_kernel(NdPlan<3> pl,
                                                             const TA *__restrict__ a,
                                                             const TB *__restrict__ b,
                                                             TO *__restrict__ out, uint32_t n_items,
                                                             int a_inner0, int b_inner0) {
    const uint32_t step = gridDim.x * kEwBlock;
    for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_items; i += step) {
        int64_t offs[3];
        nd_offsets<3>(pl, i, offs);
        if constexpr (VEC == 1) {
            out[offs[2]] = F::apply(a[offs[0]], b[offs[1]]);
        } else {
            TA ra[kEwVec];
            TB rb[kEwVec];
            TO ro[kEwVec];
            load_vec(a + offs[0], a_inner0 != 0, ra);
            load_vec(b + offs[1], b_inner0 != 0, rb);
#pragma unroll
            for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[j], rb[j]);
            store_vec(out + offs[2], ro);
        }
    }
}

struct BinaryOperand {
    const void *ptr;
    int elem_size;
};

// Host-side analysis shared by binary / where launchers.
// Fills the plan from broadcast strides, then decides which kernel shape applies.
enum class EwShape { Flat, Nd4, Nd1 };

template <int NP>
struct EwDecision {
    EwShape shape;
    NdPlan<NP> plan;
    int inner0[NP];     // operand repeats one element along the innermost run
    uint32_t n_items;   // loop trip count of the chosen kernel
};

// ptrs/elem sizes for the NP operands (output last). Returns false for empty work.
template <int NP>
inline bool ew_decide(EwDecision<NP> &dec, int rank, const int64_t *shape,
                      const int64_t (*strides)[kMaxRank], const void *const *ptrs,
                      const int *elem_sizes) {
    NdPlan<NP> &pl = dec.plan;
    if (!build_plan<NP>(pl, rank, shape, strides)) return false;
    const int last = pl.rank - 1;
    bool aligned = true;
    bool inner_unit = true;  // every operand walks the innermost run with stride 0 or 1
    for (int p = 0; p < NP; ++p) {
        int64_t s = pl.stride[p][last];
        dec.inner0[p] = (s == 0);
        if (s != 0 && s != 1) inner_unit = false;
        if (s == 1) {
            size_t vec_bytes = static_cast<size_t>(elem_sizes[p]) * kEwVec;
            if (vec_bytes > 16) vec_bytes = 16;
            if (reinterpret_cast<uintptr_t>(ptrs[p]) % vec_bytes) aligned = false;
            for (int d = 0; d < last; ++d)
                if (pl.stride[p][d] % kEwVec) aligned = false;
        }
    }
    if (pl.rank == 1 && inner_unit && aligned) {
        dec.shape = EwShape::Flat;
        dec.n_items = static_cast<uint32_t>(pl.numel);
        return true;
    }
    if (pl.rank > 1 && inner_unit && aligned && pl.dim64[last] % kEwVec == 0) {
        dec.shape = EwShape::Nd4;
        pl.dim64[last] /= kEwVec;
        pl.dim[last] = static_cast<uint32_t>(pl.dim64[last]);
        pl.fdiv[last] = FastDiv(pl.dim[last]);
        for (int p = 0; p < NP; ++p) pl.stride[p][last] *= kEwVec;
        dec.n_items = static_cast<uint32_t>(pl.numel / kEwVec);
        return true;
    }
    dec.shape = EwShape::Nd1;
    dec.n_items = static_cast<uint32_t>(pl.numel);
    return true;
}

template <typename F, typename TA, typename TB, typename TO>
inline int32_t launch_binary_typed(hipStream_t stream, int rank, const int64_t *shape,
                                   const int64_t (*strides)[kMaxRank], const void *a,
                                   const void *b, void *out) {
    EwDecision<3> dec;
    const void *ptrs[3] = {a, b, out};
    const int sizes[3] = {static_cast<int>(sizeof(TA)), static_cast<int>(sizeof(TB)),
                          static_cast<int>(sizeof(TO))};
    if (!ew_decide<3>(dec, rank, shape, strides, ptrs, sizes)) return RMLK_OK;
    const TA *pa = static_cast<const TA *>(a);
    const TB *pb = static_cast<const TB *>(b);
    TO *po = static_cast<TO *>(out);
    switch (dec.shape) {
        case EwShape::Flat: {
            unsigned grid = grid_for(dec.n_items / kEwVec + 1, kEwBlock, 16);
            binary_flat_kernel<F, TA, TB, TO><<<grid, kEwBlock, 0, stream>>>(
                pa, pb, po, dec.n_items, dec.inner0[0], dec.inner0[1]);
            break;
        }
        case EwShape::Nd4: {
            unsigned grid = grid_for(dec.n_items, kEwBlock, 16);
            binary_nd_kernel<F, TA, TB, TO, kEwVec><<<grid, kEwBlock, 0, stream>>>(
                dec.plan, pa, pb, po, dec.n_items, dec.inner0[0], dec.inner0[1]);
            break;
        }
        case EwShape::Nd1: {
            unsigned grid = grid_for(dec.n_items, kEwBlock, 16);
            binary_nd_kernel<F, TA, TB, TO, 1><<<grid, kEwBlock, 0, stream>>>(
                dec.plan, pa, pb, po, dec.n_items, 0, 0);
            break;
        }
    }
    return launch_status();
}

// Validates the C-ABI arguments of a broadcast op and splits work that exceeds the 32-bit index
// range of the kernels along the outermost dim. `fn(rank, shape, strides, elem_offsets)` launches
// one piece; elem_offsets[p] is the element offset to add to operand p's base pointer.
template <int NP, typename Fn>
inline int32_t for_each_piece(int rank, const int64_t *shape, const int64_t (*strides)[kMaxRank],
                              Fn &&fn) {
    int64_t numel = 1;
    for (int d = 0; d < rank; ++d) {
        if (shape[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (shape[d] == 0) return RMLK_OK;
    }
    for (int d = 0; d < rank; ++d) {
        if (numel > kMaxElems / shape[d]) return RMLK_ERR_TOO_LARGE;
        numel *= shape[d];
    }
    constexpr int64_t kLimit = (int64_t)1 << 30;  // elements per launch (index math is 32-bit)
    if (numel <= kLimit) {
        int64_t zero[NP] = {0};
        return fn(rank, shape, strides, zero);
    }
    // find the outermost dim that is > 1 and split it
    int d0 = 0;
    while (d0 < rank - 1 && shape[d0] == 1) ++d0;
    int64_t inner = numel / shape[d0];
    if (inner > kLimit) return RMLK_ERR_TOO_LARGE;
    int64_t rows_per = kLimit / inner;
    if (rows_per < 1) rows_per = 1;
    int64_t sub_shape[kMaxRank];
    for (int d = 0; d < rank; ++d) sub_shape[d] = shape[d];
    for (int64_t r0 = 0; r0 < shape[d0]; r0 += rows_per) {
        int64_t rows = shape[d0] - r0 < rows_per ? shape[d0] - r0 : rows_per;
        sub_shape[d0] = rows;
        int64_t offs[NP];
        for (int p = 0; p < NP; ++p) offs[p] = r0 * strides[p][d0];
        int32_t st = fn(rank, sub_shape, strides, offs);
        if (st != RMLK_OK) return st;
    }
    return RMLK_OK;
}

}  // namespace rmlk
