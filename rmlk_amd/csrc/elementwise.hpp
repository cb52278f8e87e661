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
#ifndef RMLK_EW_UNROLL
#define RMLK_EW_UNROLL 4
#endif
#ifndef RMLK_EW_BLOCKS_PER_CU
#define RMLK_EW_BLOCKS_PER_CU 8
#endif
constexpr int kEwUnroll = RMLK_EW_UNROLL;  // independent vector accesses in flight per lane
constexpr int kEwBlocksPerCu = RMLK_EW_BLOCKS_PER_CU;

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
        // Dense operands are read once: streaming loads for element sizes up to 4 bytes (two dense
        // 256 MiB float inputs: 112 -> 96 us; 8-byte elements measured slower that way, 218 -> 238 us)
        V v;
        if constexpr (sizeof(T) <= 4) v = nt_load(reinterpret_cast<const V *>(p));
        else v = *reinterpret_cast<const V *>(p);
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
    *reinterpret_cast<V *>(p) = v;   // (results are usually read next: ordinary stores)
}

// ---- two inputs ------------------------------------------------------------------------------
template <typename F, typename TA, typename TB, typename TO>
__global__ __launch_bounds__(kEwBlock) void binary_flat_kernel(const TA *__restrict__ a,
                                                               const TB *__restrict__ b,
                                                               TO *__restrict__ out, uint32_t n,
                                                               int a_bcast, int b_bcast) {
    const uint32_t n_vec = n / kEwVec;
    const uint32_t step = gridDim.x * kEwBlock;
    uint32_t i = blockIdx.x * kEwBlock + threadIdx.x;
    // main loop: kEwUnroll independent 128-bit accesses per operand in flight per lane
    for (; i + (kEwUnroll - 1) * step < n_vec; i += kEwUnroll * step) {
        TA ra[kEwUnroll][kEwVec];
        TB rb[kEwUnroll][kEwVec];
#pragma unroll
        for (int u = 0; u < kEwUnroll; ++u) {
            const size_t e = static_cast<size_t>(i + u * step) * kEwVec;
            load_vec(a_bcast ? a : a + e, a_bcast != 0, ra[u]);
            load_vec(b_bcast ? b : b + e, b_bcast != 0, rb[u]);
        }
#pragma unroll
        for (int u = 0; u < kEwUnroll; ++u) {
            TO ro[kEwVec];
#pragma unroll
            for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[u][j], rb[u][j]);
            store_vec(out + static_cast<size_t>(i + u * step) * kEwVec, ro);
        }
    }
    for (; i < n_vec; i += step) {
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
        uint32_t t = n_vec * kEwVec + threadIdx.x;
        out[t] = F::apply(a[a_bcast ? 0 : t], b[b_bcast ? 0 : t]);
    }
}

// Unroll descriptor of the nd<4> kernels: a lane handles kEwUnroll positions along one outer
// dim (the host has divided that dim by kEwUnroll in the plan), so the index decomposition is
// shared and an operand that is broadcast along that dim is loaded once.
template <int NP>
struct EwUnrollDim {
    int32_t stride[NP];  // element stride of the unroll dim per operand (0 = broadcast)
};

// plan operands: 0 = a, 1 = b, 2 = out. For VEC == 4 the host has divided the innermost dim by 4
// and multiplied the innermost strides by 4; a_inner0 / b_inner0 say the operand repeats one
// element along the innermost run. UNR is kEwUnroll (positions along the unroll dim) or 1.
template <typename F, typename TA, typename TB, typename TO, int VEC, int UNR>
__global__ __launch_bounds__(kEwBlock) void binary_nd_kernel(NdPlan<3> pl, EwUnrollDim<3> ud,
                                                             const TA *__restrict__ a,
                                                             const TB *__restrict__ b,
                                                             TO *__restrict__ out, uint32_t n_items,
                                                             int a_inner0, int b_inner0) {
    const uint32_t step = gridDim.x * kEwBlock;
    uint32_t i = blockIdx.x * kEwBlock + threadIdx.x;
    if constexpr (VEC == 1) {
        for (; i < n_items; i += step) {
            int64_t offs[3];
            nd_offsets<3>(pl, i, offs);
            out[offs[2]] = F::apply(a[offs[0]], b[offs[1]]);
        }
    } else {
        for (; i < n_items; i += step) {
            int64_t offs[3];
            nd_offsets<3>(pl, i, offs);
            TA ra[UNR][kEwVec];
            TB rb[UNR][kEwVec];
            load_vec(a + offs[0], a_inner0 != 0, ra[0]);
            load_vec(b + offs[1], b_inner0 != 0, rb[0]);
#pragma unroll
            for (int u = 1; u < UNR; ++u) {
                if (ud.stride[0] != 0) {
                    load_vec(a + offs[0] + static_cast<int64_t>(u) * ud.stride[0], a_inner0 != 0,
                             ra[u]);
                } else {
#pragma unroll
                    for (int j = 0; j < kEwVec; ++j) ra[u][j] = ra[0][j];
                }
                if (ud.stride[1] != 0) {
                    load_vec(b + offs[1] + static_cast<int64_t>(u) * ud.stride[1], b_inner0 != 0,
                             rb[u]);
                } else {
#pragma unroll
                    for (int j = 0; j < kEwVec; ++j) rb[u][j] = rb[0][j];
                }
            }
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                TO ro[kEwVec];
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[u][j], rb[u][j]);
                store_vec(out + offs[2] + static_cast<int64_t>(u) * ud.stride[2], ro);
            }
        }
    }
}

// Host-side analysis shared by binary / where launchers.
// Fills the plan from broadcast strides, then decides which kernel shape applies.
enum class EwShape { Flat, Nd4, Nd1 };

template <int NP>
struct EwDecision {
    EwShape shape;
    NdPlan<NP> plan;
    int inner0[NP];     // operand repeats one element along the innermost run
    uint32_t n_items;   // loop trip count of the chosen kernel
    bool unrolled;      // nd<4> only: an outer dim was divided by kEwUnroll
    EwUnrollDim<NP> udim;
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
        dec.unrolled = false;
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
        // unroll dim: an outer dim divisible by kEwUnroll, preferring one along which an input is
        // broadcast (its loads are then shared), then the innermost such dim (nearby addresses)
        int best = -1;
        bool best_bcast = false;
        for (int d = last - 1; d >= 0; --d) {
            if (pl.dim64[d] % kEwUnroll) continue;
            bool bc = false;
            for (int p = 0; p < NP - 1; ++p)
                if (pl.stride[p][d] == 0) bc = true;
            if (best < 0 || (bc && !best_bcast)) {
                best = d;
                best_bcast = bc;
            }
        }
        dec.unrolled = best >= 0;
        for (int p = 0; p < NP; ++p) dec.udim.stride[p] = 0;
        if (dec.unrolled) {
            // keep the low positions adjacent: position = u * (dim / U) + i, i.e. the lane's
            // kEwUnroll positions are dim / U apart and consecutive lanes stay consecutive
            const int64_t sub = pl.dim64[best] / kEwUnroll;
            for (int p = 0; p < NP; ++p) {
                int64_t us = static_cast<int64_t>(pl.stride[p][best]) * sub;
                if (us >= kStrideLimit || us <= -kStrideLimit) dec.unrolled = false;
            }
            if (dec.unrolled) {
                for (int p = 0; p < NP; ++p)
                    dec.udim.stride[p] = static_cast<int32_t>(pl.stride[p][best] * sub);
                pl.dim64[best] = sub;
                pl.dim[best] = static_cast<uint32_t>(sub);
                pl.fdiv[best] = FastDiv(pl.dim[best]);
                dec.n_items /= kEwUnroll;
            }
        }
        return true;
    }
    dec.shape = EwShape::Nd1;
    dec.unrolled = false;
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
            unsigned grid = grid_for(dec.n_items / (kEwVec * kEwUnroll) + 1, kEwBlock, kEwBlocksPerCu);
            binary_flat_kernel<F, TA, TB, TO><<<grid, kEwBlock, 0, stream>>>(
                pa, pb, po, dec.n_items, dec.inner0[0], dec.inner0[1]);
            break;
        }
        case EwShape::Nd4: {
            unsigned grid = grid_for(dec.n_items, kEwBlock, kEwBlocksPerCu);
            if (dec.unrolled)
                binary_nd_kernel<F, TA, TB, TO, kEwVec, kEwUnroll><<<grid, kEwBlock, 0, stream>>>(
                    dec.plan, dec.udim, pa, pb, po, dec.n_items, dec.inner0[0], dec.inner0[1]);
            else
                binary_nd_kernel<F, TA, TB, TO, kEwVec, 1><<<grid, kEwBlock, 0, stream>>>(
                    dec.plan, dec.udim, pa, pb, po, dec.n_items, dec.inner0[0], dec.inner0[1]);
            break;
        }
        case EwShape::Nd1: {
            unsigned grid = grid_for(dec.n_items, kEwBlock, 16);
            binary_nd_kernel<F, TA, TB, TO, 1, 1><<<grid, kEwBlock, 0, stream>>>(
                dec.plan, dec.udim, pa, pb, po, dec.n_items, 0, 0);
            break;
        }
    }
    return launch_status();
}

// Runs fn(rank, shape, strides, elem_offsets) once per piece of at most kPieceElems elements;
// elem_offsets[p] is the element offset to add to operand p's base pointer.
template <int NP, typename Fn>
inline int32_t for_each_piece(int rank, const int64_t *shape, const int64_t (*strides)[kMaxRank],
                              Fn &&fn) {
    int64_t zero[NP] = {0};
    return split_pieces<NP>(rank, shape, strides, zero,
                            [&](const int64_t *shp, const int64_t *offs) {
                                return fn(rank, shp, strides, offs);
                            });
}

}  // namespace rmlk
