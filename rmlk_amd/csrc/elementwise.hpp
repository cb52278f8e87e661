// Broadcast element-wise engine shared by the binary, compare, pow and where kernels.
//
// Three kernel shapes per (functor, types):
//   flat   : every operand is dense or a broadcast scalar and 16-byte aligned; 4 elements per
//            lane per access (128 bits for 4-byte elements), a block working through chunks of
//            block x unroll consecutive vectors, scalar tail.
//   nd<4>  : coalesced rank > 1 whose innermost run is a multiple of 4 and is walked with stride
//            0 or 1 by every operand; 128-bit accesses, outer coordinates through FastDiv, a lane
//            taking kEwUnroll ADJACENT positions along one outer dim.
//   nd<1>  : anything else (odd inner runs, unaligned pointers, strided inner dims).
// How an input walks the innermost run (a vector per access, or one element repeated) is a template
// argument of the flat and nd<4> kernels, not a run-time flag: a run-time choice between a scalar
// and a vector load puts a branch between any two loads of a lane, and the compiler then waits for
// everything in flight at every such join, which leaves ONE load in flight per wavefront (the
// 64 MiB broadcast Add took 16.4 us that way, 12 us with its eight loads issued together).
// The vector kernels write with streaming stores.
#pragma once

#include <type_traits>

#include "nd_index.hpp"

namespace rmlk {

constexpr int kEwBlock = 256;
constexpr int kEwVec = 4;
constexpr int kEwUnroll = 4;       // independent vector accesses in flight per lane and operand
constexpr int kEwChunk = kEwBlock * kEwUnroll;      // vectors a block of the flat kernel takes per trip

// An input's way through the innermost run.
constexpr int kEwDense = 0;    // consecutive elements: one vector access
constexpr int kEwRepeat = 1;   // one element repeated (stride 0): one scalar access

template <typename T>
struct VecOf {
    using type = Vec<T, kEwVec>;
};

// STREAM: the operand is read once by the whole grid (a dense operand of a flat kernel): streaming
// loads for element sizes up to 4 bytes.
template <int MODE, bool STREAM, typename T>
__device__ __forceinline__ void load_op(const T *p, T (&r)[kEwVec]) {
    if constexpr (MODE == kEwRepeat) {
        T s = *p;
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) r[j] = s;
    } else {
        using V = Vec<T, kEwVec>;
        V v;
        if constexpr (STREAM && sizeof(T) <= 4) v = nt_load(reinterpret_cast<const V *>(p));
        else v = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int j = 0; j < kEwVec; ++j) r[j] = v.v[j];
    }
}

// Results are written with streaming stores: they leave the chip as they are produced instead of
// waiting in the L2s for the write-back at the end of the kernel (the L2s of the eight XCDs are not
// coherent with one another, so the next kernel finds little there anyway). A run-time choice
// between the two kinds of store does not survive the optimiser: it merges the two stores of the
// branches into one ordinary store.
template <typename T>
__device__ __forceinline__ void store_vec(T *p, const T (&r)[kEwVec]) {
    using V = Vec<T, kEwVec>;
    V v;
#pragma unroll
    for (int j = 0; j < kEwVec; ++j) v.v[j] = r[j];
    nt_store(reinterpret_cast<V *>(p), v);
}

// ---- two inputs ------------------------------------------------------------------------------
// AM / BM: kEwDense (n elements) or kEwRepeat (one element for the whole output).
template <typename F, typename TA, typename TB, typename TO, int AM, int BM>
__global__ __launch_bounds__(kEwBlock) void binary_flat_kernel(const TA *__restrict__ a,
                                                               const TB *__restrict__ b,
                                                               TO *__restrict__ out, uint32_t n) {
    const uint32_t n_vec = n / kEwVec;
    for (uint32_t base = blockIdx.x * kEwChunk; base < n_vec; base += gridDim.x * kEwChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kEwChunk <= n_vec) {
            // whole chunk: kEwUnroll independent accesses per operand in flight per lane
            TA ra[kEwUnroll][kEwVec];
            TB rb[kEwUnroll][kEwVec];
#pragma unroll
            for (int u = 0; u < kEwUnroll; ++u) {
                const size_t e = static_cast<size_t>(i0 + u * kEwBlock) * kEwVec;
                load_op<AM, true>(AM == kEwRepeat ? a : a + e, ra[u]);
                load_op<BM, true>(BM == kEwRepeat ? b : b + e, rb[u]);
            }
#pragma unroll
            for (int u = 0; u < kEwUnroll; ++u) {
                TO ro[kEwVec];
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[u][j], rb[u][j]);
                store_vec(out + static_cast<size_t>(i0 + u * kEwBlock) * kEwVec, ro);
            }
        } else {
            for (uint32_t i = i0; i < n_vec; i += kEwBlock) {
                TA ra[kEwVec];
                TB rb[kEwVec];
                TO ro[kEwVec];
                const size_t e = static_cast<size_t>(i) * kEwVec;
                load_op<AM, true>(AM == kEwRepeat ? a : a + e, ra);
                load_op<BM, true>(BM == kEwRepeat ? b : b + e, rb);
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[j], rb[j]);
                store_vec(out + e, ro);
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n - n_vec * kEwVec)) {
        uint32_t t = n_vec * kEwVec + threadIdx.x;
        out[t] = F::apply(a[AM == kEwRepeat ? 0 : t], b[BM == kEwRepeat ? 0 : t]);
    }
}

// Unroll descriptor of the nd<4> kernels: a lane handles kEwUnroll adjacent positions along one
// outer dim (the host has divided that dim by kEwUnroll in the plan and multiplied its strides), so
// the index decomposition is shared and what a block has in flight is one contiguous piece of a
// dense operand. An operand that is broadcast along that dim has stride 0 here: its kEwUnroll
// loads fetch the same vector (from the first-level cache after the first).
template <int NP>
struct EwUnrollDim {
    int32_t stride[NP];  // element stride of the unroll dim per operand (0 = broadcast)
};

// plan operands: 0 = a, 1 = b, 2 = out. For VEC == 4 the host has divided the innermost dim by 4
// and multiplied the innermost strides by 4; AM / BM say how the operand walks the innermost run.
// UNR is kEwUnroll (positions along the unroll dim) or 1. VEC == 1 ignores AM / BM.
template <int NP, int VEC>
using EwIndexArg = std::conditional_t<VEC == 1, NdPlan<NP>, NdIndex4<NP>>;

template <typename F, typename TA, typename TB, typename TO, int VEC, int UNR, int AM, int BM>
__global__ __launch_bounds__(kEwBlock) void binary_nd_kernel(EwIndexArg<3, VEC> pl, EwUnrollDim<3> ud,
                                                             const TA *__restrict__ a,
                                                             const TB *__restrict__ b,
                                                             TO *__restrict__ out, uint32_t n_items) {
    if constexpr (VEC == 1) {
        const uint32_t step = gridDim.x * kEwBlock;
        for (uint32_t i = blockIdx.x * kEwBlock + threadIdx.x; i < n_items; i += step) {
            int64_t offs[3];
            nd_offsets<3>(pl, i, offs);
            out[offs[2]] = F::apply(a[offs[0]], b[offs[1]]);
        }
    } else {
        // one trip: the grid covers n_items (a loop here makes the compiler keep every choice of the
        // index arithmetic live in scalar registers across it, more than there are)
        // (lanes past the end work on item 0 and do not store: an early exit would put the load of
        // n_items and a branch in front of every other kernel-argument load)
        const uint32_t i_raw = blockIdx.x * kEwBlock + threadIdx.x;
        const bool live = i_raw < n_items;
        const uint32_t i = live ? i_raw : 0;
        int32_t offs[3];
        nd4_offsets<3>(pl, i, offs);
        TA ra[UNR][kEwVec];
        TB rb[UNR][kEwVec];
        // An operand that does not change along the lane's UNR positions is loaded once. Thousands of
        // wavefronts asking for the same few lines of a small broadcast operand are a queue of their
        // own in the L2, longest when the lines still have to come from HBM: four loads per lane of
        // an 8 KB b cost the 64 MiB Add 0.4 us with b in the L2 and 1.3 us with b cold.
        if (UNR > 1 && ud.stride[1] == 0) {
            load_op<BM, false>(b + offs[1], rb[0]);
#pragma unroll
            for (int u = 0; u < UNR; ++u) load_op<AM, true>(a + (offs[0] + u * ud.stride[0]), ra[u]);
#pragma unroll
            for (int u = 1; u < UNR; ++u)
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) rb[u][j] = rb[0][j];
        } else if (UNR > 1 && ud.stride[0] == 0) {
            load_op<AM, false>(a + offs[0], ra[0]);
#pragma unroll
            for (int u = 0; u < UNR; ++u) load_op<BM, true>(b + (offs[1] + u * ud.stride[1]), rb[u]);
#pragma unroll
            for (int u = 1; u < UNR; ++u)
#pragma unroll
                for (int j = 0; j < kEwVec; ++j) ra[u][j] = ra[0][j];
        } else {
#pragma unroll
            for (int u = 0; u < UNR; ++u) load_op<AM, true>(a + (offs[0] + u * ud.stride[0]), ra[u]);
#pragma unroll
            for (int u = 0; u < UNR; ++u) load_op<BM, true>(b + (offs[1] + u * ud.stride[1]), rb[u]);
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            TO ro[kEwVec];
#pragma unroll
            for (int j = 0; j < kEwVec; ++j) ro[j] = F::apply(ra[u][j], rb[u][j]);
            if (live) store_vec(out + (offs[2] + u * ud.stride[2]), ro);
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
    NdIndex4<NP> index; // what the nd<4> kernels take
    int inner0[NP];     // operand repeats one element along the innermost run
    int mode_bits;      // bit p set: input p repeats one element along the innermost run
    uint32_t n_items;   // loop trip count of the chosen kernel
    bool unrolled;      // nd<4> only: an outer dim was divided by kEwUnroll
    EwUnrollDim<NP> udim;
};

// ptrs/elem sizes for the NP operands (output last). `modes_with_kernels` has bit m set when the
// caller has flat / nd<4> kernels for the combination m of inputs that repeat one element along the
// innermost run (bit p of m = input p repeats); other combinations take nd<1>. Returns false for
// empty work.
template <int NP>
inline bool ew_decide(EwDecision<NP> &dec, int rank, const int64_t *shape,
                      const int64_t (*strides)[kMaxRank], const void *const *ptrs,
                      const int *elem_sizes, uint32_t modes_with_kernels) {
    NdPlan<NP> &pl = dec.plan;
    if (!build_plan<NP>(pl, rank, shape, strides)) return false;
    const int last = pl.rank - 1;
    bool aligned = true;
    bool inner_unit = true;  // every operand walks the innermost run with stride 0 or 1
    dec.mode_bits = 0;
    for (int p = 0; p < NP; ++p) {
        int64_t s = pl.stride[p][last];
        dec.inner0[p] = (s == 0);
        if (s == 0 && p < NP - 1) dec.mode_bits |= 1 << p;
        if (s != 0 && s != 1) inner_unit = false;
        if (s == 1) {
            size_t vec_bytes = static_cast<size_t>(elem_sizes[p]) * kEwVec;
            if (vec_bytes > 16) vec_bytes = 16;
            if (reinterpret_cast<uintptr_t>(ptrs[p]) % vec_bytes) aligned = false;
            for (int d = 0; d < last; ++d)
                if (pl.stride[p][d] % kEwVec) aligned = false;
        }
    }
    for (int p = 0; p < NP; ++p) dec.udim.stride[p] = 0;
    const bool have_kernel = (modes_with_kernels >> dec.mode_bits) & 1u;
    const bool vector_ok = inner_unit && aligned && have_kernel && !dec.inner0[NP - 1];
    if (pl.rank == 1 && vector_ok) {
        dec.shape = EwShape::Flat;
        dec.unrolled = false;
        dec.n_items = static_cast<uint32_t>(pl.numel);
        return true;
    }
    if (pl.rank > 1 && pl.rank <= kIndexRank && vector_ok && pl.dim64[last] % kEwVec == 0) {
        dec.shape = EwShape::Nd4;
        pl.dim64[last] /= kEwVec;
        pl.dim[last] = static_cast<uint32_t>(pl.dim64[last]);
        pl.fdiv[last] = FastDiv(pl.dim[last]);
        for (int p = 0; p < NP; ++p) pl.stride[p][last] *= kEwVec;
        dec.n_items = static_cast<uint32_t>(pl.numel / kEwVec);
        // unroll dim: the innermost outer dim divisible by kEwUnroll (neighbouring positions are
        // then neighbouring rows of a dense operand)
        int best = -1;
        for (int d = last - 1; d >= 0; --d) {
            if (pl.dim64[d] % kEwUnroll) continue;
            best = d;
            break;
        }
        dec.unrolled = best >= 0;
        if (dec.unrolled) {
            // position along the dim = i * kEwUnroll + u: the lane's positions are neighbours
            for (int p = 0; p < NP; ++p) {
                int64_t us = static_cast<int64_t>(pl.stride[p][best]) * kEwUnroll;
                if (us >= kStrideLimit || us <= -kStrideLimit) dec.unrolled = false;
            }
            if (dec.unrolled) {
                const int64_t sub = pl.dim64[best] / kEwUnroll;
                for (int p = 0; p < NP; ++p) {
                    dec.udim.stride[p] = pl.stride[p][best];
                    pl.stride[p][best] *= kEwUnroll;
                }
                pl.dim64[best] = sub;
                pl.dim[best] = static_cast<uint32_t>(sub);
                pl.fdiv[best] = FastDiv(pl.dim[best]);
                dec.n_items /= kEwUnroll;
            }
        }
        static_assert(kEwVec == 4 && kEwUnroll == 4, "the shifts of the index");
        int inner_shift[NP];
        for (int p = 0; p < NP; ++p) inner_shift[p] = 2;
        make_index4<NP>(dec.index, pl, inner_shift, dec.unrolled ? best : -1, 2);
        return true;
    }
    dec.shape = EwShape::Nd1;
    dec.unrolled = false;
    dec.n_items = static_cast<uint32_t>(pl.numel);
    return true;
}

// modes of two inputs with flat / nd<4> kernels: neither, a, or b repeats along the innermost run
constexpr uint32_t kBinaryModes = (1u << 0) | (1u << 1) | (1u << 2);

template <typename F, typename TA, typename TB, typename TO, int AM, int BM>
inline void launch_binary_mode(hipStream_t stream, const EwDecision<3> &dec, const TA *pa,
                               const TB *pb, TO *po) {
    if (dec.shape == EwShape::Flat) {
        unsigned grid = chunk_grid(dec.n_items / kEwVec, kEwChunk);
        binary_flat_kernel<F, TA, TB, TO, AM, BM><<<grid, kEwBlock, 0, stream>>>(pa, pb, po, dec.n_items);
    } else {
        unsigned grid = (dec.n_items + kEwBlock - 1) / kEwBlock;      // one trip
        if (dec.unrolled)
            binary_nd_kernel<F, TA, TB, TO, kEwVec, kEwUnroll, AM, BM><<<grid, kEwBlock, 0, stream>>>(
                dec.index, dec.udim, pa, pb, po, dec.n_items);
        else
            binary_nd_kernel<F, TA, TB, TO, kEwVec, 1, AM, BM><<<grid, kEwBlock, 0, stream>>>(
                dec.index, dec.udim, pa, pb, po, dec.n_items);
    }
}

template <typename F, typename TA, typename TB, typename TO>
inline int32_t launch_binary_typed(hipStream_t stream, int rank, const int64_t *shape,
                                   const int64_t (*strides)[kMaxRank], const void *a,
                                   const void *b, void *out) {
    EwDecision<3> dec;
    const void *ptrs[3] = {a, b, out};
    const int sizes[3] = {static_cast<int>(sizeof(TA)), static_cast<int>(sizeof(TB)),
                          static_cast<int>(sizeof(TO))};
    if (!ew_decide<3>(dec, rank, shape, strides, ptrs, sizes, kBinaryModes)) return RMLK_OK;
    const TA *pa = static_cast<const TA *>(a);
    const TB *pb = static_cast<const TB *>(b);
    TO *po = static_cast<TO *>(out);
    if (dec.shape == EwShape::Nd1) {
        unsigned grid = grid_for(dec.n_items, kEwBlock, 16);
        binary_nd_kernel<F, TA, TB, TO, 1, 1, kEwDense, kEwDense><<<grid, kEwBlock, 0, stream>>>(
            dec.plan, dec.udim, pa, pb, po, dec.n_items);
    } else if (dec.mode_bits == 0) {
        launch_binary_mode<F, TA, TB, TO, kEwDense, kEwDense>(stream, dec, pa, pb, po);
    } else if (dec.mode_bits == 1) {
        launch_binary_mode<F, TA, TB, TO, kEwRepeat, kEwDense>(stream, dec, pa, pb, po);
    } else {
        launch_binary_mode<F, TA, TB, TO, kEwDense, kEwRepeat>(stream, dec, pa, pb, po);
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
