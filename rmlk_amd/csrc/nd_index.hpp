// Device-side decomposition of a linear index over a coalesced NdPlan into operand offsets.
#pragma once

#include "common.hpp"

namespace rmlk {

// idx < numel (< 2^31). offs[p] receives the element offset of operand p.
template <int NP>
__device__ __forceinline__ void nd_offsets(const NdPlan<NP> &pl, uint32_t idx, int64_t (&offs)[NP]) {
#pragma unroll
    for (int p = 0; p < NP; ++p) offs[p] = 0;
    uint32_t rem = idx;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 1; --d) {
        if (d < pl.rank) {
            uint32_t q = pl.fdiv[d].div(rem);
            uint32_t i = rem - q * pl.dim[d];
            rem = q;
#pragma unroll
            for (int p = 0; p < NP; ++p)
                offs[p] += static_cast<int64_t>(static_cast<int32_t>(i)) * pl.stride[p][d];
        }
    }
#pragma unroll
    for (int p = 0; p < NP; ++p)
        offs[p] += static_cast<int64_t>(static_cast<int32_t>(rem)) * pl.stride[p][0];
}

// ---------------------------------------------------------------------------------------------
// Compact index of the vector kernels: at most four dims after coalescing (anything deeper takes the
// element-wise kernels over the full plan) and 32-bit element offsets (split_pieces hands out
// pieces whose operands reach less than 2^31 elements from their first). Everything here lives in
// kernel arguments, so choices on it are scalar branches.
//   fast       all dims are powers of two, and dims and strides fit 24-bit multiplies: the
//              decomposition is shifts and masks plus full-rate 24-bit multiply-adds (a 32-bit
//              multiply runs at a quarter of the vector ALU rate, and a launch of these kernels is
//              one trip: every wavefront pays the index arithmetic before its first load)
//   lin_shift  operands that walk the logical space densely need no per-dim arithmetic: their
//              offset is the linear index << lin_shift[p] (lin_mask[p] all ones, strides zero; other
//              operands: mask and shift zero). When an item
//              stands for 2^lin_unroll_shift neighbouring positions of one dim (whose extent was
//              divided by that), the linear index of its first position is
//              ((idx - r) << lin_unroll_shift) + r with r = idx mod lin_inner, the items inside that dim.
constexpr int kIndexRank = 4;
template <int NP>
struct NdIndex4 {
    int32_t rank;
    uint32_t fast;
    uint32_t dim[kIndexRank], mul[kIndexRank], shr[kIndexRank];   // unused dims: 1, 0, 0; fast: shr = log2(dim)
    int32_t stride[NP][kIndexRank];                               // unused dims and linear operands: 0
    uint32_t lin_shift[NP], lin_mask[NP];                         // not linear: 0, 0; linear: shift, ~0
    uint32_t lin_unroll_shift;
    uint32_t lin_inner, lin_inner_mul, lin_inner_shr;
};

template <int NP>
__device__ __forceinline__ void nd4_offsets(const NdIndex4<NP> &ix, uint32_t idx, int32_t (&offs)[NP]) {
    uint32_t rem = idx;
    uint32_t lin_r;
    if (ix.fast) {
        // straight-line: unused dims have extent 1 and stride 0
        static_assert(kIndexRank == 4, "unrolled by hand");
        const int32_t i3 = static_cast<int32_t>(rem & (ix.dim[3] - 1));
        rem >>= ix.shr[3];
        const int32_t i2 = static_cast<int32_t>(rem & (ix.dim[2] - 1));
        rem >>= ix.shr[2];
        const int32_t i1 = static_cast<int32_t>(rem & (ix.dim[1] - 1));
        rem >>= ix.shr[1];
        const int32_t i0 = static_cast<int32_t>(rem);
#pragma unroll
        for (int p = 0; p < NP; ++p)
            offs[p] = (__mul24(i3, ix.stride[p][3]) + __mul24(i2, ix.stride[p][2])) +
                      (__mul24(i1, ix.stride[p][1]) + __mul24(i0, ix.stride[p][0]));
        lin_r = idx & (ix.lin_inner - 1);
    } else {
#pragma unroll
        for (int p = 0; p < NP; ++p) offs[p] = 0;
#pragma unroll
        for (int d = kIndexRank - 1; d >= 1; --d) {
            if (d < ix.rank) {
                const uint32_t q = ix.dim[d] == 1 ? rem : (__umulhi(rem, ix.mul[d]) >> ix.shr[d]);
                const int32_t i = static_cast<int32_t>(rem - q * ix.dim[d]);
                rem = q;
#pragma unroll
                for (int p = 0; p < NP; ++p)
                    if (ix.stride[p][d] != 0) offs[p] += i * ix.stride[p][d];
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
            if (ix.stride[p][0] != 0) offs[p] += static_cast<int32_t>(rem) * ix.stride[p][0];
        lin_r = 0;
        if (ix.lin_unroll_shift != 0) {
            const uint32_t q = ix.lin_inner == 1 ? idx : (__umulhi(idx, ix.lin_inner_mul) >> ix.lin_inner_shr);
            lin_r = idx - q * ix.lin_inner;
        }
    }
    const uint32_t lin = ((idx - lin_r) << ix.lin_unroll_shift) + lin_r;   // without unroll: idx
#pragma unroll
    for (int p = 0; p < NP; ++p) offs[p] += static_cast<int32_t>((lin << ix.lin_shift[p]) & ix.lin_mask[p]);
}

// Host: the compact index of a finished plan (after any division of its innermost dim by a vector
// width and of dim `unroll_dim` by 2^unroll_shift; -1: none). `inner_shift[p]` is log2 of operand
// p's element stride along the innermost dim as it stands (2 for four-element vectors, 0 for
// units). Returns false when the plan has more than four dims.
template <int NP>
inline bool make_index4(NdIndex4<NP> &ix, const NdPlan<NP> &pl, const int *inner_shift, int unroll_dim,
                        int unroll_shift) {
    if (pl.rank > kIndexRank) return false;
    ix.rank = pl.rank;
    const int last = pl.rank - 1;
    bool fast = true;
    for (int d = 0; d < kIndexRank; ++d) {
        const bool used = d < pl.rank;
        ix.dim[d] = used ? pl.dim[d] : 1;
        ix.mul[d] = used ? pl.fdiv[d].mul : 0;
        ix.shr[d] = used ? pl.fdiv[d].shr : 0;
        for (int p = 0; p < NP; ++p) ix.stride[p][d] = used ? pl.stride[p][d] : 0;
        if (!used) continue;
        if ((ix.dim[d] & (ix.dim[d] - 1)) != 0 || ix.dim[d] > (1u << 22)) fast = false;
        for (int p = 0; p < NP; ++p)
            if (pl.stride[p][d] >= (1 << 22) || pl.stride[p][d] <= -(1 << 22)) fast = false;
    }
    int64_t inner_items = 1;    // items inside the unroll dim
    for (int d = last; d > unroll_dim && unroll_dim >= 0; --d) inner_items *= pl.dim64[d];
    if (inner_items & (inner_items - 1)) fast = false;
    for (int p = 0; p < NP; ++p) {
        int64_t expect = static_cast<int64_t>(1) << inner_shift[p];
        bool dense = true;
        for (int d = last; d >= 0 && dense; --d) {
            const int64_t want = (d == unroll_dim) ? (expect << unroll_shift) : expect;
            if (pl.dim64[d] > 1 && pl.stride[p][d] != want) dense = false;
            expect = want * pl.dim64[d];
        }
        ix.lin_shift[p] = dense ? static_cast<uint32_t>(inner_shift[p]) : 0u;
        ix.lin_mask[p] = dense ? ~0u : 0u;
        if (dense)
            for (int d = 0; d < kIndexRank; ++d) ix.stride[p][d] = 0;
    }
    ix.lin_unroll_shift = unroll_dim >= 0 ? static_cast<uint32_t>(unroll_shift) : 0;
    const FastDiv inner(static_cast<uint32_t>(inner_items));
    ix.lin_inner = inner.d;
    ix.lin_inner_mul = inner.mul;
    ix.lin_inner_shr = inner.shr;
    if (fast)
        for (int d = 0; d < kIndexRank; ++d) {
            uint32_t lg = 0;
            while ((1u << lg) < ix.dim[d]) ++lg;
            ix.shr[d] = lg;
        }
    ix.fast = fast ? 1u : 0u;
    return true;
}

}  // namespace rmlk
