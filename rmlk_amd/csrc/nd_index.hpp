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

}  // namespace rmlk
