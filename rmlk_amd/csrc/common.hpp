// Shared host/device helpers for the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "../../include/rmlk_hip.h"

namespace rmlk {

constexpr int kMaxRank = RMLK_MAX_RANK;
constexpr int kWave = 64;         // CDNA wavefront width
constexpr int kNumCU = 256;       // MI355X compute units (8 XCDs x 32)
constexpr int64_t kMaxElems = (int64_t)1 << 62;

// Streams on which small launches are being collected (batch.hip), and the call that sends the
// collected ones of a stream out. Every entry point turns its stream handle into a hipStream_t
// through as_stream before it issues anything, so whatever was collected is in the stream first.
extern std::atomic<int> g_open_batches;
int32_t batch_flush_stream(hipStream_t s);
inline hipStream_t as_stream(rmlk_stream_t s) {
    hipStream_t h = reinterpret_cast<hipStream_t>(s);
    if (g_open_batches.load(std::memory_order_relaxed) > 0) (void)batch_flush_stream(h);
    return h;
}
// (for the entry points that may hand their work to the batch instead)
inline hipStream_t as_stream_collecting(rmlk_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Status of the launch just issued (hipError_t as a positive int, 0 when fine).
inline int32_t launch_status() { return static_cast<int32_t>(hipGetLastError()); }

inline int dtype_size(int32_t dt) {
    switch (dt) {
        case RMLK_BOOL:
        case RMLK_UINT8:
        case RMLK_INT8: return 1;
        case RMLK_UINT16:
        case RMLK_INT16:
        case RMLK_FLOAT16:
        case RMLK_BFLOAT16: return 2;
        case RMLK_FLOAT:
        case RMLK_INT32:
        case RMLK_UINT32: return 4;
        case RMLK_DOUBLE:
        case RMLK_INT64:
        case RMLK_UINT64: return 8;
        default: return 0;
    }
}

inline bool dims_ok(const rmlk_dims *d) { return d && d->rank >= 1 && d->rank <= kMaxRank; }

// Product of dims, -1 when a dim is negative or the product overflows kMaxElems.
inline int64_t dims_numel(const rmlk_dims *d) {
    int64_t n = 1;
    for (int i = 0; i < d->rank; ++i) {
        if (d->v[i] < 0) return -1;
        if (d->v[i] == 0) return 0;
    }
    for (int i = 0; i < d->rank; ++i) {
        if (n > kMaxElems / d->v[i]) return -1;
        n *= d->v[i];
    }
    return n;
}

// Unsigned division by a runtime constant through one mul-high and a shift.
// Exact for dividends below 2^31 (the kernels use it only on 32-bit index paths).
struct FastDiv {
    uint32_t d, mul, shr;
    FastDiv() : d(1), mul(0), shr(0) {}
    explicit FastDiv(uint32_t div) : d(div), mul(0), shr(0) {
        if (div > 1) {
            uint32_t lg = 0;
            while ((1ull << lg) < div) ++lg;
            uint32_t p = 31 + lg;
            mul = static_cast<uint32_t>(((1ull << p) + div - 1) / div);
            shr = p - 32;
        }
    }
    __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        return d == 1 ? n : (__umulhi(n, mul) >> shr);
#else
        return d == 1 ? n : static_cast<uint32_t>((static_cast<uint64_t>(n) * mul) >> 32) >> shr;
#endif
    }
};

// ---------------------------------------------------------------------------------------------
// N-d iteration plan: one logical shape, element strides for up to NP operands (inputs and the
// output alike). The host removes size-1 dims and merges dims that are jointly contiguous in every
// operand, so dense same-shape work collapses to rank 1 and `[8,32,512,64] (.) [1,32,1,64]` keeps
// four dims with a contiguous innermost run.
template <int NP>
struct NdPlan {
    int32_t rank;                    // >= 1 after coalescing
    uint32_t dim[kMaxRank];          // dim[rank-1] is innermost
    int64_t dim64[kMaxRank];
    FastDiv fdiv[kMaxRank];
    int32_t stride[NP][kMaxRank];    // element strides, may be 0 or negative; |stride| < 2^31
    int64_t numel;
};

constexpr int64_t kPieceElems = (int64_t)1 << 30;   // elements one launch indexes (32-bit math)
constexpr int64_t kStrideLimit = (int64_t)1 << 31;  // strides a plan can hold

// Build a coalesced plan. shape[rank], strides[p][rank]. Returns false when numel == 0.
template <int NP>
inline bool build_plan(NdPlan<NP> &pl, int rank, const int64_t *shape,
                       const int64_t (*strides)[kMaxRank]) {
    int64_t shp[kMaxRank];
    int64_t st[NP][kMaxRank];
    int r = 0;
    int64_t numel = 1;
    for (int d = 0; d < rank; ++d) numel *= shape[d];
    pl.numel = numel;
    if (numel == 0) return false;
    for (int d = 0; d < rank; ++d) {
        if (shape[d] == 1) continue;
        shp[r] = shape[d];
        for (int p = 0; p < NP; ++p) st[p][r] = strides[p][d];
        ++r;
    }
    if (r == 0) {
        r = 1;
        shp[0] = 1;
        for (int p = 0; p < NP; ++p) st[p][0] = 1;
    }
    // merge dim d into d+1 when every operand walks them as one run
    int w = 0;  // write index of the current (outer-most so far) merged dim
    int64_t mshp[kMaxRank];
    int64_t mst[NP][kMaxRank];
    mshp[0] = shp[0];
    for (int p = 0; p < NP; ++p) mst[p][0] = st[p][0];
    for (int d = 1; d < r; ++d) {
        bool can = true;
        for (int p = 0; p < NP; ++p)
            if (mst[p][w] != st[p][d] * shp[d]) { can = false; break; }
        if (can) {
            mshp[w] *= shp[d];
            for (int p = 0; p < NP; ++p) mst[p][w] = st[p][d];
        } else {
            ++w;
            mshp[w] = shp[d];
            for (int p = 0; p < NP; ++p) mst[p][w] = st[p][d];
        }
    }
    pl.rank = w + 1;
    for (int d = 0; d < pl.rank; ++d) {
        pl.dim64[d] = mshp[d];
        pl.dim[d] = static_cast<uint32_t>(mshp[d]);
        pl.fdiv[d] = FastDiv(static_cast<uint32_t>(mshp[d] > 0x7fffffff ? 1 : mshp[d]));
        for (int p = 0; p < NP; ++p) pl.stride[p][d] = static_cast<int32_t>(mst[p][d]);
    }
    for (int d = pl.rank; d < kMaxRank; ++d) {
        pl.dim64[d] = 1;
        pl.dim[d] = 1;
        pl.fdiv[d] = FastDiv(1);
        for (int p = 0; p < NP; ++p) pl.stride[p][d] = 0;
    }
    return true;
}

inline void dense_strides(int rank, const int64_t *shape, int64_t *stride) {
    int64_t s = 1;
    for (int d = rank - 1; d >= 0; --d) {
        stride[d] = s;
        s *= shape[d];
    }
}

// Kernels index with 32-bit math: at most kPieceElems elements per launch and strides below
// kStrideLimit. Larger work is cut along its outermost non-unit dim, recursively.
// fn(shape, offsets) launches one piece; offsets[p] is the element offset of operand p.
template <int NP, typename Fn>
inline int32_t split_pieces(int rank, const int64_t *shape, const int64_t (*strides)[kMaxRank],
                            const int64_t *offsets, Fn &&fn) {
    int64_t numel = 1;
    for (int d = 0; d < rank; ++d) {
        if (shape[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (shape[d] == 0) return RMLK_OK;
    }
    for (int d = 0; d < rank; ++d) {
        if (numel > kMaxElems / shape[d]) return RMLK_ERR_TOO_LARGE;
        numel *= shape[d];
    }
    bool strides_fit = true;
    for (int d = 0; d < rank; ++d)
        if (shape[d] > 1)
            for (int p = 0; p < NP; ++p)
                if (strides[p][d] >= kStrideLimit || strides[p][d] <= -kStrideLimit)
                    strides_fit = false;
    // the kernels may accumulate element offsets in 32 bits: the farthest element of every operand
    // must lie within 2^31 elements of its first
    bool extents_fit = true;
    for (int p = 0; p < NP; ++p) {
        int64_t reach_up = 0, reach_down = 0;
        for (int d = 0; d < rank; ++d) {
            if (shape[d] <= 1 || strides[p][d] == 0 || !strides_fit) continue;
            const int64_t span = (shape[d] - 1) * strides[p][d];
            if (span > 0) reach_up += span; else reach_down -= span;
        }
        if (reach_up >= kStrideLimit || reach_down >= kStrideLimit) extents_fit = false;
    }
    if (numel <= kPieceElems && strides_fit && extents_fit) return fn(shape, offsets);
    int d0 = 0;
    while (d0 < rank - 1 && shape[d0] == 1) ++d0;
    if (shape[d0] == 1) return RMLK_ERR_TOO_LARGE;  // a single element cannot be too large
    const int64_t inner = numel / shape[d0];
    int64_t rows_per = inner >= kPieceElems ? 1 : kPieceElems / inner;
    if (rows_per >= shape[d0]) rows_per = (shape[d0] + 1) / 2;   // cut for the extents alone
    for (int p = 0; p < NP; ++p)
        if (strides[p][d0] >= kStrideLimit || strides[p][d0] <= -kStrideLimit) rows_per = 1;
    int64_t sub[kMaxRank];
    for (int d = 0; d < rank; ++d) sub[d] = shape[d];
    for (int64_t r0 = 0; r0 < shape[d0]; r0 += rows_per) {
        sub[d0] = shape[d0] - r0 < rows_per ? shape[d0] - r0 : rows_per;
        int64_t offs[NP];
        for (int p = 0; p < NP; ++p) offs[p] = offsets[p] + r0 * strides[p][d0];
        int32_t st = split_pieces<NP>(rank, sub, strides, offs, fn);
        if (st != RMLK_OK) return st;
    }
    return RMLK_OK;
}

// A kernel that needs more than 64 KiB of dynamic LDS must be told so once per device. One object
// per kernel (a function-local static of its launcher).
struct DynamicLdsGrant {
    static constexpr int kMaxDevices = 64;
    bool raised[kMaxDevices] = {};   // benign race: every thread writes the same value

    template <typename Kern>
    int32_t ensure(Kern kern, int bytes) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return static_cast<int32_t>(e);
        if (dev < 0 || dev >= kMaxDevices || !raised[dev]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
            if (e != hipSuccess) return static_cast<int32_t>(e);
            if (dev >= 0 && dev < kMaxDevices) raised[dev] = true;
        }
        return RMLK_OK;
    }
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant
// expression inside the body.
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Streaming (non-temporal) load of a vector of 4, 8 or n * 16 bytes, for data a kernel reads once.
// It pays where measured (dense float operands of the element-wise kernels, the rows of Softmax)
// and costs elsewhere (SwiGLU -8 %, Trilu -4 %, copies and 8-byte elements), so it is not a default.
typedef uint32_t ew_u32x4 __attribute__((ext_vector_type(4)));
template <typename V>
__device__ __forceinline__ V nt_load(const V *p) {
    V out;
    if constexpr (sizeof(V) % 16 == 0) {
#pragma unroll
        for (size_t i = 0; i < sizeof(V) / 16; ++i)
            reinterpret_cast<ew_u32x4 *>(&out)[i] =
                __builtin_nontemporal_load(reinterpret_cast<const ew_u32x4 *>(p) + i);
    } else if constexpr (sizeof(V) == 8) {
        *reinterpret_cast<uint64_t *>(&out) = __builtin_nontemporal_load(reinterpret_cast<const uint64_t *>(p));
    } else if constexpr (sizeof(V) == 4) {
        *reinterpret_cast<uint32_t *>(&out) = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p));
    } else {
        out = *p;
    }
    return out;
}
// Streaming (non-temporal) store, the counterpart of nt_load: a large result leaves the chip as it
// is produced instead of sitting in the L2s until the write-back at the end of the kernel
// (a 16 MiB + 16 MiB copy: 7.7 -> 6.7 us; 256 MiB + 256 MiB: 95 -> 90 us).
template <typename V>
__device__ __forceinline__ void nt_store(V *p, const V &v) {
    if constexpr (sizeof(V) % 16 == 0) {
#pragma unroll
        for (size_t i = 0; i < sizeof(V) / 16; ++i)
            __builtin_nontemporal_store(reinterpret_cast<const ew_u32x4 *>(&v)[i],
                                        reinterpret_cast<ew_u32x4 *>(p) + i);
    } else if constexpr (sizeof(V) == 8) {
        __builtin_nontemporal_store(*reinterpret_cast<const uint64_t *>(&v), reinterpret_cast<uint64_t *>(p));
    } else if constexpr (sizeof(V) == 4) {
        __builtin_nontemporal_store(*reinterpret_cast<const uint32_t *>(&v), reinterpret_cast<uint32_t *>(p));
    } else {
        *p = v;
    }
}

// Streaming kernels walk their index space in chunks of block x unroll consecutive items: a block
// takes a chunk, lane t of it the items t, t + block, t + 2 block, ..., so that the accesses a block
// has in flight cover one contiguous 16 KiB piece of every dense operand (accesses a whole grid
// apart, the usual grid-stride unrolling, reached 4.3 TB/s on a 256 MiB copy where this reaches 6.0).
// Grid for `items` items in chunks of `chunk`: one trip up to 32 blocks per compute unit.
inline unsigned chunk_grid(int64_t items, int chunk) {
    int64_t need = (items + chunk - 1) / chunk;
    const int64_t cap = static_cast<int64_t>(256) * 32;
    if (need < 1) need = 1;
    return static_cast<unsigned>(need < cap ? need : cap);
}

// Wavefront reductions through DPP (data-parallel primitives: an operand read from another lane of
// the same row of 16 inside the instruction itself) instead of ds_bpermute shuffles, each of which
// is a round trip through the LDS crossbar: quad swaps, then the two mirrors give every lane of a
// row the row's result; the four row results meet through readlane. The order of the additions is
// fixed, and the same in every kernel that uses these.
template <int CTRL, typename T>
__device__ __forceinline__ T dpp_take(T v) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit values");
    if constexpr (sizeof(T) == 4) {
        const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
        return __builtin_bit_cast(T, r);
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(u), CTRL, 0xf, 0xf, false));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(u >> 32), CTRL, 0xf, 0xf, false));
        return __builtin_bit_cast(T, (static_cast<uint64_t>(hi) << 32) | lo);
    }
}
template <typename T>
__device__ __forceinline__ T lane_value(T v, int lane) {
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
    } else {
        const uint64_t u = __builtin_bit_cast(uint64_t, v);
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(u), lane));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(u >> 32), lane));
        return __builtin_bit_cast(T, (static_cast<uint64_t>(hi) << 32) | lo);
    }
}
constexpr int kDppQuadSwap1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
    v += dpp_take<kDppQuadSwap1>(v);
    v += dpp_take<kDppQuadSwap2>(v);
    v += dpp_take<kDppRowHalfMirror>(v);
    v += dpp_take<kDppRowMirror>(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
template <typename T>
__device__ __forceinline__ T wave_max(T v) {
    T w = dpp_take<kDppQuadSwap1>(v);
    v = w > v ? w : v;
    w = dpp_take<kDppQuadSwap2>(v);
    v = w > v ? w : v;
    w = dpp_take<kDppRowHalfMirror>(v);
    v = w > v ? w : v;
    w = dpp_take<kDppRowMirror>(v);
    v = w > v ? w : v;
    const T a = lane_value(v, 0), b = lane_value(v, 16), c = lane_value(v, 32), d = lane_value(v, 48);
    const T ab = b > a ? b : a, cd = d > c ? d : c;
    return cd > ab ? cd : ab;
}

// Grid size for a grid-stride kernel: enough blocks to cover `work` items, capped so that a few
// waves per SIMD stay resident on all 256 CUs.
inline unsigned grid_for(int64_t work, int block, int max_blocks_per_cu = 8) {
    int64_t need = (work + block - 1) / block;
    int64_t cap = static_cast<int64_t>(kNumCU) * max_blocks_per_cu;
    if (need < 1) need = 1;
    return static_cast<unsigned>(need < cap ? need : cap);
}

// N elements moved as one access; alignment is capped at the widest (128-bit) memory operation.
template <typename T, int N>
struct alignas(sizeof(T) * N > 16 ? 16 : sizeof(T) * N) Vec {
    T v[N];
};

}  // namespace rmlk
