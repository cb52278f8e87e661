// Batched fp32 MatMul for gfx950: MFMA tiles staged through LDS for M > 1, an HBM-streaming GEMV
// for the M == 1 decode shape. Replaces the cublasGemmStridedBatchedEx call of the reference
// (cuda/src/kernels/gemm.rs:191-232) and the operand copies its MatMul backend makes to
// broadcast a 2-D operand over the batch (runtime/src/providers/cuda/backend/matmul.rs:48-86):
// a batch stride of 0 broadcasts in place.
//
// MFMA kernel (row-major, A[M,K] . B[K,N]):
//   - a 256-lane block (4 wavefronts) owns a BM x BN tile of C and walks K in steps of BK;
//   - global -> registers -> LDS with the next K-step's global loads in flight while the current
//     one is multiplied (two LDS buffers, one barrier per step);
//   - each wavefront owns a WM x WN sub-tile as (WM/32) x (WN/32) v_mfma_f32_32x32x2_f32
//     accumulators. MFMA's 2-deep K is fed with a K-permutation inside every 8-wide K chunk: lanes
//     0-31 take k = 0..3 and lanes 32-63 take k = 4..7 of the chunk, for A and B alike, so one
//     128-bit LDS read of A serves four MFMAs and the sum over K is unchanged;
//   - problems made of whole tiles with K steps of 32 take the variant whose K-step tiles go from
//     global memory straight into LDS (global_load_lds_dwordx4), see gemm_mfma_direct_kernel;
//   - split-K (grid z) writes partial tiles to the workspace, a second kernel adds them in a
//     fixed order, so results do not depend on scheduling.
//   - a K-contiguous B of constant weights may be STORED as IEEE half or bfloat16 values (StoredF16,
//     StoredBF16): they are widened exactly and everything is computed in fp32 as before, from half
//     the bytes. The tiled kernels widen on the way into LDS (same MFMAs, same bits as over the
//     widened weights), the one-row kernels in registers.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <type_traits>

#include "common.hpp"

// This file is compiled twice, so that the two halves of its many tiled-GEMM instantiations build
// side by side: as it stands (everything but the tiled products over 16-bit weights), and included
// by matmul_stored16.hip with RMLK_MATMUL_PART 2 (only those, behind the two functions below).
#ifndef RMLK_MATMUL_PART
#define RMLK_MATMUL_PART 1
#endif

namespace rmlk {
// the tiled products over weights stored as 16-bit values (`seg`: a Segments of this file, or null)
int32_t stored16_gemm_tiled(hipStream_t s, int64_t batch, int64_t m, int64_t n, int64_t k, const float *pa,
                            int64_t lda, int64_t stride_a, int32_t b_dtype, const void *pb, int64_t ldb,
                            int64_t stride_b, int32_t trans_b, float *pc, int64_t ldc, int64_t stride_c,
                            void *workspace, size_t workspace_bytes, const void *seg, int32_t *partial_splits);
int32_t stored16_gemm_swiglu(hipStream_t s, int64_t m, int64_t n, int64_t k, const float *pa, int64_t lda,
                             int32_t b_dtype, const void *pb, int64_t ldb, int32_t trans_b, int64_t gate_offset,
                             int64_t up_offset, float *pc, int64_t ldc);

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// How the second operand of a product over constant weights is held in memory: as floats, or as
// IEEE half or bfloat16 values (half the bytes to stream). The arithmetic is fp32 whatever the
// storage: both 16-bit formats are subsets of float, a stored value is widened exactly before it
// is multiplied, and every sum is formed in float - the result is that of the fp32 product over the
// weights rounded once, when they were stored.
struct StoredF32 {
    using elem = float;
    static constexpr int kUnit = 4;      // weights per 128-bit unit
};
struct StoredF16 {
    using elem = uint16_t;
    static constexpr int kUnit = 8;
    static __device__ __forceinline__ float widen(uint16_t v) {
        return static_cast<float>(__builtin_bit_cast(_Float16, v));
    }
    // two neighbours of a row, the one at the lower address in the low half
    static __device__ __forceinline__ void widen2(uint32_t pair, float &lo, float &hi) {
        const v2h h = __builtin_bit_cast(v2h, pair);
        lo = static_cast<float>(h[0]);
        hi = static_cast<float>(h[1]);
    }
};
struct StoredBF16 {
    using elem = uint16_t;
    static constexpr int kUnit = 8;
    static __device__ __forceinline__ float widen(uint16_t v) {
        return __uint_as_float(static_cast<uint32_t>(v) << 16);
    }
    static __device__ __forceinline__ void widen2(uint32_t pair, float &lo, float &hi) {
        lo = __uint_as_float(pair << 16);
        hi = __uint_as_float(pair & 0xffff0000u);
    }
};
template <typename WS>
constexpr bool kStored16 = !std::is_same<WS, StoredF32>::value;

// The eight weights of one 128-bit unit of a 16-bit row, in row order.
template <typename WS>
__device__ __forceinline__ void widen_unit(const v4u &raw, float (&w)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) WS::widen2(raw[i], w[2 * i], w[2 * i + 1]);
}

// f(storage tag) for the storage type `w_dtype` names; UNSUPPORTED for any other type.
template <typename F>
int32_t with_storage(int32_t w_dtype, F &&f) {
    switch (w_dtype) {
        case RMLK_FLOAT: return f(StoredF32{});
        case RMLK_FLOAT16: return f(StoredF16{});
        case RMLK_BFLOAT16: return f(StoredBF16{});
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

// The same for the tiled MFMA kernels: each compilation of this file instantiates its share.
template <typename F>
int32_t with_storage_tiled(int32_t w_dtype, F &&f) {
    switch (w_dtype) {
#if RMLK_MATMUL_PART == 1
        case RMLK_FLOAT: return f(StoredF32{});
#else
        case RMLK_FLOAT16: return f(StoredF16{});
        case RMLK_BFLOAT16: return f(StoredBF16{});
#endif
        default: return RMLK_ERR_UNSUPPORTED;
    }
}

constexpr int kMaxSegments = 4;

struct GemmArgs {
    const float *a;
    const float *b;
    float *c;
    int32_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;  // batch strides (elements)
    int32_t k_per_split;                   // K range of one z-slice (multiple of BK)
    int32_t tiles_m, tiles_n;
    int32_t aligned;                       // rows of A and B start on 16-byte boundaries
    // Column blocks of C with a destination each (grouped products): block i covers columns
    // [seg_begin[i], seg_begin[i + 1]) and is written to seg_c[i] with leading dimension seg_ldc[i].
    // n_seg == 0: plain C. Block boundaries are multiples of 32 (one MFMA result block).
    int32_t n_seg;
    int32_t seg_begin[kMaxSegments + 1];
    float *seg_c[kMaxSegments];
    int64_t seg_ldc[kMaxSegments];
    // SwiGLU epilogue: columns of the gate and of the up projection inside B
    int32_t gate_offset, up_offset;
};

constexpr int kThreads = 256;
constexpr int kSkinnyRows = 8;  // up to this many rows of A take the B-streaming kernels
constexpr int kPadA = 4;  // floats of padding per LDS row of A
constexpr int kPadB = 8;  // floats of padding per LDS row of B

// TB: B is stored [N][K] (K contiguous) and staged in LDS exactly like A, [BN][BK + pad].
template <int BM, int BN, int BK, bool TB = false>
struct SmemLayout {
    static constexpr int kAStride = BK + kPadA;
    static constexpr int kBStride = TB ? BK + kPadA : BN + kPadB;
    static constexpr int kAFloats = BM * kAStride;
    static constexpr int kBFloats = TB ? BN * kBStride : BK * kBStride;
    static constexpr int kBytes = 2 * (kAFloats + kBFloats) * 4;
};

// tile index -> (tile_m, tile_n). Consecutive hardware block ids go round-robin over the 8 XCDs,
// each with a private L2; blocks are renumbered so that one XCD works on a compact group of
// tiles that share rows of A and columns of B.
__device__ __forceinline__ void tile_coords(const GemmArgs &g, int &tm, int &tn, int &split) {
    const int n_tiles = g.tiles_m * g.tiles_n;
    int pid = blockIdx.x;
    split = blockIdx.z;
    constexpr int kXcd = 8;
    if (gridDim.y == 1 && gridDim.z > 1 && (n_tiles * gridDim.z) % kXcd == 0) {
        // split-K of one matrix: the (split, tile) pairs are dealt to the XCDs in contiguous runs,
        // split-major, so that an XCD works on ONE K slab where it can and fetches that slab of A
        // once instead of every slab of A
        const int linear = blockIdx.x + n_tiles * blockIdx.z;   // hardware order: x fastest
        const int per = n_tiles * gridDim.z / kXcd;
        const int item = (linear % kXcd) * per + linear / kXcd;
        split = item / n_tiles;
        pid = item - split * n_tiles;
    } else if (n_tiles % kXcd == 0) {
        const int per = n_tiles / kXcd;
        pid = (pid % kXcd) * per + pid / kXcd;
    }
    // groups of kGroupM tile-rows swept column by column
    constexpr int kGroupM = 4;
    const int width = kGroupM * g.tiles_n;
    const int group = pid / width;
    const int first_m = group * kGroupM;
    const int gsz = g.tiles_m - first_m < kGroupM ? g.tiles_m - first_m : kGroupM;
    const int in_group = pid - group * width;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// EDGE == false: every tile is full (m % BM == 0, n % BN == 0, the K range of a split is a
// multiple of BK) and rows are 16-byte aligned, so the main loop has no bounds checks at all.
// EDGE == true: guarded loads (zero fill) and guarded stores; `aligned` still allows 128-bit
// loads where a whole vector is in range.
// TB == true: B is given as [N][K] rows (C = A . B^T); both operands are then K-contiguous and the
// B fragment is one 128-bit LDS read like A's.
// WS: B (K-contiguous only) may be stored as 16-bit values; they are widened on their way from
// global memory to LDS, which holds floats either way.
template <int BM, int BN, int BK, int WM, int WN, bool EDGE, bool TB = false, typename WS = StoredF32>
__global__ __launch_bounds__(kThreads) void gemm_mfma_kernel(GemmArgs g) {
    using L = SmemLayout<BM, BN, BK, TB>;
    using BE = typename WS::elem;
    static_assert(!kStored16<WS> || TB, "16-bit weights are K-contiguous");
    // four consecutive values of a row of B as floats
    auto load_b4 = [](const BE *src) -> v4f {
        if constexpr (kStored16<WS>) {
            const v2u raw = *reinterpret_cast<const v2u *>(src);
            v4f v;
            float lo, hi;
            WS::widen2(raw[0], lo, hi);
            v[0] = lo;
            v[1] = hi;
            WS::widen2(raw[1], lo, hi);
            v[2] = lo;
            v[3] = hi;
            return v;
        } else {
            return *reinterpret_cast<const v4f *>(src);
        }
    };
    auto load_b1 = [](const BE *src) -> float {
        if constexpr (kStored16<WS>) return WS::widen(*src);
        else return *src;
    };
    extern __shared__ __align__(16) float smem[];
    float *As = smem;                     // [2][BM][kAStride]
    float *Bs = smem + 2 * L::kAFloats;   // [2][BK][kBStride]

    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == kThreads / kWave, "four wavefronts per block");
    static_assert(BK % 8 == 0, "K chunks of 8");

    // global -> LDS staging shapes: float4 per lane
    constexpr int A_VECS_PER_ROW = BK / 4;
    constexpr int A_ROWS_PER_PASS = kThreads / A_VECS_PER_ROW;
    constexpr int A_PASSES = BM / A_ROWS_PER_PASS;
    constexpr int B_VECS_PER_ROW = (TB ? BK : BN) / 4;
    constexpr int B_ROWS_PER_PASS = kThreads / B_VECS_PER_ROW;
    constexpr int B_PASSES = (TB ? BN : BK) / B_ROWS_PER_PASS;
    static_assert(A_PASSES >= 1 && B_PASSES >= 1, "tile too small for 256 lanes");

    int tile_m, tile_n, split;
    tile_coords(g, tile_m, tile_n, split);
    const int batch = blockIdx.y;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int k_begin = split * g.k_per_split;
    const int k_end = min(g.k, k_begin + g.k_per_split);

    const float *A = g.a + batch * g.stride_a;
    const BE *B = reinterpret_cast<const BE *>(g.b) + batch * g.stride_b;
    float *C = g.c + (static_cast<int64_t>(split) * gridDim.y + batch) * g.stride_c;

    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane % 32, half = lane / 32;

    const int a_vec = tid % A_VECS_PER_ROW, a_row = tid / A_VECS_PER_ROW;
    const int b_vec = tid % B_VECS_PER_ROW, b_row = tid / B_VECS_PER_ROW;

    v4f a_reg[A_PASSES], b_reg[B_PASSES];

    // per-lane source pointers of the first K step; they advance by BK (A) and BK rows (B)
    const float *a_src = A + static_cast<int64_t>(m0 + a_row) * g.lda + k_begin + a_vec * 4;
    const BE *b_src = TB ? B + static_cast<int64_t>(n0 + b_row) * g.ldb + k_begin + b_vec * 4
                         : B + static_cast<int64_t>(k_begin + b_row) * g.ldb + n0 + b_vec * 4;
    const int64_t a_pass_stride = static_cast<int64_t>(A_ROWS_PER_PASS) * g.lda;
    const int64_t b_pass_stride = static_cast<int64_t>(B_ROWS_PER_PASS) * g.ldb;
    const int64_t b_step_stride = TB ? BK : static_cast<int64_t>(BK) * g.ldb;
    const bool vec_ok = g.aligned != 0;

    auto load_global = [&](int k0) {
        if constexpr (!EDGE) {
#pragma unroll
            for (int p = 0; p < A_PASSES; ++p)
                a_reg[p] = *reinterpret_cast<const v4f *>(a_src + p * a_pass_stride);
#pragma unroll
            for (int p = 0; p < B_PASSES; ++p) b_reg[p] = load_b4(b_src + p * b_pass_stride);
        } else {
#pragma unroll
            for (int p = 0; p < A_PASSES; ++p) {
                const int r = m0 + a_row + p * A_ROWS_PER_PASS;
                const int kk = k0 + a_vec * 4;
                v4f v = {0.f, 0.f, 0.f, 0.f};
                if (r < g.m) {
                    const float *src = a_src + p * a_pass_stride;
                    if (vec_ok && kk + 3 < k_end) {
                        v = *reinterpret_cast<const v4f *>(src);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (kk + j < k_end) v[j] = src[j];
                    }
                }
                a_reg[p] = v;
            }
#pragma unroll
            for (int p = 0; p < B_PASSES; ++p) {
                if constexpr (TB) {
                    const int r = n0 + b_row + p * B_ROWS_PER_PASS;
                    const int kk = k0 + b_vec * 4;
                    v4f v = {0.f, 0.f, 0.f, 0.f};
                    if (r < g.n) {
                        const BE *src = b_src + p * b_pass_stride;
                        if (vec_ok && kk + 3 < k_end) {
                            v = load_b4(src);
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                if (kk + j < k_end) v[j] = load_b1(src + j);
                        }
                    }
                    b_reg[p] = v;
                    continue;
                }
                const int kk = k0 + b_row + p * B_ROWS_PER_PASS;
                const int c = n0 + b_vec * 4;
                v4f v = {0.f, 0.f, 0.f, 0.f};
                if (kk < k_end) {
                    const BE *src = b_src + p * b_pass_stride;
                    if (vec_ok && c + 3 < g.n) {
                        v = load_b4(src);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (c + j < g.n) v[j] = load_b1(src + j);
                    }
                }
                b_reg[p] = v;
            }
        }
        a_src += BK;
        b_src += b_step_stride;
    };
    auto store_lds = [&](int buf) {
        float *as = As + buf * L::kAFloats;
        float *bs = Bs + buf * L::kBFloats;
#pragma unroll
        for (int p = 0; p < A_PASSES; ++p)
            *reinterpret_cast<v4f *>(as + (a_row + p * A_ROWS_PER_PASS) * L::kAStride +
                                     a_vec * 4) = a_reg[p];
#pragma unroll
        for (int p = 0; p < B_PASSES; ++p)
            *reinterpret_cast<v4f *>(bs + (b_row + p * B_ROWS_PER_PASS) * L::kBStride +
                                     b_vec * 4) = b_reg[p];
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int n_steps = (k_end - k_begin + BK - 1) / BK;
    const int a_frag = (wm * WM + l32) * L::kAStride + half * 4;
    const int b_frag = TB ? (wn * WN + l32) * L::kBStride + half * 4
                          : (half * 4) * L::kBStride + wn * WN + l32;
    constexpr int KC = BK / 8;
    static_assert(KC % 2 == 0, "fragment double buffering assumes an even number of K chunks");

    // MFMA operands of one 8-wide K chunk, read from LDS buffer `buf`
    v4f af[2][TM];
    float bf[2][TN][4];
    auto read_frags = [&](int buf, int kc, int slot) {
        const float *as = As + buf * L::kAFloats + a_frag;
        const float *bs = Bs + buf * L::kBFloats + b_frag;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            af[slot][i] = *reinterpret_cast<const v4f *>(as + i * 32 * L::kAStride + kc * 8);
        if constexpr (TB) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4f bv = *reinterpret_cast<const v4f *>(bs + j * 32 * L::kBStride + kc * 8);
#pragma unroll
                for (int s = 0; s < 4; ++s) bf[slot][j][s] = bv[s];
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    bf[slot][j][s] = bs[(kc * 8 + s) * L::kBStride + j * 32];
        }
    };
    // LDS traffic of this wavefront has drained, then the block meets. (Global loads of a later
    // K step stay in flight across the barrier.)
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // Software pipeline over K steps s = 0 .. n_steps-1, LDS buffer s & 1. Program order inside a
    // step (the scheduler is told not to move work across the marked points):
    //   chunk 0         : after its first MFMAs, the tile of step s+1 (in registers since step s-1)
    //                     goes to the other LDS buffer and the global loads of step s+2 are issued;
    //   chunk kc        : request the operands of chunk kc+1 from LDS, then issue chunk kc's MFMAs
    //                     (they run while the requests complete);
    //   last chunk      : this wavefront's reads of the buffer are complete, the block meets
    //                     (everyone's stores of step s+1 are long done), the first operands of
    //                     step s+1 are requested, and the last chunk's MFMAs cover that latency.
    if (n_steps > 0) {
        load_global(k_begin);
        store_lds(0);
        if (n_steps > 1) load_global(k_begin + BK);
        lds_barrier();
        read_frags(0, 0, 0);
    }
    auto mfma_chunk = [&](int slot, int s_begin, int s_end) {
#pragma unroll
        for (int s = s_begin; s < s_end; ++s)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[slot][i][s], bf[slot][j][s],
                                                                     acc[i][j], 0, 0, 0);
    };
    for (int step = 0; step < n_steps; ++step) {
        const int buf = step & 1;
        const bool more = step + 1 < n_steps;
        // chunk 0: its first MFMAs go out before anything else (their operands were requested a
        // whole chunk ago), the LDS stores and global loads issue in their shadow
        mfma_chunk(0, 0, 1);
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
            store_lds(buf ^ 1);
            if (step + 2 < n_steps) load_global(k_begin + (step + 2) * BK);
        }
        read_frags(buf, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_chunk(0, 1, 4);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kc = 1; kc < KC; ++kc) {
            const int slot = kc & 1;
            if (kc + 1 < KC) {
                read_frags(buf, kc + 1, slot ^ 1);
            } else {
                lds_barrier();
                if (more) read_frags(buf ^ 1, 0, slot ^ 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            mfma_chunk(slot, 0, 4);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // C fragment: column = l32, row = 8 * (r / 4) + 4 * half + r % 4
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + wn * WN + j * 32 + l32;
            if (!EDGE || col < g.n) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (!EDGE || row < g.m)
                        C[static_cast<int64_t>(row) * g.ldc + col] = acc[i][j][r];
                }
            }
        }
    }
}

// ---- kernel with direct global -> LDS loads -------------------------------------------------------
// For problems with whole K steps (BK = 32) and 16-byte aligned rows the K-step tiles do not pass
// through registers: each wavefront issues `global_load_lds_dwordx4`, which
// writes 64 lanes x 16 bytes as one contiguous 1 KiB piece of LDS while every lane picks its own
// global address. Rows of 32 floats are therefore unpadded in LDS; bank conflicts on the
// fragment reads of K-contiguous operands are avoided by a swizzle instead: the 16-byte unit q of
// row r lives in unit q ^ ((r >> 1) & 7), applied on the global side when the unit is fetched and
// again when it is read back. (A 128-bit read serves sixteen lanes together - sixteen consecutive
// rows, one unit each; rows of 128 bytes alternate between the two halves of the 64 banks, and the
// eight rows of one parity take eight different units: every bank once.) The loads are opaque to
// the compiler (inline asm), so completion is awaited by hand (vmcnt) before the block-wide barrier
// that publishes a stage.
//
// SWIGLU: the block's B tile is half gate columns, half up columns of one joint weight matrix,
// arranged so that a wavefront's first accumulator column holds gate values and its second the up
// values of the SAME output columns; the epilogue writes silu(gate) * up, BN / 2 columns per tile.
//
// EDGE: m and n need not be whole tiles (K steps stay whole, rows 16-byte aligned). Rows and columns
// past the end are fetched from the last valid row / 16-byte unit instead -- what they feed is
// never stored -- so the main loop is the same; only the stores are guarded.
//
// WS: a K-contiguous B stored as 16-bit values. LDS holds floats in the same swizzled layout, so
// fragments, MFMAs and epilogue are those of the fp32 kernel and the result equals the fp32 product
// over the widened weights bit for bit. Only B's way into LDS differs: every lane fetches 128-bit
// units of eight weights into registers one K step ahead of A's direct loads, and widens and stores
// them as two units of four floats at the start of the next step (dealt out between the MFMAs like
// every other instruction of a step).
template <int BM, int BN, int WM, int WN, bool TB, int STAGES, bool SWIGLU = false, bool EDGE = false,
          typename WS = StoredF32>
__global__ __launch_bounds__(kThreads) void gemm_mfma_direct_kernel(GemmArgs g) {
    static_assert(STAGES == 2, "two LDS stages");
    constexpr bool B16 = kStored16<WS>;
    static_assert(!B16 || TB, "16-bit weights are K-contiguous");
    static_assert(!SWIGLU || WN == 64,
                  "SwiGLU epilogue: two accumulator columns (EDGE: partial tiles in m only)");
    constexpr int BK = 32;
    constexpr int KC = BK / 8;
    constexpr int kAFloats = BM * BK;   // one stage of A, floats
    constexpr int kBFloats = BK * BN;
    extern __shared__ __align__(16) float smem[];
    float *As = smem;                        // [STAGES][BM][BK] swizzled
    float *Bs = smem + STAGES * kAFloats;    // [STAGES][BK][BN], or [STAGES][BN][BK] swizzled (TB)

    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int WAVES_N = BN / WN;
    static_assert((BM / WM) * (BN / WN) == kThreads / kWave, "four wavefronts per block");
    constexpr int A_PASSES = BM / 32;   // 1 KiB pieces (8 rows of A) per wavefront and stage
    constexpr int B_PASSES = B16 ? 0 : BN / 32;
    constexpr int B_ROW_UNITS = BN / 4;             // 16-byte units per K-row of a row-major B tile
    // 16-bit B: 128-bit units of eight weights per stage (four per row), dealt to the 256 lanes
    constexpr int B16_UNITS = BN * 4;
    constexpr int B16_PASSES = B16 ? (B16_UNITS + kThreads - 1) / kThreads : 0;
    constexpr int kB16Slots = B16_PASSES > 0 ? B16_PASSES : 1;

    int tile_m, tile_n, split;
    tile_coords(g, tile_m, tile_n, split);
    const int batch = blockIdx.y;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int k_begin = split * g.k_per_split;
    const int k_end = min(g.k, k_begin + g.k_per_split);
    const int n_steps = (k_end - k_begin) / BK;

    const float *A = g.a + batch * g.stride_a;
    const float *B = g.b + batch * g.stride_b;
    float *C = g.c + (static_cast<int64_t>(split) * gridDim.y + batch) * g.stride_c;

    const int tid = threadIdx.x;
    const int lane = tid % kWave;
    const int wave = tid / kWave;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane % 32, half = lane / 32;

    // Global sources of a stage: piece (p * 4 + wave) goes to this wavefront. The address is a
    // wave-uniform base (scalar registers, advanced by one K step with scalar adds) plus a per-lane
    // byte offset per piece that never changes, so the loads cost no vector ALU work.
    const int sw_row = lane / 8, sw_unit = (lane % 8) ^ ((wave * 4 + sw_row / 2) & 7);
    uint32_t a_voff[A_PASSES], b_voff[B_PASSES > 0 ? B_PASSES : 1];
    const float *a_ptr = A + static_cast<int64_t>(m0) * g.lda + k_begin;
#pragma unroll
    for (int p = 0; p < A_PASSES; ++p) {
        int row = p * 32 + wave * 8 + sw_row;
        if constexpr (EDGE) row = min(row, g.m - 1 - m0);
        a_voff[p] = static_cast<uint32_t>((row * g.lda + sw_unit * 4) * static_cast<int64_t>(4));
    }
    const float *b_ptr = nullptr;
    int64_t b_step_stride = 0;
    // 16-bit B: the unit this lane fetches in pass p, as a byte offset from b16_ptr (which walks K),
    // and the float index of the first of the two LDS units it becomes (stage 0)
    [[maybe_unused]] const uint16_t *b16_ptr = nullptr;
    [[maybe_unused]] uint32_t b16_voff[kB16Slots];
    [[maybe_unused]] int b16_lds[kB16Slots][2];
    [[maybe_unused]] v4u b_raw[kB16Slots];
    if constexpr (B16) {
        b16_ptr = reinterpret_cast<const uint16_t *>(g.b) + batch * g.stride_b +
                  (SWIGLU ? 0 : static_cast<int64_t>(n0) * g.ldb) + k_begin;
#pragma unroll
        for (int p = 0; p < B16_PASSES; ++p) {
            const int id = min(p * kThreads + tid, B16_UNITS - 1);
            const int lrow = id / 4, u = id % 4;       // row of the tile, unit of eight weights in it
            int row = lrow;
            if constexpr (SWIGLU) {
                // LDS row r: wavefront column r / 64, accumulator (r % 64) / 32, lane r % 32
                const int out_col = tile_n * (BN / 2) + (row / 64) * 32 + row % 32;
                row = ((row % 64) / 32 ? g.up_offset : g.gate_offset) + out_col;
            } else if constexpr (EDGE) {
                row = min(row, g.n - 1 - n0);
            }
            b16_voff[p] = static_cast<uint32_t>((row * g.ldb + u * 8) * static_cast<int64_t>(2));
            b16_lds[p][0] = lrow * BK + ((2 * u) ^ ((lrow >> 1) & 7)) * 4;
            b16_lds[p][1] = lrow * BK + ((2 * u + 1) ^ ((lrow >> 1) & 7)) * 4;
        }
    } else if constexpr (TB) {
        b_ptr = B + (SWIGLU ? 0 : static_cast<int64_t>(n0) * g.ldb) + k_begin;
        b_step_stride = BK;
#pragma unroll
        for (int p = 0; p < B_PASSES; ++p) {
            int row = p * 32 + wave * 8 + sw_row;
            if constexpr (SWIGLU) {
                // LDS row r: wavefront column r / 64, accumulator (r % 64) / 32, lane r % 32
                const int out_col = tile_n * (BN / 2) + (row / 64) * 32 + row % 32;
                row = ((row % 64) / 32 ? g.up_offset : g.gate_offset) + out_col;
            } else if constexpr (EDGE) {
                row = min(row, g.n - 1 - n0);
            }
            b_voff[p] = static_cast<uint32_t>((row * g.ldb + sw_unit * 4) * static_cast<int64_t>(4));
        }
    } else {
        b_ptr = B + static_cast<int64_t>(k_begin) * g.ldb + (SWIGLU ? 0 : n0);
        b_step_stride = static_cast<int64_t>(BK) * g.ldb;
#pragma unroll
        for (int p = 0; p < B_PASSES; ++p) {
            // the tile is [BK][BN] in LDS, filled in 1 KiB pieces of 64 consecutive 16-byte units
            const int unit = (p * 4 + wave) * kWave + lane;
            const int krow = unit / B_ROW_UNITS;
            int col = (unit % B_ROW_UNITS) * 4;    // LDS column of the tile this lane fills
            if constexpr (SWIGLU) {
                // LDS column c: wavefront column c / 64, accumulator (c % 64) / 32, lane c % 32
                const int out_col = tile_n * (BN / 2) + (col / 64) * 32 + col % 32;
                col = ((col % 64) / 32 ? g.up_offset : g.gate_offset) + out_col;
            } else if constexpr (EDGE) {
                col = min(col, g.n - 4 - n0);
            }
            b_voff[p] = static_cast<uint32_t>((krow * g.ldb + col) * static_cast<int64_t>(4));
        }
    }
    // LDS byte addresses of this wavefront's first piece of A and B in stage 0 (wave-uniform)
    const uint32_t lds_a = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(As)) + wave * 1024u);
    const uint32_t lds_b = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(Bs)) + wave * 1024u);

    auto direct_load = [&](uint32_t lds_addr, const float *base, uint32_t voff) {
        // (one wait state between a scalar write of M0 and the LDS-bound load that reads it)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(base)
                     : "memory", "m0");
    };
    constexpr int kLoadsPerStage = A_PASSES + B_PASSES;
    // load number o of the stage that goes to LDS buffer `buf`
    auto load_op = [&](int buf, int o) {
        if (o < A_PASSES)
            direct_load(lds_a + static_cast<uint32_t>(buf * kAFloats * 4 + o * 4096), a_ptr, a_voff[o]);
        else
            direct_load(lds_b + static_cast<uint32_t>(buf * kBFloats * 4 + (o - A_PASSES) * 4096), b_ptr,
                        b_voff[o - A_PASSES]);
    };
    auto advance_sources = [&]() {
        a_ptr += BK;
        b_ptr += b_step_stride;
    };
    // 16-bit B: request pass p of the stage b16_ptr stands at; widen and store pass p of the stage in
    // the registers to LDS buffer `buf`
    [[maybe_unused]] auto b16_load = [&](int p) {
        if constexpr (B16) {
            if (B16_UNITS % kThreads == 0 || p * kThreads + tid < B16_UNITS)
                b_raw[p] = *reinterpret_cast<const v4u *>(reinterpret_cast<const char *>(b16_ptr) + b16_voff[p]);
        }
    };
    // (one half of a unit per call: four values widened, one 128-bit LDS store - a short enough run
    // of instructions to fit between two MFMAs)
    [[maybe_unused]] auto b16_store = [&](int buf, int p, int h) {
        if constexpr (B16) {
            if (B16_UNITS % kThreads == 0 || p * kThreads + tid < B16_UNITS) {
                float w0, w1, w2, w3;
                WS::widen2(b_raw[p][2 * h], w0, w1);
                WS::widen2(b_raw[p][2 * h + 1], w2, w3);
                *reinterpret_cast<v4f *>(Bs + buf * kBFloats + b16_lds[p][h]) = v4f{w0, w1, w2, w3};
            }
        }
    };

    // fragment addressing
    const int xr = (l32 >> 1) & 7;
    const int a_row = (wm * WM + l32) * BK;
    const int b_base = TB ? (wn * WN + l32) * BK : (half * 4) * BN + wn * WN + l32;
    v4f af[2][TM];
    float bf[2][TN][4];
    // The fragments of one 8-wide K chunk are fetched by kFragOps LDS reads: TM 128-bit reads of A,
    // then B as TN 128-bit reads (K-contiguous B) or 2 * TN pairs of 32-bit reads.
    constexpr int kFragOps = TM + (TB ? TN : 2 * TN);
    // in the order the MFMAs want them: A row block 0, the first half of every B column block,
    // the other A row blocks, the second halves of B
    auto frag_op = [&](int buf, int kc, int slot, int o) {
        const int unit = ((kc * 2 + half) ^ xr) * 4;
        if (o == 0 || (o > TN && o < TN + TM)) {
            const int i = o == 0 ? 0 : o - TN;
            af[slot][i] = *reinterpret_cast<const v4f *>(As + buf * kAFloats + a_row + i * 32 * BK + unit);
        } else if constexpr (TB) {
            const int j = o - 1;
            const v4f bv = *reinterpret_cast<const v4f *>(Bs + buf * kBFloats + b_base + j * 32 * BK + unit);
#pragma unroll
            for (int s = 0; s < 4; ++s) bf[slot][j][s] = bv[s];
        } else {
            const int j = o <= TN ? o - 1 : o - TN - TM, s0 = o <= TN ? 0 : 2;
            const float *bs = Bs + buf * kBFloats + b_base + j * 32;
            bf[slot][j][s0] = bs[(kc * 8 + s0) * BN];
            bf[slot][j][s0 + 1] = bs[(kc * 8 + s0 + 1) * BN];
        }
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // This wavefront's LDS reads are complete and its direct loads have landed; then the block
    // meets: the stage just loaded may be read, the stage just read may be overwritten.
    auto stage_barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // One K step. The matrix pipe takes a new MFMA every 64 cycles and the wavefront issues in
    // order, so everything else -- the next chunk's fragment reads, the next stage's global loads,
    // the barrier -- is dealt out between the MFMAs a few instructions at a time instead of in
    // bursts that would let the pipe run dry. Chunks 0 .. KC-2 read the fragments of the chunk after
    // them and issue the loads of the next stage; the last chunk meets the block a quarter of the
    // way in and then reads chunk 0 of the next stage.
    constexpr int NM = 4 * TM * TN;                  // MFMAs per chunk
    constexpr int kLoadChunks = 1;   // chunks (from the first) that carry the loads
    constexpr int kLoadsPerChunk = (kLoadsPerStage + kLoadChunks - 1) / kLoadChunks;
    constexpr int kBarrierAt = NM * 2 / 4 < NM - 1 ? NM * 2 / 4 : NM - 2;
    // (The LDS buffer of a step is fixed in its code, two steps per trip of the loop: the addresses
    // of the fragment reads are then a lane offset that never changes plus an immediate. With the
    // buffer in a register every read had a vector add in front of it, and a vector ALU
    // instruction between two MFMAs whose result an LDS read waits for holds the next MFMA back
    // by some 25 cycles.)
    auto k_step = [&](auto buf_tag, auto load_tag, auto more_tag, auto load2_tag) {
        constexpr int buf = decltype(buf_tag)::value;
        constexpr bool LOAD = decltype(load_tag)::value;   // another stage to fetch
        constexpr bool MORE = decltype(more_tag)::value;   // another step follows
        constexpr bool LOAD2 = decltype(load2_tag)::value; // 16-bit B: a stage after that one to request
        constexpr int other = buf ^ 1;
        static_for<KC>([&](auto kc_tag) {
            constexpr int kc = decltype(kc_tag)::value;
            constexpr int slot = kc & 1;
            constexpr bool last = kc == KC - 1;
            constexpr bool loads_here = LOAD && kc < kLoadChunks;
            constexpr int load_lo = loads_here ? (kc * kLoadsPerChunk < kLoadsPerStage ? kc * kLoadsPerChunk
                                                                                       : kLoadsPerStage)
                                               : 0;
            constexpr int load_hi =
                loads_here ? ((kc + 1) * kLoadsPerChunk < kLoadsPerStage ? (kc + 1) * kLoadsPerChunk
                                                                         : kLoadsPerStage)
                           : 0;
            constexpr int n_frag = last ? (MORE ? kFragOps : 0) : kFragOps;
            // 16-bit B, first chunk: the stage in the registers goes to LDS before the loads of this
            // step are issued, the stage after it is requested behind them
            constexpr int n_store = B16 && LOAD && kc == 0 ? 2 * B16_PASSES : 0;
            constexpr int n_direct = load_hi - load_lo;
            constexpr int n_b16 = B16 && LOAD2 && kc == 0 ? B16_PASSES : 0;
            constexpr int n_ops = n_frag + n_store + n_direct + n_b16;
            constexpr int first = last ? kBarrierAt + 1 : 0;     // first MFMA that carries an op
            constexpr int room = NM - first;
            static_for<NM>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value;
                constexpr int s = q / (TM * TN), i = (q / TN) % TM, j = q % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[slot][i][s], bf[slot][j][s],
                                                                 acc[i][j], 0, 0, 0);
                if constexpr (last && MORE && q == kBarrierAt) stage_barrier();
                static_for<n_ops>([&](auto o_tag) {
                    constexpr int o = decltype(o_tag)::value;
                    // one op per MFMA from `first` on while they fit, else spread evenly
                    if constexpr ((n_ops <= room ? first + o : first + o * room / n_ops) == q) {
                        if constexpr (o < n_frag) {
                            if constexpr (last) frag_op(other, 0, slot ^ 1, o);
                            else frag_op(buf, kc + 1, slot ^ 1, o);
                        } else if constexpr (o < n_frag + n_store) {
                            b16_store(other, (o - n_frag) / 2, (o - n_frag) % 2);
                        } else if constexpr (o < n_frag + n_store + n_direct) {
                            load_op(other, load_lo + o - n_frag - n_store);
                        } else {
                            b16_load(o - n_frag - n_store - n_direct);
                        }
                    }
                });
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (LOAD && kc == kLoadChunks - 1) advance_sources();
            if constexpr (B16 && LOAD2 && kc == 0) b16_ptr += BK;
        });
    };

    if (n_steps > 0) {
#pragma unroll
        for (int o = 0; o < kLoadsPerStage; ++o) load_op(0, o);
        advance_sources();
        if constexpr (B16) {
            // stage 0 of B through the registers, then stage 1 requested
#pragma unroll
            for (int p = 0; p < B16_PASSES; ++p) b16_load(p);
            b16_ptr += BK;
#pragma unroll
            for (int p = 0; p < B16_PASSES; ++p) {
                b16_store(0, p, 0);
                b16_store(0, p, 1);
            }
            if (n_steps > 1) {
#pragma unroll
                for (int p = 0; p < B16_PASSES; ++p) b16_load(p);
                b16_ptr += BK;
            }
        }
        stage_barrier();
#pragma unroll
        for (int o = 0; o < kFragOps; ++o) frag_op(0, 0, 0, o);
        const std::integral_constant<int, 0> even{};
        const std::integral_constant<int, 1> odd{};
        const std::true_type yes{};
        const std::false_type no{};
        int left = n_steps;   // steps to go; the next one reads buffer 0
        if constexpr (B16) {
            // the last step fetches nothing, the one before it requests no stage behind the one it fetches
            for (; left > 3; left -= 2) {
                k_step(even, yes, yes, yes);
                k_step(odd, yes, yes, yes);
            }
            if (left == 3) {
                k_step(even, yes, yes, yes);
                k_step(odd, yes, yes, no);
                k_step(even, no, no, no);
            } else if (left == 2) {
                k_step(even, yes, yes, no);
                k_step(odd, no, no, no);
            } else {
                k_step(even, no, no, no);
            }
        } else {
            for (; left > 2; left -= 2) {
                k_step(even, yes, yes, no);
                k_step(odd, yes, yes, no);
            }
            if (left == 2) {
                k_step(even, yes, yes, no);
                k_step(odd, no, no, no);
            } else {
                k_step(even, no, no, no);
            }
        }
    }

    if constexpr (SWIGLU) {
        const int col = tile_n * (BN / 2) + wn * 32 + l32;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                const float gate = acc[i][0][r];
                const float silu = gate * (1.0f / (1.0f + expf(-gate)));
                if (!EDGE || row < g.m) C[static_cast<int64_t>(row) * g.ldc + col] = silu * acc[i][1][r];
            }
        }
        return;
    }
    const bool segmented = g.n_seg > 0 && gridDim.z == 1;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        // destination of this 32-column block (block boundaries are multiples of 32)
        const int cb = n0 + wn * WN + j * 32;
        float *dst = C;
        int64_t ldc = g.ldc;
        int col = cb + l32;
        if (segmented) {
            // constant indices only: the argument struct stays in scalar registers
            dst = g.seg_c[0];
            ldc = g.seg_ldc[0];
#pragma unroll
            for (int sgm = 1; sgm < kMaxSegments; ++sgm)
                if (sgm < g.n_seg && cb >= g.seg_begin[sgm]) {
                    dst = g.seg_c[sgm];
                    ldc = g.seg_ldc[sgm];
                    col = cb - g.seg_begin[sgm] + l32;
                }
        }
        if (EDGE && cb + l32 >= g.n) continue;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                if (!EDGE || row < g.m) dst[static_cast<int64_t>(row) * ldc + col] = acc[i][j][r];
            }
        }
    }
}

// Sum `splits` partial matrices laid out [split][batch][m][n] into C (fixed order).
__global__ __launch_bounds__(kThreads) void splitk_reduce_kernel(const float *__restrict__ ws,
                                                                 float *__restrict__ c, int splits,
                                                                 int64_t batch, int32_t m,
                                                                 int32_t n, int64_t ldc,
                                                                 int64_t stride_c) {
    const int64_t per = static_cast<int64_t>(m) * n;
    const int64_t total = batch * per;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        float s = 0.f;
        for (int z = 0; z < splits; ++z) s += ws[z * total + i];
        const int64_t b = i / per, rem = i - b * per;
        const int64_t r = rem / n, col = rem - r * n;
        c[b * stride_c + r * ldc + col] = s;
    }
}

// Destinations of the column blocks of one [m][n] matrix (see GemmArgs).
struct Segments {
    int32_t n_seg;
    int32_t begin[kMaxSegments + 1];
    float *c[kMaxSegments];
    int64_t ldc[kMaxSegments];
};

// The same sum, four columns per lane; n, every block boundary and every leading dimension are
// multiples of 4 and all pointers 16-byte aligned. One matrix (batch 1).
__global__ __launch_bounds__(kThreads) void splitk_reduce_vec_kernel(const float *__restrict__ ws,
                                                                     Segments sg, int splits,
                                                                     int32_t m, int32_t n) {
    const int n4 = n / 4;
    const int64_t total4 = static_cast<int64_t>(m) * n4;
    const int64_t slab = static_cast<int64_t>(m) * n;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total4;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        const float *src = ws + i * 4;
        v4f s = *reinterpret_cast<const v4f *>(src);
        for (int z = 1; z < splits; ++z) s += *reinterpret_cast<const v4f *>(src + z * slab);
        const int r = static_cast<int>(i / n4);
        const int col = static_cast<int>(i - static_cast<int64_t>(r) * n4) * 4;
        float *dst = sg.c[0];
        int64_t ldc = sg.ldc[0];
        int col0 = col;
#pragma unroll
        for (int j = 1; j < kMaxSegments; ++j)
            if (j < sg.n_seg && col >= sg.begin[j]) {
                dst = sg.c[j];
                ldc = sg.ldc[j];
                col0 = col - sg.begin[j];
            }
        *reinterpret_cast<v4f *>(dst + static_cast<int64_t>(r) * ldc + col0) = s;
    }
}

// ---- GEMV: y[n] = sum_k x[k] * W[k][n], W row-major -------------------------------------------
// A block covers kThreads / 64 * ... columns: VEC columns per lane, 64 lanes per wavefront, and
// the block's 4 wavefronts split the block's K slice; partial sums meet in LDS.
constexpr int kGemvRowMajorDepth = 16;

struct GemvArgs {
    const float *x;   // [batch][k], element stride x_inc
    const float *w;
    float *y;         // y or partial workspace [split][batch][n]
    int32_t n, k;
    int64_t x_inc, ldb;
    int64_t stride_x, stride_w, stride_y;
    int32_t k_per_split;
};



template <int VEC>
__global__ __launch_bounds__(kThreads) void gemv_kernel(GemvArgs g) {
    constexpr int kWaves = kThreads / kWave;
    constexpr int kCols = kWave * VEC;  // columns per block
    __shared__ float red[kWaves][kCols];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int batch = blockIdx.y, split = blockIdx.z;
    const int col = blockIdx.x * kCols + lane * VEC;
    const int k_begin = split * g.k_per_split;
    const int k_end = min(g.k, k_begin + g.k_per_split);
    const float *x = g.x + batch * g.stride_x;
    const float *w = g.w + batch * g.stride_w;

    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;

    // this wavefront's contiguous quarter of the slice
    const int len = k_end - k_begin;
    const int per_wave = (len + kWaves - 1) / kWaves;
    const int kb = k_begin + wave * per_wave;
    const int ke = min(k_end, kb + per_wave);
    if (col < g.n) {
        const float *wp = w + static_cast<int64_t>(kb) * g.ldb + col;
        int kk = kb;
        if constexpr (VEC == 4) {
            // U rows of weights requested before any is used: a slab of 16 rows per wavefront is
            // one round trip to HBM
            auto rows = [&](auto u_tag) {
                constexpr int U = decltype(u_tag)::value;
                v4f wv[U];
                float xv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    wv[u] = __builtin_nontemporal_load(
                        reinterpret_cast<const v4f *>(wp + static_cast<int64_t>(u) * g.ldb));
                    xv[u] = x[static_cast<int64_t>(kk + u) * g.x_inc];
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[j] = fmaf(xv[u], wv[u][j], acc[j]);
                wp += static_cast<int64_t>(U) * g.ldb;
                kk += U;
            };
            while (kk + kGemvRowMajorDepth <= ke) rows(std::integral_constant<int, kGemvRowMajorDepth>{});
            if (kGemvRowMajorDepth > 8 && kk + 8 <= ke) rows(std::integral_constant<int, 8>{});
            if (kk + 4 <= ke) rows(std::integral_constant<int, 4>{});
            for (; kk < ke; ++kk) {
                v4f wv = *reinterpret_cast<const v4f *>(wp);
                float xv = x[static_cast<int64_t>(kk) * g.x_inc];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = fmaf(xv, wv[j], acc[j]);
                wp += g.ldb;
            }
        } else {
            constexpr int U = 8;
            for (; kk + U <= ke; kk += U) {
                float wv[U], xv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    wv[u] = wp[static_cast<int64_t>(u) * g.ldb];
                    xv[u] = x[static_cast<int64_t>(kk + u) * g.x_inc];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) acc[0] = fmaf(xv[u], wv[u], acc[0]);
                wp += static_cast<int64_t>(U) * g.ldb;
            }
            for (; kk < ke; ++kk) {
                acc[0] = fmaf(x[static_cast<int64_t>(kk) * g.x_inc], *wp, acc[0]);
                wp += g.ldb;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) red[wave][lane * VEC + j] = acc[j];
    __syncthreads();
    // one split: y itself; several: this split's slab of the workspace [split][batch][n]
    float *y = g.y + (static_cast<int64_t>(split) * gridDim.y + batch) * g.stride_y;
    for (int c = threadIdx.x; c < kCols; c += kThreads) {
        const int oc = blockIdx.x * kCols + c;
        if (oc < g.n) {
            float s = 0.f;
#pragma unroll
            for (int wv = 0; wv < kWaves; ++wv) s += red[wv][c];
            y[oc] = s;
        }
    }
}

// Combine GEMV partials [split][total] -> y: 32 outputs per block, 8 lanes per output take the
// splits round-robin with four independent loads in flight, then the eight sums meet in LDS in
// a fixed order (the result depends on `splits` only, never on timing).
__global__ __launch_bounds__(kThreads) void gemv_reduce_kernel(const float *__restrict__ ws,
                                                               float *__restrict__ y, int splits,
                                                               int64_t batch, int32_t m, int32_t n,
                                                               int64_t ldc, int64_t stride_y) {
    constexpr int kOut = 32, kGroups = kThreads / kOut;
    __shared__ float part[kGroups][kOut];
    const int64_t per = static_cast<int64_t>(m) * n;
    const int64_t total = batch * per;
    const int ox = threadIdx.x % kOut, sy = threadIdx.x / kOut;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kOut + ox;
    float s = 0.f;
    if (i < total) {
        const float *p = ws + i;
        int z = sy;
        for (; z + 3 * kGroups < splits; z += 4 * kGroups) {
            const float v0 = p[static_cast<int64_t>(z) * total];
            const float v1 = p[static_cast<int64_t>(z + kGroups) * total];
            const float v2 = p[static_cast<int64_t>(z + 2 * kGroups) * total];
            const float v3 = p[static_cast<int64_t>(z + 3 * kGroups) * total];
            s += (v0 + v1) + (v2 + v3);
        }
        for (; z < splits; z += kGroups) s += p[static_cast<int64_t>(z) * total];
    }
    part[sy][ox] = s;
    __syncthreads();
    if (sy == 0 && i < total) {
        const int64_t b = i / per, rem = i - b * per;
        const int64_t row = rem / n, col = rem - row * n;
        float r = 0.f;
#pragma unroll
        for (int q = 0; q < kGroups; ++q) r += part[q][ox];
        y[b * stride_y + row * ldc + col] = r;
    }
}

// ---- skinny GEMM: 2..8 rows of A against a streamed B ---------------------------------------------
// The decode-time shapes of grouped-query attention (the few query heads of one KV head against
// its cache) and of small-batch projections: B is read from HBM once, every lane keeps ROWS x 4
// accumulators. Same blocking as gemv_kernel<4>; rows beyond m are computed on row m-1 and dropped.
struct SkinnyArgs {
    const float *x;   // [batch][m][k] rows of lda
    const float *w;   // [batch][k][n] rows of ldb, or [n][k] for the dot kernel
    float *y;         // C, or partial workspace [split][batch][m][n]
    int32_t m, n, k;
    int64_t lda, ldb, ldy;
    int64_t stride_x, stride_w, stride_y;
    int32_t k_per_split;
};

template <int ROWS>
__global__ __launch_bounds__(kThreads) void skinny_kernel(SkinnyArgs g) {
    constexpr int kWaves = kThreads / kWave;
    constexpr int kCols = kWave * 4;
    __shared__ float red[kWaves][ROWS][kCols];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int batch = blockIdx.y, split = blockIdx.z;
    const int col = blockIdx.x * kCols + lane * 4;
    const int k_begin = split * g.k_per_split;
    const int k_end = min(g.k, k_begin + g.k_per_split);
    const float *x = g.x + batch * g.stride_x;
    const float *w = g.w + batch * g.stride_w;
    const float *xr[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) xr[r] = x + static_cast<int64_t>(min(r, g.m - 1)) * g.lda;

    float acc[ROWS][4];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[r][j] = 0.f;

    const int len = k_end - k_begin;
    const int per_wave = (len + kWaves - 1) / kWaves;
    const int kb = k_begin + wave * per_wave;
    const int ke = min(k_end, kb + per_wave);
    if (col < g.n) {
        const float *wp = w + static_cast<int64_t>(kb) * g.ldb + col;
        int kk = kb;
        constexpr int U = 4;
        for (; kk + U <= ke; kk += U) {
            v4f wv[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                wv[u] = __builtin_nontemporal_load(
                    reinterpret_cast<const v4f *>(wp + static_cast<int64_t>(u) * g.ldb));
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const float xv = xr[r][kk + u];
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[r][j] = fmaf(xv, wv[u][j], acc[r][j]);
                }
            wp += static_cast<int64_t>(U) * g.ldb;
        }
        for (; kk < ke; ++kk) {
            const v4f wv = *reinterpret_cast<const v4f *>(wp);
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const float xv = xr[r][kk];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[r][j] = fmaf(xv, wv[j], acc[r][j]);
            }
            wp += g.ldb;
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[wave][r][lane * 4 + j] = acc[r][j];
    __syncthreads();
    float *y = g.y + (static_cast<int64_t>(split) * gridDim.y + batch) * g.stride_y;
    for (int t = threadIdx.x; t < ROWS * kCols; t += kThreads) {
        const int r = t / kCols, c = t - r * kCols;
        const int oc = blockIdx.x * kCols + c;
        if (r < g.m && oc < g.n) {
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < kWaves; ++wv) sum += red[wv][r][c];
            y[static_cast<int64_t>(r) * g.ldy + oc] = sum;
        }
    }
}

// B stored [n][k] (C = A . B^T): a wavefront per output column, ROWS dots along contiguous k.
// (WS: B may be stored as 16-bit values, see StoredF16; g.w, ldb and stride_w then count those.)
template <int ROWS, typename WS = StoredF32>
__global__ __launch_bounds__(kThreads) void skinny_dot_kernel(SkinnyArgs g) {
    using E = typename WS::elem;
    const int lane = threadIdx.x % kWave;
    const int batch = blockIdx.y;
    const float *x = g.x + batch * g.stride_x;
    const E *w = reinterpret_cast<const E *>(g.w) + batch * g.stride_w;
    float *y = g.y + batch * g.stride_y;
    const float *xr[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) xr[r] = x + static_cast<int64_t>(min(r, g.m - 1)) * g.lda;
    for (int n = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave; n < g.n;
         n += gridDim.x * (kThreads / kWave)) {
        const E *wr = w + static_cast<int64_t>(n) * g.ldb;
        float acc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[r] = 0.f;
        for (int kk = lane; kk < g.k; kk += kWave) {
            float wv;
            if constexpr (kStored16<WS>) wv = WS::widen(wr[kk]);
            else wv = wr[kk];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[r] = fmaf(xr[r][kk], wv, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
#pragma unroll
            for (int o = kWave / 2; o > 0; o >>= 1) acc[r] += __shfl_xor(acc[r], o, kWave);
            if (lane == 0 && r < g.m) y[static_cast<int64_t>(r) * g.ldy + n] = acc[r];
        }
    }
}

// GEMV with W stored [n][k] (trans_b): a wavefront per output column, dot along contiguous k.
template <typename WS = StoredF32>
__global__ __launch_bounds__(kThreads) void gemv_dot_kernel(GemvArgs g) {
    using E = typename WS::elem;
    const int lane = threadIdx.x % kWave;
    const int batch = blockIdx.y;
    const float *x = g.x + batch * g.stride_x;
    const E *w = reinterpret_cast<const E *>(g.w) + batch * g.stride_w;
    float *y = g.y + batch * g.stride_y;
    for (int n = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave; n < g.n;
         n += gridDim.x * (kThreads / kWave)) {
        const E *wr = w + static_cast<int64_t>(n) * g.ldb;
        float acc = 0.f;
        for (int kk = lane; kk < g.k; kk += kWave) {
            float wv;
            if constexpr (kStored16<WS>) wv = WS::widen(wr[kk]);
            else wv = wr[kk];
            acc = fmaf(x[static_cast<int64_t>(kk) * g.x_inc], wv, acc);
        }
#pragma unroll
        for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
        if (lane == 0) y[n] = acc;
    }
}

// One-row product with K-contiguous weights, y[n] = sum_k x[k] * Wt[n][k]: a wavefront owns ONE output
// and walks its row(s) of Wt in chunks of eight 128-bit units per lane (8 KiB per wavefront and row
// in flight, streaming loads), x following the weights; the lanes' partial sums meet in a DPP
// reduction. A column is finished inside its wavefront, so there is no split-K, no workspace and
// no combine launch whatever the width. (Measured against two and four outputs per wavefront and
// against wavefronts that walk several rows with the next row's loads in flight: the short-lived
// wavefront with eight loads per lane wins at every width, 20.0 against 23.9 us on 16384 x 2048
// and 142 against 158 us on 128256 x 2048, 7.4 TB/s.)
// SWIGLU: the wavefront's two rows of Wt are the gate and the up row of its output (rows
// gate_row + i and up_row + i, sharing the loads of x); it writes silu(gate) * up.
// NORM: x is the row BEFORE an RMSNorm and the product is taken with RMSNorm(x) * gamma, which is
// never stored in memory: every block first normalises the row into LDS exactly as the norm
// kernel's block-per-row form does (squares rounded to float, summed in double per lane, wavefront
// and block in that kernel's order), so the result equals the norm kernel followed by the product
// bit for bit. The block's loads of x and gamma are issued BEFORE the first weight loads (loads of a
// wavefront return in order: behind the weights, the row - which the caches hold - would arrive
// only after a full trip to HBM) and the arithmetic runs while the weights are in flight.
// `residual` (may be null) is added to the outputs (the Add behind an output projection).
struct RowNormArgs {
    const float *gamma;
    float eps;
    int32_t reciprocal;
};

constexpr int kGemvDepth = 8;                    // 128-bit units per lane, row and chunk
constexpr int kGemvNormUnits = 8;                // NORM: units of x a lane holds (k <= 256 * 8 * 4)

// The dot products of one wavefront: COLS rows of Wt (wv[c], K-contiguous) with x or, NORM, with
// RMSNorm(x) * gamma formed by the whole block in LDS. Every wavefront of the block calls this
// (barriers); one that is not `active` skips the products. acc[c] is valid in every lane.
struct NoExtraLoads {
    __device__ __forceinline__ void operator()() const {}
};
// `extra_loads()` is called once the first chunk of weights has been requested: loads an epilogue
// needs, on their way with the weights but not in front of the row (loads return in order).
// NU: 128-bit units of the row a lane holds during the NORM prologue (k <= 256 * NU * 4); the
// common k <= 2048 takes NU = 2 and with it 48 registers less than NU = 8, i.e. five or six
// resident wavefronts per SIMD instead of four.
// WS, DEPTH: how the weights are stored and how many 128-bit units of a row a lane requests per
// chunk. A unit of 16-bit weights meets two units of x; rows of up to 2048 such weights are one
// chunk of four units per lane, longer ones chunks of eight.
template <int COLS, bool NORM, int NU = kGemvNormUnits, typename WS = StoredF32, int DEPTH = kGemvDepth,
          typename Extra = NoExtraLoads>
__device__ __forceinline__ void gemv_wave_dots(const float *__restrict__ x, const v4f *const (&wv)[COLS],
                                               int32_t k, const RowNormArgs &norm, bool active,
                                               float (&acc)[COLS], Extra extra_loads = Extra()) {
    constexpr int kWaves = kThreads / kWave;
    constexpr int kX = WS::kUnit / 4;          // units of x one unit of weights meets
    // the normalised row of the block (NORM): k floats of dynamic LDS
    extern __shared__ __align__(16) float xs[];
    __shared__ double partial[kWaves];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int k4 = k / 4;                      // units of x
    const int kw = k / WS::kUnit;              // units of a row of weights
    const v4f *xv = reinterpret_cast<const v4f *>(x);
    // NORM: this lane's share of the row and of gamma, requested before any weight
    [[maybe_unused]] v4f xn[NU], gn[NU];
    if constexpr (NORM) {
        const v4f *gv = reinterpret_cast<const v4f *>(norm.gamma);
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int c = threadIdx.x + i * kThreads;
            if (i * kThreads < k4) {             // (uniform)
                xn[i] = xv[min(c, k4 - 1)];
                gn[i] = gv[min(c, k4 - 1)];
            }
        }
    }
    // Chunks of DEPTH * 64 units. Whole chunks are addressed as pointer + constant (the loads
    // carry their offsets as immediates: with two wavefronts per SIMD, as on the 2048-wide outputs,
    // address arithmetic per load is time nothing else covers - it cost the k = 8192 product 2 us);
    // the last, partial chunk of a row that is no whole number of chunks clamps its units and
    // zeroes them.
    constexpr int kChunkUnits = kWave * DEPTH;
    const int full_chunks = kw / kChunkUnits;
    v4f wr[DEPTH][COLS];
    auto load_w = [&](int chunk, bool partial_chunk) {
        if (!partial_chunk) {
#pragma unroll
            for (int c = 0; c < COLS; ++c) {
                const v4f *p = wv[c] + chunk * kChunkUnits + lane;
#pragma unroll
                for (int j = 0; j < DEPTH; ++j) wr[j][c] = __builtin_nontemporal_load(p + j * kWave);
            }
        } else {
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) {
                const int u = min(chunk * kChunkUnits + lane + j * kWave, kw - 1);
#pragma unroll
                for (int c = 0; c < COLS; ++c) wr[j][c] = __builtin_nontemporal_load(wv[c] + u);
            }
        }
    };
    // one unit of weights against the units of x under it
    auto unit_fma = [&](const v4f (&xu)[kX], const v4f &w, float &sum) {
        if constexpr (kStored16<WS>) {
            float wf[8];
            widen_unit<WS>(__builtin_bit_cast(v4u, w), wf);
#pragma unroll
            for (int e = 0; e < 8; ++e) sum = fmaf(xu[e / 4][e % 4], wf[e], sum);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) sum = fmaf(xu[0][e], w[e], sum);
        }
    };
    load_w(0, full_chunks == 0);      // in flight during the NORM prologue
    extra_loads();
    if constexpr (NORM) {
        double sq_sum = 0.0;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            if (i * kThreads < k4) {
                const bool live = threadIdx.x + i * kThreads < k4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float sq = xn[i][j] * xn[i][j];
                    sq_sum += live ? static_cast<double>(sq) : 0.0;
                }
            }
        }
        sq_sum = wave_sum(sq_sum);
        if (lane == 0) partial[wave] = sq_sum;
        __syncthreads();
        sq_sum = 0.0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sq_sum += partial[w];
        const double kd = static_cast<double>(k);
        const float mean = static_cast<float>((k & (k - 1)) == 0 ? sq_sum * (1.0 / kd) : sq_sum / kd);
        const float var = mean + norm.eps;
        const float r = sqrtf(var);
        const float inv = 1.0f / r;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int c = threadIdx.x + i * kThreads;
            if (c < k4) {
                v4f v = xn[i];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float normed = norm.reciprocal ? v[j] * inv : v[j] / r;
                    v[j] = normed * gn[i][j];
                }
                reinterpret_cast<v4f *>(xs)[c] = v;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[c] = 0.f;
    if (!active) return;
    const v4f *xsrc = NORM ? reinterpret_cast<const v4f *>(xs) : xv;
    for (int chunk = 0; chunk < full_chunks; ++chunk) {
        if (chunk > 0) load_w(chunk, false);
        const v4f *px = xsrc + (chunk * kChunkUnits + lane) * kX;
        v4f xr[DEPTH][kX];
#pragma unroll
        for (int j = 0; j < DEPTH; ++j)
#pragma unroll
            for (int h = 0; h < kX; ++h) xr[j][h] = px[j * kWave * kX + h];
#pragma unroll
        for (int j = 0; j < DEPTH; ++j)
#pragma unroll
            for (int c = 0; c < COLS; ++c) unit_fma(xr[j], wr[j][c], acc[c]);
    }
    if (full_chunks * kChunkUnits < kw) {
        if (full_chunks > 0) load_w(full_chunks, true);
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            const int u = full_chunks * kChunkUnits + lane + j * kWave;
            v4f xr[kX];
#pragma unroll
            for (int h = 0; h < kX; ++h) xr[h] = xsrc[min(u, kw - 1) * kX + h];
            if (u >= kw) {
#pragma unroll
                for (int h = 0; h < kX; ++h) xr[h] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < COLS; ++c) wr[j][c] = v4f{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int c = 0; c < COLS; ++c) unit_fma(xr, wr[j][c], acc[c]);
        }
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[c] = wave_sum(acc[c]);
}

// COLS == 2 (rows of 16-bit weights that are one chunk of four units per lane): a wavefront takes
// two rows of Wt, so that it has eight loads per lane in flight like a wavefront over one row of
// floats - two neighbouring outputs, or SWIGLU the gate and the up row of its output, which then
// meet in registers.
template <bool SWIGLU = false, bool NORM = false, int NU = kGemvNormUnits, typename WS = StoredF32,
          int DEPTH = kGemvDepth, int COLS = 1>
__global__ __launch_bounds__(kThreads) void gemv_kmajor_kernel(const float *__restrict__ x,
                                                          const typename WS::elem *__restrict__ wt,
                                                          float *__restrict__ y, int32_t n, int32_t k,
                                                          int64_t ldw, int32_t gate_row, int32_t up_row,
                                                          const float *__restrict__ residual,
                                                          RowNormArgs norm) {
    // A wavefront per row of Wt. SWIGLU: wavefronts 2 p and 2 p + 1 of a block take the gate and
    // the up row of one output and meet in LDS (both rows in one wavefront, sixteen loads per lane
    // in flight, was 22.0 against 20.5 us on 2 x 8192 rows of floats).
    constexpr int kWaves = kThreads / kWave;
    constexpr int kOutputs = SWIGLU ? kWaves * COLS / 2 : kWaves * COLS;    // per block
    [[maybe_unused]] __shared__ float pair_acc[kWaves];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    if constexpr (COLS == 2) {
        const int col = blockIdx.x * kOutputs + (SWIGLU ? wave : 2 * wave);
        // (a wavefront past the last column keeps valid addresses and takes part in the barriers)
        const int col_c = min(col, n - 1);
        const int64_t row0 = SWIGLU ? gate_row + col_c : col_c;
        const int64_t row1 = SWIGLU ? up_row + col_c : min(col + 1, n - 1);
        const v4f *wv[2];
        wv[0] = reinterpret_cast<const v4f *>(wt + row0 * ldw);
        wv[1] = reinterpret_cast<const v4f *>(wt + row1 * ldw);
        float acc[2];
        gemv_wave_dots<2, NORM, NU, WS, DEPTH>(x, wv, k, norm, col < n, acc);
        if (col >= n || lane != 0) return;
        if constexpr (SWIGLU) {
            const float gate = acc[0], up = acc[1];
            const float silu = gate * (1.0f / (1.0f + expf(-gate)));
            y[col] = silu * up;
        } else {
            y[col] = residual ? acc[0] + residual[col] : acc[0];
            if (col + 1 < n) y[col + 1] = residual ? acc[1] + residual[col + 1] : acc[1];
        }
    } else {
        const int col = blockIdx.x * kOutputs + (SWIGLU ? wave / 2 : wave);
        const int col_c = min(col, n - 1);
        const int64_t row = SWIGLU ? ((wave & 1) ? up_row : gate_row) + col_c : col_c;
        const v4f *wv[1];
        wv[0] = reinterpret_cast<const v4f *>(wt + row * ldw);
        float acc[1];
        gemv_wave_dots<1, NORM, NU, WS, DEPTH>(x, wv, k, norm, col < n, acc);
        if constexpr (SWIGLU) {
            if (lane == 0) pair_acc[wave] = acc[0];
            __syncthreads();
            if (col < n && lane == 0 && !(wave & 1)) {
                const float gate = acc[0], up = pair_acc[wave + 1];
                const float silu = gate * (1.0f / (1.0f + expf(-gate)));
                y[col] = silu * up;
            }
        } else {
            if (col < n && lane == 0) y[col] = residual ? acc[0] + residual[col] : acc[0];
        }
    }
}

// The same product with its result handed on as head rows (what rmlk_hip_head_rows does to the
// output of a q/k/v projection) instead of being stored: the columns form up to four streams of
// heads of D columns each, [first_col, first_col + heads * D); two wavefronts compute columns d and
// d + D / 2 of a head, which is the pair a rotation needs; one of them rotates them (cos, sin) or leaves them,
// and writes them to a dense [heads, D] output or to the row of a ScatterND destination that the
// head's index tuple names. The table values and the index tuple are requested before the weights.
constexpr int kGemvMaxStreams = 4;
constexpr int kGemvMaxTuple = 4;
struct GemvRowStream {
    const float *cos, *sin;          // null: the pair is not rotated
    float *out;
    const int64_t *idx;              // null: dense output
    int32_t first_col, heads;
    int32_t first_pair;              // pairs of the streams before this one
    int32_t tuple_size;
    int64_t cs_head, ss_head;        // element strides of cos / sin from one head to the next
    int64_t dim[kGemvMaxTuple], stride[kGemvMaxTuple];   // leading dims of the scatter destination, in rows
};
struct GemvRowStreams {
    GemvRowStream s[kGemvMaxStreams];
    int32_t n_streams, half, total_pairs;
    int32_t *err;
};

template <bool NORM, int NU = kGemvNormUnits, typename WS = StoredF32, int DEPTH = kGemvDepth, int COLS = 1>
__global__ __launch_bounds__(kThreads) void gemv_kmajor_rows_kernel(const float *__restrict__ x,
                                                                    const typename WS::elem *__restrict__ wt,
                                                                    int32_t k,
                                                                    int64_t ldw, RowNormArgs norm,
                                                                    GemvRowStreams rs) {
    // A wavefront per column, like the plain product (two columns per wavefront left the SIMDs with
    // one or two wavefronts each, 8.5 against 6.3 us on the 3072 columns of q, k and v): wavefronts
    // 2 p and 2 p + 1 of a block take columns d and d + D / 2 of a pair and meet in LDS.
    // COLS == 2 (see gemv_kmajor_kernel): one wavefront takes both columns of a pair.
    constexpr int kWaves = kThreads / kWave;
    [[maybe_unused]] __shared__ float pair_acc[kWaves];
    // (the wavefront's number as a scalar: everything derived from it - the stream, the head, the
    // row of the weights - then lives in scalar registers and the stream table is read with scalar loads)
    const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int pair = COLS == 2 ? blockIdx.x * kWaves + wave : blockIdx.x * (kWaves / 2) + wave / 2;
    const int second = COLS == 2 ? 0 : wave & 1;
    const bool active = pair < rs.total_pairs;
    const int pair_c = min(pair, rs.total_pairs - 1);
    int si = 0;
#pragma unroll
    for (int i = 1; i < kGemvMaxStreams; ++i)
        if (i < rs.n_streams && pair_c >= rs.s[i].first_pair) si = i;
    const GemvRowStream &st = rs.s[si];
    const int local = pair_c - st.first_pair;
    const int head = local / rs.half, d = local - head * rs.half;
    const int col = st.first_col + head * (2 * rs.half) + d + second * rs.half;
    const v4f *wv[COLS];
    wv[0] = reinterpret_cast<const v4f *>(wt + static_cast<int64_t>(col) * ldw);
    if constexpr (COLS == 2) wv[1] = reinterpret_cast<const v4f *>(wt + static_cast<int64_t>(col + rs.half) * ldw);
    // what the epilogue needs from memory (in the wavefront that runs it), requested behind the
    // first weights
    float c1 = 1.f, c2 = 1.f, s1 = 0.f, s2 = 0.f;
    int64_t ix[kGemvMaxTuple];
    auto epilogue_loads = [&]() {
        if (second) return;
        if (st.cos) {
            const float *cp = st.cos + head * st.cs_head + d, *sp = st.sin + head * st.ss_head + d;
            c1 = cp[0];
            c2 = cp[rs.half];
            s1 = sp[0];
            s2 = sp[rs.half];
        }
        if (st.idx) {
#pragma unroll
            for (int t = 0; t < kGemvMaxTuple; ++t)
                ix[t] = t < st.tuple_size ? st.idx[static_cast<int64_t>(head) * st.tuple_size + t] : 0;
        }
    };
    float acc[COLS];
    gemv_wave_dots<COLS, NORM, NU, WS, DEPTH>(x, wv, k, norm, active, acc, epilogue_loads);
    float x2;
    if constexpr (COLS == 2) {
        x2 = acc[1];
    } else {
        if (lane == 0) pair_acc[wave] = acc[0];
        __syncthreads();
        x2 = second ? 0.f : pair_acc[wave + 1];
    }
    if (!active || lane != 0 || second) return;
    const float x1 = acc[0];
    float y1 = x1, y2 = x2;
    if (st.cos) {
        // (products and sums rounded one by one, although this file is compiled with contraction
        // allowed: the expressions and roundings of rotary_kernel / head_rows_kernel)
#pragma clang fp contract(off)
        const float a1 = x1 * c1;
        const float r1 = (-x2) * s1;
        y1 = a1 + r1;
        const float a2 = x2 * c2;
        const float r2 = x1 * s2;
        y2 = a2 + r2;
    }
    int64_t out_row = head;
    if (st.idx) {
        out_row = 0;
        bool bad = false;
#pragma unroll
        for (int t = 0; t < kGemvMaxTuple; ++t)
            if (t < st.tuple_size) {
                int64_t i = ix[t];
                if (i < 0) i += st.dim[t];
                if (i < 0 || i >= st.dim[t]) bad = true;
                out_row += i * st.stride[t];
            }
        if (bad) {
            if (rs.err) *rs.err = 1;
            return;
        }
    }
    float *o = st.out + out_row * (2 * rs.half) + d;
    o[0] = y1;
    o[rs.half] = y2;
}

// Any-layout fallback (transposed operands with M > 1): one lane per C element.
__global__ __launch_bounds__(kThreads) void gemm_naive_kernel(const float *__restrict__ a,
                                                              const float *__restrict__ b,
                                                              float *__restrict__ c, int64_t batch,
                                                              int32_t m, int32_t n, int32_t k,
                                                              int64_t a_rs, int64_t a_cs,
                                                              int64_t b_rs, int64_t b_cs,
                                                              int64_t ldc, int64_t stride_a,
                                                              int64_t stride_b, int64_t stride_c) {
    const int64_t per = static_cast<int64_t>(m) * n;
    const int64_t total = batch * per;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        const int64_t bb = i / per, rem = i - bb * per;
        const int64_t r = rem / n, col = rem - r * n;
        const float *pa = a + bb * stride_a + r * a_rs;
        const float *pb = b + bb * stride_b + col * b_cs;
        float s = 0.f;
        for (int kk = 0; kk < k; ++kk) s = fmaf(pa[kk * a_cs], pb[kk * b_rs], s);
        c[bb * stride_c + r * ldc + col] = s;
    }
}

struct TileChoice {
    int bm, bn;     // block tile
    int bk;         // K step
    int splits;     // split-K factor
    int k_per_split;
};

constexpr int kGemmSplitTarget = 1;   // blocks per CU a split-K product aims for

// allow_wide: the 128 x 192 and 128 x 64 tiles may be chosen (they exist for the direct-to-LDS kernel
// only; a caller whose operands do not qualify asks again without it).
inline TileChoice choose_tiles(int64_t batch, int64_t m, int64_t n, int64_t k, bool allow_wide = true) {
    TileChoice t;
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn) * batch; };
    // A 64 x 64 wavefront tile (four MFMA accumulators) keeps the matrix pipe busiest, so the
    // 128 x 128 block (256 x 64 for narrow outputs) is preferred and K is split until the chip is
    // covered; 64 x 64 blocks remain for small problems. Long K uses the deeper K step.
    t.splits = 1;
    if (n <= 64 && tiles(256, 64) >= kNumCU) {
        t.bm = 256;
        t.bn = 64;
    } else if (tiles(128, 128) >= kNumCU) {
        t.bm = 128;
        t.bn = 128;
    } else if (m >= 128 && n >= 128 && k >= 1024 && tiles(128, 128) * 8 >= kNumCU) {
        t.bm = 128;
        t.bn = 128;
    } else {
        t.bm = 64;
        t.bn = 64;
    }
    t.bk = k >= 256 ? 32 : 16;
    auto split_for = [&](int bm, int bn, int *k_per_split) {
        const int64_t nt = tiles(bm, bn);
        int splits = 1;
        if (nt < kNumCU) {
            splits = static_cast<int>((kGemmSplitTarget * kNumCU + nt - 1) / nt);
            int64_t max_splits = k / (8 * t.bk);
            if (max_splits < 1) max_splits = 1;
            if (splits > max_splits) splits = static_cast<int>(max_splits);
            if (splits > 32) splits = 32;
            // a split count that cuts K into equal whole K steps keeps the kernel without bounds checks
            for (int more = splits; more <= 2 * splits && more <= max_splits; ++more)
                if (k % (static_cast<int64_t>(more) * t.bk) == 0) {
                    splits = more;
                    break;
                }
        }
        int64_t kps = (k + splits - 1) / splits;
        kps = (kps + t.bk - 1) / t.bk * t.bk;
        *k_per_split = static_cast<int>(kps);
        splits = static_cast<int>((k + kps - 1) / kps);
        return splits < 1 ? 1 : splits;
    };
    t.splits = split_for(t.bm, t.bn, &t.k_per_split);
    // Widths that are 3 * 2^j (the joint q/k/v width of grouped-query attention) often leave the
    // 128 x 128 tiling with a block count that covers the chip one and a half times; 128 x 192 tiles
    // may cover it in whole rounds. Compare rounds x K steps x tile area (MFMA time) and take the
    // wider tile only when it is clearly ahead.
    if (allow_wide && t.bm == 128 && t.bn == 128 && t.bk == 32 && batch == 1 && n % 192 == 0) {
        int kps_w;
        const int splits_w = split_for(128, 192, &kps_w);
        auto rounds = [&](int64_t blocks) { return (blocks + kNumCU - 1) / kNumCU; };
        const int64_t cost = rounds(tiles(128, 128) * t.splits) * t.k_per_split * 2;
        const int64_t cost_w = rounds(tiles(128, 192) * splits_w) * kps_w * 3;
        if (cost_w * 10 <= cost * 9) {
            t.bn = 192;
            t.splits = splits_w;
            t.k_per_split = kps_w;
            // the same blocks as half-width tiles with half the split: half the partial sums to
            // write and to add up again, twice the K steps per block behind one prologue
            if (splits_w % 2 == 0 && n % 96 == 0 && tiles(128, 96) * (splits_w / 2) <= kNumCU) {
                t.bn = 96;
                t.splits = splits_w / 2;
                t.k_per_split = kps_w * 2;
            }
        }
    }
    // split-K products whose 128 x 128 tiles give one block per CU: 128 x 64 tiles with the same
    // split put two or three blocks on a CU, which overlap each other's first stage and epilogue
    if (allow_wide && t.bm == 128 && t.bn == 128 && t.bk == 32 && t.splits > 1 && n % 64 == 0 &&
        tiles(128, 128) * t.splits <= kNumCU)
        t.bn = 64;
    return t;
}

// the larger split-K factor of the two tilings a product may end up with
inline int max_tile_splits(int64_t batch, int64_t m, int64_t n, int64_t k) {
    const int wide = choose_tiles(batch, m, n, k, true).splits;
    const int narrow = choose_tiles(batch, m, n, k, false).splits;
    return wide > narrow ? wide : narrow;
}

inline int gemv_splits(int64_t batch, int64_t n, int64_t k, int cols_per_block, int *k_per_split) {
    int64_t blocks = (n + cols_per_block - 1) / cols_per_block * batch;
    int64_t splits = 1;
    constexpr int kGemvBlocksPerCu = 6;   // blocks per CU that keep enough loads in flight
    constexpr int kGemvMinRows = 64;      // rows of K a split keeps at least
    if (blocks < kGemvBlocksPerCu * kNumCU)
        splits = (kGemvBlocksPerCu * kNumCU + blocks - 1) / blocks;
    int64_t max_splits = k / kGemvMinRows;
    if (max_splits < 1) max_splits = 1;
    if (splits > max_splits) splits = max_splits;
    if (splits > 64) splits = 64;
    int64_t kps = (k + splits - 1) / splits;
    kps = (kps + 7) / 8 * 8;
    *k_per_split = static_cast<int>(kps);
    return static_cast<int>((k + kps - 1) / kps);
}

template <int BM, int BN, int BK, int WM, int WN, bool EDGE, bool TB = false, typename WS = StoredF32>
int32_t launch_mfma(hipStream_t s, const GemmArgs &g, int64_t batch, int splits) {
    using L = SmemLayout<BM, BN, BK, TB>;
    auto kern = gemm_mfma_kernel<BM, BN, BK, WM, WN, EDGE, TB, WS>;
    if (L::kBytes > 64 * 1024) {
        static DynamicLdsGrant grant;   // one per instantiation, i.e. per kernel
        const int32_t st = grant.ensure(kern, L::kBytes);
        if (st) return st;
    }
    dim3 grid(static_cast<unsigned>(g.tiles_m * g.tiles_n), static_cast<unsigned>(batch),
              static_cast<unsigned>(splits));
    kern<<<grid, kThreads, L::kBytes, s>>>(g);
    return launch_status();
}

template <int BM, int BN, int WM, int WN, bool TB, int STAGES, bool SWIGLU = false, bool EDGE = false,
          typename WS = StoredF32>
int32_t launch_direct(hipStream_t s, const GemmArgs &g, int64_t batch, int splits) {
    constexpr int kBytes = STAGES * (BM * 32 + 32 * BN) * 4;
    auto kern = gemm_mfma_direct_kernel<BM, BN, WM, WN, TB, STAGES, SWIGLU, EDGE, WS>;
    if (kBytes > 64 * 1024) {
        static DynamicLdsGrant grant;   // one per instantiation, i.e. per kernel
        const int32_t st = grant.ensure(kern, kBytes);
        if (st) return st;
    }
    dim3 grid(static_cast<unsigned>(g.tiles_m * g.tiles_n), static_cast<unsigned>(batch),
              static_cast<unsigned>(splits));
    kern<<<grid, kThreads, kBytes, s>>>(g);
    return launch_status();
}

// The tiled MFMA path of a product (m > 1, A not transposed). `seg`: column blocks of C with their
// own destinations (see Segments; their rows must be 16-byte aligned) instead of c/ldc; the call
// then answers RMLK_ERR_UNSUPPORTED unless the whole-tile kernel applies.
// b_dtype: how B is stored (RMLK_FLOAT, or a 16-bit type for a K-contiguous B; ldb and stride_b
// count stored values).
int32_t gemm_tiled(hipStream_t s, int64_t batch, int64_t m, int64_t n, int64_t k, const float *pa,
                   int64_t lda, int64_t stride_a, int32_t b_dtype, const void *pb, int64_t ldb,
                   int64_t stride_b, int32_t trans_b, float *pc, int64_t ldc, int64_t stride_c,
                   void *workspace, size_t workspace_bytes, const Segments *seg,
                   int32_t *partial_splits = nullptr) {
    const bool b16 = b_dtype != RMLK_FLOAT;
    if (b16 && !trans_b) return RMLK_ERR_UNSUPPORTED;
#if RMLK_MATMUL_PART == 1
    if (b16)
        return stored16_gemm_tiled(s, batch, m, n, k, pa, lda, stride_a, b_dtype, pb, ldb, stride_b, trans_b, pc, ldc,
                                   stride_c, workspace, workspace_bytes, seg, partial_splits);
#endif
    // (rows of 16-bit values: whole 128-bit units)
    const int64_t b_unit = b16 ? 8 : 4;
    const bool aligned = lda % 4 == 0 && ldb % b_unit == 0 && stride_a % 4 == 0 && stride_b % b_unit == 0 &&
                         reinterpret_cast<uintptr_t>(pa) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(pb) % 16 == 0;
    // the direct-to-LDS kernel: whole K steps and aligned rows; partial tiles in m and n are fine
    // (for row-major B as long as n is a multiple of 4); per-lane byte offsets are 32-bit
    auto direct_ok = [&](const TileChoice &c) {
        return c.bk == 32 && aligned && c.k_per_split % c.bk == 0 &&
               k % c.k_per_split == 0 && (trans_b || n % 4 == 0) && lda < (1ll << 21) && ldb < (1ll << 21);
    };
    TileChoice t = choose_tiles(batch, m, n, k);
    if ((t.bn == 192 || t.bn == 96 || (t.bm == 128 && t.bn == 64)) && !direct_ok(t)) t = choose_tiles(batch, m, n, k, false);
    GemmArgs g{};
    g.a = pa;
    g.b = static_cast<const float *>(pb);   // (the kernels of a 16-bit B read it as such)
    g.m = static_cast<int32_t>(m);
    g.n = static_cast<int32_t>(n);
    g.k = static_cast<int32_t>(k);
    g.lda = lda;
    g.ldb = ldb;
    g.stride_a = stride_a;
    g.stride_b = stride_b;
    g.k_per_split = t.k_per_split;
    g.tiles_m = static_cast<int32_t>((m + t.bm - 1) / t.bm);
    g.tiles_n = static_cast<int32_t>((n + t.bn - 1) / t.bn);
    if (static_cast<int64_t>(g.tiles_m) * g.tiles_n >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (t.splits > 1 || partial_splits) {
        // split-K slabs [split][batch][m][n]; with `partial_splits` they are the result (the caller's
        // consumer adds them up), even when there is only one
        const size_t need = static_cast<size_t>(t.splits) * batch * m * n * sizeof(float);
        if (!workspace || workspace_bytes < need) return RMLK_ERR_WORKSPACE;
        g.c = static_cast<float *>(workspace);
        g.ldc = n;
        g.stride_c = m * n;
    } else {
        g.c = pc;
        g.ldc = ldc;
        g.stride_c = stride_c;
        if (seg) {
            g.n_seg = seg->n_seg;
            for (int i = 0; i < seg->n_seg; ++i) {
                g.seg_begin[i] = seg->begin[i];
                g.seg_c[i] = seg->c[i];
                g.seg_ldc[i] = seg->ldc[i];
            }
            g.seg_begin[seg->n_seg] = seg->begin[seg->n_seg];
        }
    }
    g.aligned = aligned ? 1 : 0;
    const bool full = aligned && m % t.bm == 0 && n % t.bn == 0 && t.k_per_split % t.bk == 0 &&
                      k % t.k_per_split == 0;
    const bool whole = m % t.bm == 0 && n % t.bn == 0;
    const bool direct = direct_ok(t);
    if (seg) {
        // column blocks with their own destinations: whole tiles only, no tile across a boundary
        if (!direct || batch != 1) return RMLK_ERR_UNSUPPORTED;
        for (int i = 0; i <= seg->n_seg; ++i)
            if (seg->begin[i] % 32 != 0) return RMLK_ERR_UNSUPPORTED;
    }
#define RMLK_LAUNCH_TB(BM_, BN_, WM_, WN_, TB_, WS_)                                              \
    (t.bk == 32                                                                                  \
         ? (full ? launch_mfma<BM_, BN_, 32, WM_, WN_, false, TB_, WS_>(s, g, batch, t.splits)   \
                 : launch_mfma<BM_, BN_, 32, WM_, WN_, true, TB_, WS_>(s, g, batch, t.splits))   \
         : (full ? launch_mfma<BM_, BN_, 16, WM_, WN_, false, TB_, WS_>(s, g, batch, t.splits)   \
                 : launch_mfma<BM_, BN_, 16, WM_, WN_, true, TB_, WS_>(s, g, batch, t.splits)))
#define RMLK_DIRECT_E(BM_, BN_, WM_, WN_, TB_, E_, WS_)                                           \
    launch_direct<BM_, BN_, WM_, WN_, TB_, 2, false, E_, WS_>(s, g, batch, t.splits)
    // two LDS stages: a third (loads two K steps ahead) measured no faster and halves the blocks
    // that fit a CU
#define RMLK_DIRECT(BM_, BN_, WM_, WN_, TB_, WS_)                                                 \
    (whole ? RMLK_DIRECT_E(BM_, BN_, WM_, WN_, TB_, false, WS_) : RMLK_DIRECT_E(BM_, BN_, WM_, WN_, TB_, true, WS_))
    // every tile shape for one layout and storage of B
    auto launch_layout = [&](auto tb_tag, auto ws) -> int32_t {
        constexpr bool TB_ = decltype(tb_tag)::value;
        using WS_ = decltype(ws);
        if (direct && t.bm == 256) return RMLK_DIRECT(256, 64, 64, 64, TB_, WS_);
        if (direct && t.bn == 192) return RMLK_DIRECT(128, 192, 64, 96, TB_, WS_);
        if (direct && t.bn == 96) return RMLK_DIRECT(128, 96, 32, 96, TB_, WS_);
        if (direct && t.bm == 128 && t.bn == 64) return RMLK_DIRECT(128, 64, 64, 32, TB_, WS_);
        if (direct && t.bm == 128) return RMLK_DIRECT(128, 128, 64, 64, TB_, WS_);
        if (direct) return RMLK_DIRECT(64, 64, 32, 32, TB_, WS_);
        if (t.bm == 256) return RMLK_LAUNCH_TB(256, 64, 64, 64, TB_, WS_);
        if (t.bm == 128) return RMLK_LAUNCH_TB(128, 128, 64, 64, TB_, WS_);
        return RMLK_LAUNCH_TB(64, 64, 32, 32, TB_, WS_);
    };
    int32_t st = with_storage_tiled(b_dtype, [&](auto ws) -> int32_t {
        if constexpr (kStored16<decltype(ws)>) return launch_layout(std::true_type{}, ws);
        else return trans_b ? launch_layout(std::true_type{}, ws) : launch_layout(std::false_type{}, ws);
    });
#undef RMLK_DIRECT
#undef RMLK_DIRECT_E
#undef RMLK_LAUNCH_TB
    if (st) return st;
    if (partial_splits) {
        *partial_splits = t.splits;
        return RMLK_OK;
    }
    if (t.splits > 1) {
        Segments one{};
        if (!seg && batch == 1 && n % 4 == 0 && ldc % 4 == 0 &&
            reinterpret_cast<uintptr_t>(pc) % 16 == 0 && reinterpret_cast<uintptr_t>(g.c) % 16 == 0) {
            one.n_seg = 1;
            one.begin[1] = static_cast<int32_t>(n);
            one.c[0] = pc;
            one.ldc[0] = ldc;
            seg = &one;
        }
        if (seg) {
            unsigned rg = grid_for(m * n / 4, kThreads, 8);
            splitk_reduce_vec_kernel<<<rg, kThreads, 0, s>>>(g.c, *seg, t.splits, g.m, g.n);
        } else {
            unsigned rg = grid_for(batch * m * n, kThreads, 8);
            splitk_reduce_kernel<<<rg, kThreads, 0, s>>>(g.c, pc, t.splits, batch, g.m, g.n, ldc,
                                                         stride_c);
        }
        return launch_status();
    }
    return RMLK_OK;
}

// silu(A . B[:, gate..]) * (A . B[:, up..]) in one launch: 128 x 128 tiles of 64 gate and 64 up
// columns. Whole tiles in n and k, no split-K, enough tiles to cover the chip; otherwise UNSUPPORTED.
int32_t gemm_swiglu(hipStream_t s, int64_t m, int64_t n, int64_t k, const float *pa, int64_t lda,
                    int32_t b_dtype, const void *pb, int64_t ldb, int32_t trans_b, int64_t gate_offset,
                    int64_t up_offset, float *pc, int64_t ldc) {
    const bool b16 = b_dtype != RMLK_FLOAT;
    if (b16 && !trans_b) return RMLK_ERR_UNSUPPORTED;
#if RMLK_MATMUL_PART == 1
    if (b16)
        return stored16_gemm_swiglu(s, m, n, k, pa, lda, b_dtype, pb, ldb, trans_b, gate_offset, up_offset, pc, ldc);
#endif
    const bool aligned = lda % 4 == 0 && ldb % (b16 ? 8 : 4) == 0 && gate_offset % 4 == 0 && up_offset % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(pa) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(pb) % 16 == 0;
    if (!aligned || n % 64 != 0 || k % 32 != 0 || k < 32 || lda >= (1ll << 21) || ldb >= (1ll << 21))
        return RMLK_ERR_UNSUPPORTED;
    if (m < 32) return RMLK_ERR_UNSUPPORTED;   // a 128-row tile would be nearly empty
    const int64_t tiles_m = (m + 127) / 128;
    const int64_t tiles = tiles_m * (n / 64);
    if (tiles < kNumCU || tiles >= (1ll << 31)) return RMLK_ERR_UNSUPPORTED;
    GemmArgs g{};
    g.a = pa;
    g.b = static_cast<const float *>(pb);
    g.c = pc;
    g.m = static_cast<int32_t>(m);
    g.n = static_cast<int32_t>(2 * n);
    g.k = static_cast<int32_t>(k);
    g.lda = lda;
    g.ldb = ldb;
    g.ldc = ldc;
    g.k_per_split = g.k;
    g.tiles_m = static_cast<int32_t>(tiles_m);
    g.tiles_n = static_cast<int32_t>(n / 64);
    g.aligned = 1;
    g.gate_offset = static_cast<int32_t>(gate_offset);
    g.up_offset = static_cast<int32_t>(up_offset);
    if (trans_b) {
        // (a lane's byte offset into B covers a row number of the whole matrix here)
        const int64_t last_row = (gate_offset > up_offset ? gate_offset : up_offset) + n;
        if (last_row * ldb >= (1ll << 30)) return RMLK_ERR_UNSUPPORTED;
        return with_storage_tiled(b_dtype, [&](auto ws) -> int32_t {
            using WS = decltype(ws);
            if (m % 128 == 0) return launch_direct<128, 128, 64, 64, true, 2, true, false, WS>(s, g, 1, 1);
            return launch_direct<128, 128, 64, 64, true, 2, true, true, WS>(s, g, 1, 1);
        });
    }
#if RMLK_MATMUL_PART == 1
    if (m % 128 == 0) return launch_direct<128, 128, 64, 64, false, 2, true, false>(s, g, 1, 1);
    return launch_direct<128, 128, 64, 64, false, 2, true, true>(s, g, 1, 1);
#else
    return RMLK_ERR_UNSUPPORTED;
#endif
}

}  // namespace

#if RMLK_MATMUL_PART == 2
int32_t stored16_gemm_tiled(hipStream_t s, int64_t batch, int64_t m, int64_t n, int64_t k, const float *pa,
                            int64_t lda, int64_t stride_a, int32_t b_dtype, const void *pb, int64_t ldb,
                            int64_t stride_b, int32_t trans_b, float *pc, int64_t ldc, int64_t stride_c,
                            void *workspace, size_t workspace_bytes, const void *seg, int32_t *partial_splits) {
    return gemm_tiled(s, batch, m, n, k, pa, lda, stride_a, b_dtype, pb, ldb, stride_b, trans_b, pc, ldc, stride_c,
                      workspace, workspace_bytes, static_cast<const Segments *>(seg), partial_splits);
}
int32_t stored16_gemm_swiglu(hipStream_t s, int64_t m, int64_t n, int64_t k, const float *pa, int64_t lda,
                             int32_t b_dtype, const void *pb, int64_t ldb, int32_t trans_b, int64_t gate_offset,
                             int64_t up_offset, float *pc, int64_t ldc) {
    return gemm_swiglu(s, m, n, k, pa, lda, b_dtype, pb, ldb, trans_b, gate_offset, up_offset, pc, ldc);
}
#endif
}  // namespace rmlk

#if RMLK_MATMUL_PART == 1
using namespace rmlk;

extern "C" size_t rmlk_hip_matmul_workspace_size(int32_t dtype, int64_t batch, int64_t m,
                                                 int64_t n, int64_t k) {
    if (dtype != RMLK_FLOAT || batch <= 0 || m <= 0 || n <= 0 || k <= 0) return 0;
    if (m == 1) {
        // the larger of the two column widths the GEMV may pick
        int kps;
        int s4 = gemv_splits(batch, n, k, kWave * 4, &kps);
        int s1 = gemv_splits(batch, n, k, kWave, &kps);
        int sp = s4 > s1 ? s4 : s1;
        return sp > 1 ? static_cast<size_t>(sp) * batch * n * sizeof(float) : 0;
    }
    const int tile_splits = max_tile_splits(batch, m, n, k);
    size_t need = tile_splits > 1 ? static_cast<size_t>(tile_splits) * batch * m * n * sizeof(float) : 0;
    if (m <= kSkinnyRows) {
        int kps;
        const int sp = gemv_splits(batch, n, k, kWave * 4, &kps);
        const size_t skinny = sp > 1 ? static_cast<size_t>(sp) * batch * m * n * sizeof(float) : 0;
        if (skinny > need) need = skinny;
    }
    return need;
}

extern "C" int32_t rmlk_hip_matmul_describe(int32_t dtype, int64_t batch, int64_t m, int64_t n,
                                            int64_t k, char *buf, int32_t size) {
    char tmp[64];
    if (dtype != RMLK_FLOAT || batch <= 0 || m <= 0 || n <= 0 || k <= 0) {
        snprintf(tmp, sizeof(tmp), "none");
    } else if (m == 1) {
        int kps;
        const bool vec = n % 4 == 0;
        snprintf(tmp, sizeof(tmp), "gemv%s splitk=%d", vec ? "x4" : "x1",
                 gemv_splits(batch, n, k, vec ? kWave * 4 : kWave, &kps));
    } else if (m <= kSkinnyRows && n % 4 == 0) {
        int kps;
        snprintf(tmp, sizeof(tmp), "skinny%d splitk=%d", m <= 2 ? 2 : m <= 4 ? 4 : 8,
                 gemv_splits(batch, n, k, kWave * 4, &kps));
    } else {
        TileChoice t = choose_tiles(batch, m, n, k);
        // dense row-major operands assumed (lda = k, ldb = n): whole K steps take the direct-to-LDS kernel
        auto direct_ok = [&](const TileChoice &c) {
            return c.bk == 32 && k % 4 == 0 && n % 4 == 0 && c.k_per_split % c.bk == 0 &&
                   k % c.k_per_split == 0;
        };
        if ((t.bn == 192 || t.bn == 96 || (t.bm == 128 && t.bn == 64)) && !direct_ok(t)) t = choose_tiles(batch, m, n, k, false);
        const bool direct = direct_ok(t);
        snprintf(tmp, sizeof(tmp), "mfma%dx%dx%d%s splitk=%d", t.bm, t.bn, t.bk,
                 direct ? " direct" : "", t.splits);
    }
    const int32_t len = static_cast<int32_t>(strlen(tmp));
    if (buf && size > 0) {
        strncpy(buf, tmp, size - 1);
        buf[size - 1] = 0;
    }
    return len + 1;
}

namespace {
// float -> 16-bit storage, round to nearest even
template <typename WS>
__device__ __forceinline__ uint16_t round_to_storage(float v) {
    if constexpr (std::is_same<WS, StoredF16>::value) {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
    } else {
        uint32_t u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) u = (u >> 16) | 0x40u;            // NaN stays (quiet) NaN
        else u = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;                        // ties to even
        return static_cast<uint16_t>(u);
    }
}

template <typename WS>
__global__ __launch_bounds__(kThreads) void store_weights_kernel(const float *__restrict__ src,
                                                                 uint16_t *__restrict__ dst, int64_t n) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * kThreads)
        dst[i] = round_to_storage<WS>(src[i]);
}

// *fits = 0 when storing a value would change it (compared as bits: a NaN never fits).
template <typename WS>
__global__ __launch_bounds__(kThreads) void weights_fit_kernel(const float *__restrict__ src, int64_t n,
                                                               int32_t *__restrict__ fits) {
    bool same = true;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
        const float v = src[i];
        same = same && __float_as_uint(WS::widen(round_to_storage<WS>(v))) == __float_as_uint(v) && v == v;
    }
    if (!same) *fits = 0;
}
}  // namespace

extern "C" int32_t rmlk_hip_weights_fit(rmlk_stream_t stream, int32_t w_dtype, int64_t n, const void *src,
                                        int32_t *fits) {
    if (w_dtype != RMLK_FLOAT16 && w_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n == 0) return RMLK_OK;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    if (!src || !fits) return RMLK_ERR_NULL_POINTER;
    const unsigned grid = grid_for(n, kThreads, 8);
    const float *ps = static_cast<const float *>(src);
    if (w_dtype == RMLK_FLOAT16) weights_fit_kernel<StoredF16><<<grid, kThreads, 0, as_stream(stream)>>>(ps, n, fits);
    else weights_fit_kernel<StoredBF16><<<grid, kThreads, 0, as_stream(stream)>>>(ps, n, fits);
    return launch_status();
}

extern "C" int32_t rmlk_hip_store_weights(rmlk_stream_t stream, int32_t w_dtype, int64_t n, const void *src,
                                          void *dst) {
    if (w_dtype != RMLK_FLOAT16 && w_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n == 0) return RMLK_OK;
    if (n >= kMaxElems) return RMLK_ERR_TOO_LARGE;
    if (!src || !dst) return RMLK_ERR_NULL_POINTER;
    const unsigned grid = grid_for(n, kThreads, 8);
    const float *ps = static_cast<const float *>(src);
    uint16_t *pd = static_cast<uint16_t *>(dst);
    if (w_dtype == RMLK_FLOAT16) store_weights_kernel<StoredF16><<<grid, kThreads, 0, as_stream(stream)>>>(ps, pd, n);
    else store_weights_kernel<StoredBF16><<<grid, kThreads, 0, as_stream(stream)>>>(ps, pd, n);
    return launch_status();
}

namespace {
// rmlk_hip_matmul with the storage type of B as an argument: a B of 16-bit values must be
// K-contiguous (trans_b) under a row-major A; ldb and stride_b count stored values.
int32_t matmul_stored(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t m, int64_t n, int64_t k,
                      const void *a, int64_t lda, int64_t stride_a, int32_t trans_a, int32_t b_dtype,
                      const void *b, int64_t ldb, int64_t stride_b, int32_t trans_b, void *c, int64_t ldc,
                      int64_t stride_c, void *workspace, size_t workspace_bytes) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    const bool b16 = b_dtype != RMLK_FLOAT;
    if (b16 && b_dtype != RMLK_FLOAT16 && b_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (b16 && (!trans_b || trans_a)) return RMLK_ERR_UNSUPPORTED;
    if (batch < 0 || m < 0 || n < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (batch == 0 || m == 0 || n == 0) return RMLK_OK;
    if (m >= (1ll << 31) || n >= (1ll << 31) || k >= (1ll << 31) || batch >= 65536)
        return RMLK_ERR_TOO_LARGE;
    if (!c) return RMLK_ERR_NULL_POINTER;
    if (k > 0 && (!a || !b)) return RMLK_ERR_NULL_POINTER;
    const int64_t a_cols = trans_a ? m : k, b_cols = trans_b ? k : n;
    if (lda < a_cols || ldb < b_cols || ldc < n) return RMLK_ERR_SIZE_MISMATCH;
    if (stride_a < 0 || stride_b < 0 || stride_c < 0) return RMLK_ERR_INVALID_ARGUMENT;
    hipStream_t s = as_stream(stream);
    const float *pa = static_cast<const float *>(a);
    const float *pb = static_cast<const float *>(b);   // (a 16-bit B is only handed on, never read here)
    float *pc = static_cast<float *>(c);

    if (k == 0) {
        // empty sum: C = 0
        float zero = 0.f;
        for (int64_t bb = 0; bb < batch; ++bb)
            for (int64_t r = 0; r < m; ++r) {
                int32_t st = rmlk_hip_fill(stream, RMLK_FLOAT, n, &zero,
                                           pc + bb * stride_c + r * ldc);
                if (st) return st;
            }
        return RMLK_OK;
    }

    if (m == 1) {
        GemvArgs g{};
        g.x = pa;
        g.w = pb;
        g.n = static_cast<int32_t>(n);
        g.k = static_cast<int32_t>(k);
        g.x_inc = trans_a ? lda : 1;
        g.ldb = ldb;
        g.stride_x = stride_a;
        g.stride_w = stride_b;
        if (trans_b) {
            g.y = pc;
            g.stride_y = stride_c;
            g.k_per_split = g.k;
            int64_t blocks = (n + 3) / 4;
            if (blocks > 8 * kNumCU) blocks = 8 * kNumCU;
            dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch), 1);
            return with_storage(b_dtype, [&](auto ws) -> int32_t {
                gemv_dot_kernel<decltype(ws)><<<grid, kThreads, 0, s>>>(g);
                return launch_status();
            });
        }
        const bool vec = n % 4 == 0 && ldb % 4 == 0 && stride_b % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(pb) % 16 == 0;
        const int cols = vec ? kWave * 4 : kWave;
        int kps;
        const int splits = gemv_splits(batch, n, k, cols, &kps);
        g.k_per_split = kps;
        if (splits > 1) {
            const size_t need = static_cast<size_t>(splits) * batch * n * sizeof(float);
            if (!workspace || workspace_bytes < need) return RMLK_ERR_WORKSPACE;
            g.y = static_cast<float *>(workspace);
            g.stride_y = n;
        } else {
            g.y = pc;
            g.stride_y = stride_c;
        }
        dim3 grid(static_cast<unsigned>((n + cols - 1) / cols), static_cast<unsigned>(batch),
                  static_cast<unsigned>(splits));
        if (vec) gemv_kernel<4><<<grid, kThreads, 0, s>>>(g);
        else gemv_kernel<1><<<grid, kThreads, 0, s>>>(g);
        int32_t st = launch_status();
        if (st) return st;
        if (splits > 1) {
            const int64_t total = batch * n;
            gemv_reduce_kernel<<<static_cast<unsigned>((total + 31) / 32), kThreads, 0, s>>>(
                static_cast<const float *>(workspace), pc, splits, batch, 1, g.n, ldc, stride_c);
            return launch_status();
        }
        return RMLK_OK;
    }

    if (m <= kSkinnyRows && !trans_a) {
        SkinnyArgs g{};
        g.x = pa;
        g.w = pb;
        g.m = static_cast<int32_t>(m);
        g.n = static_cast<int32_t>(n);
        g.k = static_cast<int32_t>(k);
        g.lda = lda;
        g.ldb = ldb;
        g.stride_x = stride_a;
        g.stride_w = stride_b;
        if (trans_b) {
            g.y = pc;
            g.ldy = ldc;
            g.stride_y = stride_c;
            g.k_per_split = g.k;
            int64_t blocks = (n + 3) / 4;
            if (blocks > 8 * kNumCU) blocks = 8 * kNumCU;
            dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch), 1);
            return with_storage(b_dtype, [&](auto ws) -> int32_t {
                using WS = decltype(ws);
                if (m <= 2) skinny_dot_kernel<2, WS><<<grid, kThreads, 0, s>>>(g);
                else if (m <= 4) skinny_dot_kernel<4, WS><<<grid, kThreads, 0, s>>>(g);
                else skinny_dot_kernel<8, WS><<<grid, kThreads, 0, s>>>(g);
                return launch_status();
            });
        }
        const bool vec = n % 4 == 0 && ldb % 4 == 0 && stride_b % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(pb) % 16 == 0;
        if (vec) {
            int kps;
            const int splits = gemv_splits(batch, n, k, kWave * 4, &kps);
            g.k_per_split = kps;
            if (splits > 1) {
                const size_t need = static_cast<size_t>(splits) * batch * m * n * sizeof(float);
                if (!workspace || workspace_bytes < need) return RMLK_ERR_WORKSPACE;
                g.y = static_cast<float *>(workspace);
                g.ldy = n;
                g.stride_y = m * n;
            } else {
                g.y = pc;
                g.ldy = ldc;
                g.stride_y = stride_c;
            }
            dim3 grid(static_cast<unsigned>((n + kWave * 4 - 1) / (kWave * 4)),
                      static_cast<unsigned>(batch), static_cast<unsigned>(splits));
            if (m <= 2) skinny_kernel<2><<<grid, kThreads, 0, s>>>(g);
            else if (m <= 4) skinny_kernel<4><<<grid, kThreads, 0, s>>>(g);
            else skinny_kernel<8><<<grid, kThreads, 0, s>>>(g);
            int32_t st = launch_status();
            if (st) return st;
            if (splits > 1) {
                const int64_t total = batch * m * n;
                gemv_reduce_kernel<<<static_cast<unsigned>((total + 31) / 32), kThreads, 0, s>>>(
                    static_cast<const float *>(workspace), pc, splits, batch, g.m, g.n, ldc,
                    stride_c);
                return launch_status();
            }
            return RMLK_OK;
        }
        // unaligned B: the MFMA kernel below handles it
    }

    if (trans_a) {
        unsigned grid = grid_for(batch * m * n, kThreads, 16);
        gemm_naive_kernel<<<grid, kThreads, 0, s>>>(
            pa, pb, pc, batch, static_cast<int32_t>(m), static_cast<int32_t>(n),
            static_cast<int32_t>(k), trans_a ? 1 : lda, trans_a ? lda : 1, trans_b ? 1 : ldb,
            trans_b ? ldb : 1, ldc, stride_a, stride_b, stride_c);
        return launch_status();
    }

    return gemm_tiled(s, batch, m, n, k, pa, lda, stride_a, b_dtype, b, ldb, stride_b, trans_b, pc, ldc,
                      stride_c, workspace, workspace_bytes, nullptr);
}
}  // namespace

extern "C" int32_t rmlk_hip_matmul(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t m,
                                   int64_t n, int64_t k, const void *a, int64_t lda,
                                   int64_t stride_a, int32_t trans_a, const void *b, int64_t ldb,
                                   int64_t stride_b, int32_t trans_b, void *c, int64_t ldc,
                                   int64_t stride_c, void *workspace, size_t workspace_bytes) {
    return matmul_stored(stream, dtype, batch, m, n, k, a, lda, stride_a, trans_a, dtype, b, ldb, stride_b,
                         trans_b, c, ldc, stride_c, workspace, workspace_bytes);
}

extern "C" size_t rmlk_hip_gemv_partials_workspace_size(int32_t dtype, int64_t n, int64_t k) {
    if (dtype != RMLK_FLOAT || n <= 0 || k <= 0 || n % 4 != 0) return 0;
    int kps;
    const int splits = gemv_splits(1, n, k, kWave * 4, &kps);
    return static_cast<size_t>(splits) * n * sizeof(float);
}

extern "C" int32_t rmlk_hip_gemv_partials(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                          const void *x, const void *b, int64_t ldb, void *workspace,
                                          size_t workspace_bytes, int32_t *splits_out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n <= 0 || k <= 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= (1ll << 31) || k >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (!x || !b || !workspace || !splits_out) return RMLK_ERR_NULL_POINTER;
    if (ldb < n) return RMLK_ERR_SIZE_MISMATCH;
    if (n % 4 != 0 || ldb % 4 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return RMLK_ERR_UNSUPPORTED;
    int kps;
    const int splits = gemv_splits(1, n, k, kWave * 4, &kps);
    if (workspace_bytes < static_cast<size_t>(splits) * n * sizeof(float)) return RMLK_ERR_WORKSPACE;
    GemvArgs g{};
    g.x = static_cast<const float *>(x);
    g.w = static_cast<const float *>(b);
    g.n = static_cast<int32_t>(n);
    g.k = static_cast<int32_t>(k);
    g.x_inc = 1;
    g.ldb = ldb;
    g.k_per_split = kps;
    g.y = static_cast<float *>(workspace);
    g.stride_y = n;
    dim3 grid(static_cast<unsigned>((n + kWave * 4 - 1) / (kWave * 4)), 1, static_cast<unsigned>(splits));
    gemv_kernel<4><<<grid, kThreads, 0, as_stream(stream)>>>(g);
    *splits_out = splits;
    return launch_status();
}

extern "C" size_t rmlk_hip_matmul_grouped_workspace_size(int32_t dtype, int64_t m, int64_t k,
                                                         int32_t groups, const int64_t *widths) {
    if (dtype != RMLK_FLOAT || !widths || groups <= 0 || groups > kMaxSegments) return 0;
    int64_t total = 0;
    size_t need = 0;
    for (int i = 0; i < groups; ++i) {
        if (widths[i] < 0) return 0;
        total += widths[i];
        const size_t one = rmlk_hip_matmul_workspace_size(dtype, 1, m, widths[i], k);
        if (one > need) need = one;
    }
    const size_t joint = rmlk_hip_matmul_workspace_size(dtype, 1, m, total, k);
    return joint > need ? joint : need;
}

extern "C" int32_t rmlk_hip_matmul_grouped(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t k,
                                           const void *a, int64_t lda, int32_t w_dtype, const void *b,
                                           int64_t ldb, int32_t trans_b, int32_t groups,
                                           const int64_t *widths, void *const *outs, void *workspace,
                                           size_t workspace_bytes) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (w_dtype != RMLK_FLOAT && w_dtype != RMLK_FLOAT16 && w_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (w_dtype != RMLK_FLOAT && !trans_b) return RMLK_ERR_UNSUPPORTED;
    if (!widths || !outs) return RMLK_ERR_NULL_POINTER;
    if (groups <= 0 || groups > kMaxSegments || m < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t total = 0;
    Segments sg{};
    sg.n_seg = groups;
    bool joint = m > kSkinnyRows && k > 0;
    for (int i = 0; i < groups; ++i) {
        if (widths[i] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (widths[i] > 0 && m > 0 && !outs[i]) return RMLK_ERR_NULL_POINTER;
        sg.begin[i] = static_cast<int32_t>(total);
        sg.c[i] = static_cast<float *>(outs[i]);
        sg.ldc[i] = widths[i];
        joint = joint && widths[i] > 0 && widths[i] % 4 == 0 &&
                reinterpret_cast<uintptr_t>(outs[i]) % 16 == 0;
        total += widths[i];
    }
    if (total >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (ldb < (trans_b ? k : total)) return RMLK_ERR_SIZE_MISMATCH;
    sg.begin[groups] = static_cast<int32_t>(total);
    if (m == 0 || total == 0) return RMLK_OK;
    if (!a || !b) return RMLK_ERR_NULL_POINTER;
    if (joint) {
        const size_t need = rmlk_hip_matmul_workspace_size(dtype, 1, m, total, k);
        if (need && (!workspace || workspace_bytes < need)) return RMLK_ERR_WORKSPACE;
        const int32_t st = gemm_tiled(as_stream(stream), 1, m, total, k, static_cast<const float *>(a),
                                      lda, 0, w_dtype, b, ldb, 0, trans_b, sg.c[0], sg.ldc[0], 0, workspace,
                                      workspace_bytes, &sg);
        if (st != RMLK_ERR_UNSUPPORTED) return st;
    }
    int64_t off = 0;
    for (int i = 0; i < groups; ++i) {
        if (widths[i] > 0) {
            // block i: the next widths[i] columns of a row-major B, the next widths[i] rows of a K-contiguous one
            const int64_t first = trans_b ? off * ldb : off;   // in stored values
            const char *bi = static_cast<const char *>(b) + first * (w_dtype == RMLK_FLOAT ? 4 : 2);
            const int32_t st = matmul_stored(stream, dtype, 1, m, widths[i], k, a, lda, 0, 0, w_dtype, bi, ldb,
                                             0, trans_b, outs[i], widths[i], 0, workspace, workspace_bytes);
            if (st) return st;
        }
        off += widths[i];
    }
    return RMLK_OK;
}

extern "C" int32_t rmlk_hip_matmul_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t n,
                                          int64_t k, const void *a, int64_t lda, int32_t w_dtype,
                                          const void *b, int64_t ldb, int32_t trans_b, int64_t gate_offset,
                                          int64_t up_offset, void *out, int64_t ldc) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (w_dtype != RMLK_FLOAT && w_dtype != RMLK_FLOAT16 && w_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (m < 0 || n < 0 || k < 0 || gate_offset < 0 || up_offset < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (m >= (1ll << 31) || n >= (1ll << 30) || k >= (1ll << 31) || gate_offset >= (1ll << 30) ||
        up_offset >= (1ll << 30))
        return RMLK_ERR_TOO_LARGE;
    if (lda < k || ldc < n) return RMLK_ERR_SIZE_MISMATCH;
    if (trans_b ? ldb < k : (ldb < gate_offset + n || ldb < up_offset + n)) return RMLK_ERR_SIZE_MISMATCH;
    if (m == 0 || n == 0) return RMLK_OK;
    if (!a || !b || !out) return RMLK_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(out) % 4 != 0) return RMLK_ERR_UNSUPPORTED;
    return gemm_swiglu(as_stream(stream), m, n, k, static_cast<const float *>(a), lda, w_dtype, b, ldb,
                       trans_b, gate_offset, up_offset, static_cast<float *>(out), ldc);
}

extern "C" size_t rmlk_hip_matmul_partials_workspace_size(int32_t dtype, int64_t m, int64_t n, int64_t k) {
    if (dtype != RMLK_FLOAT || m <= kSkinnyRows || n <= 0 || k <= 0) return 0;
    return static_cast<size_t>(max_tile_splits(1, m, n, k)) * m * n * sizeof(float);
}

extern "C" int32_t rmlk_hip_matmul_partials(rmlk_stream_t stream, int32_t dtype, int64_t m, int64_t n,
                                            int64_t k, const void *a, int64_t lda, int32_t w_dtype,
                                            const void *b, int64_t ldb, int32_t trans_b, void *workspace,
                                            size_t workspace_bytes, int32_t *splits_out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (w_dtype != RMLK_FLOAT && w_dtype != RMLK_FLOAT16 && w_dtype != RMLK_BFLOAT16) return RMLK_ERR_UNSUPPORTED;
    if (m < 0 || n < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (m >= (1ll << 31) || n >= (1ll << 31) || k >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (m <= kSkinnyRows || n == 0 || k == 0) return RMLK_ERR_UNSUPPORTED;   // not the tiled kernels' case
    if (!a || !b || !workspace || !splits_out) return RMLK_ERR_NULL_POINTER;
    if (lda < k || ldb < (trans_b ? k : n)) return RMLK_ERR_SIZE_MISMATCH;
    if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
    return gemm_tiled(as_stream(stream), 1, m, n, k, static_cast<const float *>(a), lda, 0, w_dtype, b, ldb,
                      0, trans_b, nullptr, n, 0, workspace, workspace_bytes, nullptr, splits_out);
}

namespace {

// Shared argument checks and launches of the K-major one-row products. `norm`: x is normalised on
// the fly (see gemv_kmajor_kernel); `residual`: added to the outputs.
// What every K-major one-row product checks of its weights: rows of whole 128-bit units that
// start on 16-byte boundaries.
template <typename WS>
bool kmajor_rows_ok(int64_t k, const void *wt, int64_t ldw) {
    return k % WS::kUnit == 0 && ldw % WS::kUnit == 0 && reinterpret_cast<uintptr_t>(wt) % 16 == 0;
}

// f(storage tag, units per lane and chunk, rows per wavefront) for a row of k weights stored as
// `w_dtype`: short rows of 16-bit weights are walked four units at a time, two rows per wavefront.
template <typename F>
int32_t with_storage_depth(int32_t w_dtype, int64_t k, F &&f) {
    return with_storage(w_dtype, [&](auto ws) -> int32_t {
        using WS = decltype(ws);
        if constexpr (kStored16<WS>) {
            if (k < 64 * 8 * WS::kUnit)
                return f(ws, std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
        }
        return f(ws, std::integral_constant<int, kGemvDepth>{}, std::integral_constant<int, 1>{});
    });
}

int32_t gemv_kmajor_launch(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k, const void *x,
                           int32_t w_dtype, const void *wt, int64_t ldw, const void *residual,
                           const RowNormArgs *norm, void *y) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= (1ll << 31) || k >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (n == 0) return RMLK_OK;
    if (!y || (k > 0 && (!x || !wt)) || (norm && !norm->gamma)) return RMLK_ERR_NULL_POINTER;
    if (ldw < k) return RMLK_ERR_SIZE_MISMATCH;
    if (k % 4 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
    // the widths the norm kernel gives one block
    if (norm && (k == 0 || k > kThreads * 4 * 8 || reinterpret_cast<uintptr_t>(norm->gamma) % 16 != 0))
        return RMLK_ERR_UNSUPPORTED;
    const float *px = static_cast<const float *>(x);
    const float *pr = static_cast<const float *>(residual);
    float *py = static_cast<float *>(y);
    hipStream_t s = as_stream(stream);
    constexpr int kWaves = kThreads / kWave;
    const int32_t ni = static_cast<int32_t>(n), ki = static_cast<int32_t>(k);
    return with_storage_depth(w_dtype, k, [&](auto ws, auto depth, auto cols) -> int32_t {
        using WS = decltype(ws);
        constexpr int D = decltype(depth)::value, C = decltype(cols)::value;
        if (!kmajor_rows_ok<WS>(k, wt, ldw)) return RMLK_ERR_UNSUPPORTED;
        const typename WS::elem *pw = static_cast<const typename WS::elem *>(wt);
        const unsigned grid = static_cast<unsigned>((n + kWaves * C - 1) / (kWaves * C));
        if (norm && k <= kThreads * 4 * 2)
            gemv_kmajor_kernel<false, true, 2, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(px, pw, py, ni, ki, ldw, 0, 0, pr, *norm);
        else if (norm)
            gemv_kmajor_kernel<false, true, kGemvNormUnits, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(px, pw, py, ni, ki, ldw, 0, 0, pr, *norm);
        else
            gemv_kmajor_kernel<false, false, kGemvNormUnits, WS, D, C><<<grid, kThreads, 0, s>>>(px, pw, py, ni, ki, ldw, 0, 0, pr, RowNormArgs{});
        return launch_status();
    });
}

int32_t gemv_kmajor_swiglu_launch(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k, const void *x,
                                  int32_t w_dtype, const void *wt, int64_t ldw, int64_t gate_row,
                                  int64_t up_row, const RowNormArgs *norm, void *y) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n < 0 || k < 0 || gate_row < 0 || up_row < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n >= (1ll << 30) || k >= (1ll << 31) || gate_row >= (1ll << 30) || up_row >= (1ll << 30))
        return RMLK_ERR_TOO_LARGE;
    if (n == 0) return RMLK_OK;
    if (!y || (k > 0 && (!x || !wt)) || (norm && !norm->gamma)) return RMLK_ERR_NULL_POINTER;
    if (ldw < k) return RMLK_ERR_SIZE_MISMATCH;
    if (k % 4 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
    if (norm && (k == 0 || k > kThreads * 4 * 8 || reinterpret_cast<uintptr_t>(norm->gamma) % 16 != 0))
        return RMLK_ERR_UNSUPPORTED;
    constexpr int kOutputsPerBlock = kThreads / kWave / 2;   // a wavefront per gate row and per up row
    const float *px = static_cast<const float *>(x);
    float *py = static_cast<float *>(y);
    const int32_t ni = static_cast<int32_t>(n), ki = static_cast<int32_t>(k);
    const int32_t gr = static_cast<int32_t>(gate_row), ur = static_cast<int32_t>(up_row);
    hipStream_t s = as_stream(stream);
    return with_storage_depth(w_dtype, k, [&](auto ws, auto depth, auto cols) -> int32_t {
        using WS = decltype(ws);
        constexpr int D = decltype(depth)::value, C = decltype(cols)::value;
        if (!kmajor_rows_ok<WS>(k, wt, ldw)) return RMLK_ERR_UNSUPPORTED;
        const typename WS::elem *pw = static_cast<const typename WS::elem *>(wt);
        // (two rows per wavefront: the gate and the up row of one output)
        const unsigned grid = static_cast<unsigned>((n + kOutputsPerBlock * C - 1) / (kOutputsPerBlock * C));
        if (norm && k <= kThreads * 4 * 2)
            gemv_kmajor_kernel<true, true, 2, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(
                px, pw, py, ni, ki, ldw, gr, ur, nullptr, *norm);
        else if (norm)
            gemv_kmajor_kernel<true, true, kGemvNormUnits, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(
                px, pw, py, ni, ki, ldw, gr, ur, nullptr, *norm);
        else
            gemv_kmajor_kernel<true, false, kGemvNormUnits, WS, D, C><<<grid, kThreads, 0, s>>>(
                px, pw, py, ni, ki, ldw, gr, ur, nullptr, RowNormArgs{});
        return launch_status();
    });
}

}  // namespace

extern "C" int32_t rmlk_hip_gemv_kmajor_head_rows(rmlk_stream_t stream, int32_t dtype, int64_t k,
                                                  const void *x, const void *gamma, float eps,
                                                  int32_t reciprocal_form, int32_t w_dtype, const void *wt,
                                                  int64_t ldw, int32_t n_streams,
                                                  const rmlk_row_stream *streams, const int64_t *first_col,
                                                  int32_t *err_flag) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n_streams < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n_streams == 0) return RMLK_OK;
    if (n_streams > kGemvMaxStreams) return RMLK_ERR_UNSUPPORTED;
    if (!streams || !first_col || (k > 0 && (!x || !wt))) return RMLK_ERR_NULL_POINTER;
    if (k >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    if (ldw < k) return RMLK_ERR_SIZE_MISMATCH;
    if (k == 0 || k % 4 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
    if (gamma && (k > kThreads * 4 * kGemvNormUnits || reinterpret_cast<uintptr_t>(gamma) % 16 != 0))
        return RMLK_ERR_UNSUPPORTED;
    GemvRowStreams rs{};
    rs.err = err_flag;
    int64_t d_common = -1, pairs = 0;
    for (int i = 0; i < n_streams; ++i) {
        const rmlk_row_stream &in = streams[i];
        const bool rotate = in.cos || in.sin;
        if (!dims_ok(&in.shape) || in.shape.rank != 4) return RMLK_ERR_BAD_RANK;
        if (rotate && (!dims_ok(&in.cos_stride) || !dims_ok(&in.sin_stride) || in.cos_stride.rank != 4 ||
                       in.sin_stride.rank != 4))
            return RMLK_ERR_BAD_RANK;
        if (dims_numel(&in.shape) <= 0) return RMLK_ERR_INVALID_ARGUMENT;
        // one row of the product: one token of one sequence
        if (in.shape.v[0] != 1 || in.shape.v[2] != 1) return RMLK_ERR_UNSUPPORTED;
        const int64_t heads = in.shape.v[1], d = in.shape.v[3];
        if (d % 2 != 0 || (d_common >= 0 && d != d_common)) return RMLK_ERR_UNSUPPORTED;
        d_common = d;
        if (!in.out || (rotate && (!in.cos || !in.sin))) return RMLK_ERR_NULL_POINTER;
        if (rotate && (in.cos_stride.v[3] != 1 || in.sin_stride.v[3] != 1 || in.cos_stride.v[1] < 0 ||
                       in.sin_stride.v[1] < 0))
            return RMLK_ERR_UNSUPPORTED;
        if (first_col[i] < 0 || first_col[i] + heads * d >= (1ll << 31)) return RMLK_ERR_INVALID_ARGUMENT;
        GemvRowStream &a = rs.s[i];
        a.cos = rotate ? static_cast<const float *>(in.cos) : nullptr;
        a.sin = rotate ? static_cast<const float *>(in.sin) : nullptr;
        a.out = static_cast<float *>(in.out);
        a.idx = in.idx;
        a.first_col = static_cast<int32_t>(first_col[i]);
        a.heads = static_cast<int32_t>(heads);
        a.first_pair = static_cast<int32_t>(pairs);
        a.cs_head = rotate ? in.cos_stride.v[1] : 0;
        a.ss_head = rotate ? in.sin_stride.v[1] : 0;
        a.tuple_size = 0;
        if (in.idx) {
            if (!dims_ok(&in.data_shape)) return RMLK_ERR_BAD_RANK;
            if (in.tuple_size < 1 || in.tuple_size != in.data_shape.rank - 1) return RMLK_ERR_INVALID_ARGUMENT;
            if (in.tuple_size > kGemvMaxTuple) return RMLK_ERR_UNSUPPORTED;
            if (in.data_shape.v[in.tuple_size] != d || dims_numel(&in.data_shape) < 0)
                return RMLK_ERR_INVALID_ARGUMENT;
            if (dims_numel(&in.data_shape) >= ((int64_t)1 << 40)) return RMLK_ERR_TOO_LARGE;
            a.tuple_size = in.tuple_size;
            int64_t stride = 1;
            for (int t = a.tuple_size - 1; t >= 0; --t) {
                a.dim[t] = in.data_shape.v[t];
                a.stride[t] = stride;
                stride *= in.data_shape.v[t];
            }
        }
        pairs += heads * (d / 2);
        if (pairs >= (1ll << 30)) return RMLK_ERR_TOO_LARGE;
    }
    rs.n_streams = n_streams;
    rs.half = static_cast<int32_t>(d_common / 2);
    rs.total_pairs = static_cast<int32_t>(pairs);
    constexpr int kPairsPerBlock = kThreads / kWave / 2;
    const float *px = static_cast<const float *>(x);
    const int32_t ki = static_cast<int32_t>(k);
    hipStream_t s = as_stream(stream);
    return with_storage_depth(w_dtype, k, [&](auto ws, auto depth, auto cols) -> int32_t {
        using WS = decltype(ws);
        constexpr int D = decltype(depth)::value, C = decltype(cols)::value;
        if (!kmajor_rows_ok<WS>(k, wt, ldw)) return RMLK_ERR_UNSUPPORTED;
        const typename WS::elem *pw = static_cast<const typename WS::elem *>(wt);
        const unsigned grid = static_cast<unsigned>((pairs + kPairsPerBlock * C - 1) / (kPairsPerBlock * C));
        if (gamma) {
            const RowNormArgs norm{static_cast<const float *>(gamma), eps, reciprocal_form};
            if (k <= kThreads * 4 * 2)
                gemv_kmajor_rows_kernel<true, 2, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(px, pw, ki, ldw, norm, rs);
            else
                gemv_kmajor_rows_kernel<true, kGemvNormUnits, WS, D, C><<<grid, kThreads, k * sizeof(float), s>>>(px, pw, ki, ldw, norm, rs);
        } else {
            gemv_kmajor_rows_kernel<false, kGemvNormUnits, WS, D, C><<<grid, kThreads, 0, s>>>(px, pw, ki, ldw, RowNormArgs{}, rs);
        }
        return launch_status();
    });
}

extern "C" int32_t rmlk_hip_gemv_kmajor(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                   const void *x, int32_t w_dtype, const void *wt, int64_t ldw, void *y) {
    return gemv_kmajor_launch(stream, dtype, n, k, x, w_dtype, wt, ldw, nullptr, nullptr, y);
}

extern "C" int32_t rmlk_hip_gemv_kmajor_add(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                            const void *x, int32_t w_dtype, const void *wt, int64_t ldw,
                                            const void *residual, void *y) {
    if (n > 0 && !residual) return RMLK_ERR_NULL_POINTER;
    return gemv_kmajor_launch(stream, dtype, n, k, x, w_dtype, wt, ldw, residual, nullptr, y);
}

extern "C" int32_t rmlk_hip_gemv_kmajor_normed(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                               const void *x, const void *gamma, float eps,
                                               int32_t reciprocal_form, int32_t w_dtype, const void *wt,
                                               int64_t ldw, void *y) {
    const RowNormArgs norm{static_cast<const float *>(gamma), eps, reciprocal_form};
    if (n > 0 && !gamma) return RMLK_ERR_NULL_POINTER;
    return gemv_kmajor_launch(stream, dtype, n, k, x, w_dtype, wt, ldw, nullptr, &norm, y);
}

extern "C" int32_t rmlk_hip_gemv_kmajor_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n, int64_t k,
                                          const void *x, int32_t w_dtype, const void *wt, int64_t ldw,
                                          int64_t gate_row, int64_t up_row, void *y) {
    return gemv_kmajor_swiglu_launch(stream, dtype, n, k, x, w_dtype, wt, ldw, gate_row, up_row, nullptr, y);
}

extern "C" int32_t rmlk_hip_gemv_kmajor_swiglu_normed(rmlk_stream_t stream, int32_t dtype, int64_t n,
                                                      int64_t k, const void *x, const void *gamma,
                                                      float eps, int32_t reciprocal_form, int32_t w_dtype,
                                                      const void *wt, int64_t ldw, int64_t gate_row,
                                                      int64_t up_row, void *y) {
    const RowNormArgs norm{static_cast<const float *>(gamma), eps, reciprocal_form};
    if (n > 0 && !gamma) return RMLK_ERR_NULL_POINTER;
    return gemv_kmajor_swiglu_launch(stream, dtype, n, k, x, w_dtype, wt, ldw, gate_row, up_row, &norm, y);
}

// ---- MatMul for callers that cannot allocate ----------------------------------------------------
// The split-K partials of rmlk_hip_matmul live in a workspace the caller allocates. A caller under
// HIP graph capture, in a tight serving loop or in a harness that forbids hipMalloc cannot do that:
// for them the partials go to a fixed array in device memory that is part of the code object. Every
// GPU the library runs on holds its own copy of the array, at its own address, until the process ends.
static __device__ __align__(256) unsigned char scratch[RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES];

namespace {
// Device address of `scratch` per GPU, looked up on the entry point's first call on that GPU (the
// array's name is a host-side stand-in in host code, not an address a kernel can use).
constexpr int kScratchDevices = 64;
std::atomic<void *> g_scratch_ptr[kScratchDevices];

int32_t scratch_for_current_device(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int32_t>(e);
    if (dev < 0 || dev >= kScratchDevices) return RMLK_ERR_INVALID_ARGUMENT;
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // threads that race here all get the same answer for this device
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int32_t>(e);
        if (!p) return RMLK_ERR_NULL_POINTER;
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return RMLK_OK;
}
}  // namespace

extern "C" int32_t rmlk_hip_matmul_noalloc(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t m,
                                           int64_t n, int64_t k, const void *a, int64_t lda,
                                           int64_t stride_a, int32_t trans_a, const void *b, int64_t ldb,
                                           int64_t stride_b, int32_t trans_b, void *c, int64_t ldc,
                                           int64_t stride_c) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (batch < 0 || m < 0 || n < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    const size_t need = rmlk_hip_matmul_workspace_size(dtype, batch, m, n, k);
    if (need > static_cast<size_t>(RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES)) return RMLK_ERR_SCRATCH_LIMIT;
    void *ws = nullptr;
    if (need) {
        // the partials are written before they are read: nothing in the array has to start at zero
        const int32_t st = scratch_for_current_device(&ws);
        if (st) return st;
    }
    return rmlk_hip_matmul(stream, dtype, batch, m, n, k, a, lda, stride_a, trans_a, b, ldb, stride_b,
                           trans_b, c, ldc, stride_c, ws, need);
}
#endif   // RMLK_MATMUL_PART == 1
