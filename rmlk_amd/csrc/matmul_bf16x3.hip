// Many-row products over weights stored as bfloat16 values, on the bf16 matrix cores, with fp32
// results: C[m][n] = A[m][k] . W[n][k]^T, A fp32, W bfloat16 (K-contiguous).
//
// A float has 24 significant bits, a bfloat16 eight: a = hi + mid + lo holds EXACTLY with three
// bfloat16 pieces (hi = a truncated to 8 bits, mid = (a - hi) truncated, lo = the rest). A product of
// two bfloat16 values is exact in fp32 (16 significant bits), so
//     sum_k a[k] * w[k]  =  sum_k hi[k] * w[k] + mid[k] * w[k] + lo[k] * w[k]
// with every product exact and only the fp32 accumulation rounding - the error of an fp32 product
// with its sums in another order. Three v_mfma_f32_32x32x16_bf16 do per K chunk of 16 what eight
// v_mfma_f32_32x32x2_f32 do, in 96 cycles instead of 512.
//
// Two launches: rmlk_hip_bf16x3_split writes the three pieces of A as planes [3][m_pad][k] (m_pad =
// m rounded up to whole 128-row tiles, the padding rows zero) - once per A, however many column
// tiles read it afterwards; the product kernel streams K steps of 32 of the three planes' tile rows
// and of W's tile rows straight from global memory into LDS (global_load_lds_dwordx4) through two to
// four stages, and every wavefront multiplies a 64 x (32 * TN) tile: per K chunk TN fragments of W
// against 3 x 2 fragments of A, 6 * TN MFMAs. Kernels that produce an operand of such a product can
// store its pieces themselves and save the split launch: the RMSNorm kernels (reduce.hip), the
// attention kernel (attention.hip) and the SwiGLU epilogue below do.
//
// No counterpart in the reference (its products are fp32 cuBLAS calls, cuda/src/kernels/gemm.rs:191-232).
#include "common.hpp"

namespace rmlk {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 v8bf;
typedef __attribute__((ext_vector_type(16))) float v16f;
typedef __attribute__((ext_vector_type(4))) uint32_t v4u;
typedef __attribute__((ext_vector_type(4))) float v4f;

constexpr int kThreads = 256;
constexpr int kTileRows = 128;   // rows of A per block tile
constexpr int kMaxGroups = 4;    // members of a grouped product

inline int64_t padded_rows(int64_t m) { return (m + kTileRows - 1) / kTileRows * kTileRows; }

// planes[p][row][k], p = 0 (hi), 1 (mid), 2 (lo); rows m .. m_pad-1 are zero. One 128-bit unit of
// eight values per plane and lane. Infinities and NaNs stay in hi alone (inf - inf would poison
// the other two).
__global__ __launch_bounds__(kThreads) void split_bf16x3_kernel(const float *__restrict__ a, int64_t lda,
                                                                 int32_t m, int32_t k, int32_t m_pad,
                                                                 uint16_t *__restrict__ planes) {
    const int units_per_row = k / 8;
    const int64_t total = static_cast<int64_t>(m_pad) * units_per_row;
    const int64_t plane = static_cast<int64_t>(m_pad) * k;
    for (int64_t id = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; id < total;
         id += static_cast<int64_t>(gridDim.x) * kThreads) {
        const int row = static_cast<int>(id / units_per_row), u = static_cast<int>(id % units_per_row);
        uint32_t hi[8], mid[8], lo[8];
        if (row < m) {
            const v4f x0 = *reinterpret_cast<const v4f *>(a + row * lda + u * 8);
            const v4f x1 = *reinterpret_cast<const v4f *>(a + row * lda + u * 8 + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float x = e < 4 ? x0[e] : x1[e - 4];
                const uint32_t xb = __float_as_uint(x);
                const uint32_t hb = xb & 0xffff0000u;
                const bool finite = (xb & 0x7f800000u) != 0x7f800000u;
                const float r1 = finite ? x - __uint_as_float(hb) : 0.f;       // exact: <= 16 bits
                const uint32_t mb = __float_as_uint(r1) & 0xffff0000u;
                const float r2 = r1 - __uint_as_float(mb);                     // exact: <= 8 bits
                hi[e] = hb >> 16;
                mid[e] = mb >> 16;
                lo[e] = __float_as_uint(r2) >> 16;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) hi[e] = mid[e] = lo[e] = 0;
        }
        auto pack = [](const uint32_t *v) {
            return v4u{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
        };
        const int64_t at = static_cast<int64_t>(row) * k + u * 8;
        *reinterpret_cast<v4u *>(planes + at) = pack(hi);
        *reinterpret_cast<v4u *>(planes + plane + at) = pack(mid);
        *reinterpret_cast<v4u *>(planes + 2 * plane + at) = pack(lo);
    }
}

struct X3Args {
    const uint16_t *a3;   // [3][m_pad][k]
    const uint16_t *b;    // [rows][ldb], K-contiguous
    float *c;             // [split][m][ldc]
    int32_t m, n, k, m_pad;
    int64_t ldb, ldc, slab;
    int32_t k_per_split, tiles_m, tiles_n, per_xcd;
    int64_t gate_row, up_row;   // SWIGLU: the rows of b that hold the gate and the up weights
    // Destinations per block of columns (n_seg > 0, one slab): columns [seg_begin[i], seg_begin[i+1])
    // go to seg_c[i] (leading dimension seg_ldc[i], column 0 = seg_begin[i]); boundaries are
    // multiples of 32, so a 32-column accumulator block has one destination.
    // SWIGLU: the result also as three bfloat16 pieces (planes of `act_plane` elements, rows of n), for
    // a product that reads it; null: not wanted
    uint16_t *act_pieces;
    int64_t act_plane;
    int32_t n_seg;
    int32_t seg_begin[kMaxGroups + 1];
    float *seg_c[kMaxGroups];
    int64_t seg_ldc[kMaxGroups];
};

// Block tile 128 x (64 * TN), four wavefronts (2 x 2) of 64 x (32 * TN). LDS rows are 64 bytes (32
// bfloat16, four 16-byte units), unpadded - a direct load writes 64 lanes x 16 bytes as one
// contiguous KiB - and unit u of row r lives at position u ^ ((r >> 2) & 3) of its row, applied on
// the global side when a unit is fetched (each lane of a direct load picks its own source) and again
// when it is read back: the sixteen lanes that a 128-bit fragment read serves together (sixteen
// consecutive rows, one unit each) then cover all 64 banks once.
//
// The stage for K step s + STAGES - 1 is requested during step s, into the LDS stage that was read
// in step s - 1; a wavefront's loads complete in order, so "all but the loads of the STAGES - 2
// newest stages have landed" (vmcnt) says that the next stage is there. One block-wide barrier per K
// step, a quarter into its second chunk: before it every wavefront has read the step's second chunk
// into registers, after it the first chunk of the next step is read. The matrix pipe takes a new
// MFMA every 32 cycles and a wavefront issues in order, so the LDS reads and the direct loads are
// dealt out between the MFMAs one at a time (loads and reads alternating) instead of in bursts.
//
// SWIGLU: the tile's rows of W are half gate rows, half up rows, arranged so that a wavefront's
// accumulator columns j and j + TN / 2 hold the gate and the up value of the same output column; the
// epilogue stores silu(gate) * up, 32 * TN output columns per block.
template <int TN, int STAGES, bool SWIGLU>
__global__ __launch_bounds__(kThreads) void gemm_bf16x3_kernel(X3Args g) {
    constexpr int TM = 2;
    constexpr int BM = kTileRows, BN = 64 * TN, WN = 32 * TN, BK = 32;
    constexpr int kPlane = BM * BK * 2;            // bytes of one plane's tile in a stage
    constexpr int kAStage = 3 * kPlane;
    constexpr int kBStage = BN * BK * 2;
    constexpr int kStage = kAStage + kBStage;
    constexpr int A_LOADS = 3 * BM / 16 / 4;       // 1 KiB pieces (16 rows) per wavefront and stage
    constexpr int B_LOADS = BN / 16 / 4;
    constexpr int kLoads = A_LOADS + B_LOADS;
    static_assert(!SWIGLU || TN % 2 == 0, "gate and up columns in pairs");
    extern __shared__ __align__(16) unsigned char smem[];

    // Consecutive tiles share their rows of W (they differ in tile_m) and run next to each other on
    // one XCD (workgroups go to the XCDs round-robin), whose L2 then fetches those rows once.
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int t = xcd * g.per_xcd + slot;
    if (t >= g.tiles_m * g.tiles_n) return;        // (the whole block: no barrier is left waiting)
    const int tile_m = t % g.tiles_m, tile_n = t / g.tiles_m;
    const int split = blockIdx.y;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int k_begin = split * g.k_per_split;
    const int n_steps = (min(g.k, k_begin + g.k_per_split) - k_begin) / BK;

    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int wm = wave / 2, wn = wave % 2;
    const int l32 = lane % 32, half = lane / 32;

    // Sources. Lane l of a piece fills LDS unit l of the piece: row l / 4, position l % 4.
    const int src_row = lane / 4, src_unit = (lane % 4) ^ ((lane / 16) & 3);
    uint32_t a_voff[A_LOADS], b_voff[B_LOADS];
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
        const int q = wave + 4 * j;                // piece: plane q / 8, rows (q % 8) * 16 ..
        const int64_t row = static_cast<int64_t>(q / 8) * g.m_pad + (q % 8) * 16 + src_row;
        a_voff[j] = static_cast<uint32_t>((row * g.k + src_unit * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
        const int q = wave + 4 * j;
        int64_t row = q * 16 + src_row;            // row of the tile in LDS
        if constexpr (SWIGLU) {
            // LDS row r: wavefront column r / WN, accumulator (r % WN) / 32, lane r % 32
            const int64_t col = tile_n * (BN / 2) + (row / WN) * (WN / 2) + ((row % WN) / 32 % (TN / 2)) * 32 + row % 32;
            row = ((row % WN) / 32 < TN / 2 ? g.gate_row : g.up_row) + col;
        }
        b_voff[j] = static_cast<uint32_t>((row * g.ldb + src_unit * 8) * 2);
    }
    const uint16_t *a_ptr = g.a3 + static_cast<int64_t>(m0) * g.k + k_begin;
    const uint16_t *b_ptr = g.b + (SWIGLU ? 0 : static_cast<int64_t>(n0) * g.ldb) + k_begin;
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem)) + wave * 1024u);

    auto direct_load = [&](uint32_t lds_addr, const uint16_t *base, uint32_t voff) {
        // (one wait state between a scalar write of M0 and the LDS-bound load that reads it)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(base)
                     : "memory", "m0");
    };
    auto load_stage = [&](int buf) {
        const uint32_t base = lds0 + static_cast<uint32_t>(buf * kStage);
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) direct_load(base + j * 4096, a_ptr, a_voff[j]);
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) direct_load(base + kAStage + j * 4096, b_ptr, b_voff[j]);
        a_ptr += BK;
        b_ptr += BK;
    };
    auto load_op = [&](int buf, auto o_tag) {
        constexpr int o = decltype(o_tag)::value;
        const uint32_t base = lds0 + static_cast<uint32_t>(buf * kStage);
        if constexpr (o < A_LOADS) direct_load(base + o * 4096, a_ptr, a_voff[o]);
        else direct_load(base + kAStage + (o - A_LOADS) * 4096, b_ptr, b_voff[o - A_LOADS]);
    };

    // Fragments: for K chunk c lane (l32, half) reads unit c * 2 + half of its row - eight
    // consecutive K values, the same eight for A and W.
    int frag_off[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) frag_off[c] = l32 * 64 + ((c * 2 + half) ^ ((l32 / 4) & 3)) * 16;
    const int a_base = wm * 64 * 64, b_base = kAStage + wn * WN * 64;
    v4u af[2][3][TM], bfr[2][TN];
    // read number o of a chunk, in the order the MFMAs want them: W's column blocks, then the lo,
    // the mid and the hi piece of A's row blocks
    constexpr int kFragOps = TN + 3 * TM;
    auto frag_op = [&](int buf, int c, auto s_tag, auto o_tag) {
        constexpr int s = decltype(s_tag)::value, o = decltype(o_tag)::value;
        const unsigned char *st = smem + buf * kStage;
        if constexpr (o < TN) {
            bfr[s][o] = *reinterpret_cast<const v4u *>(st + b_base + o * 2048 + frag_off[c]);
        } else {
            constexpr int q = o - TN, p = 2 - q / TM, i = q % TM;
            af[s][p][i] = *reinterpret_cast<const v4u *>(st + p * kPlane + a_base + i * 2048 + frag_off[c]);
        }
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // MFMA number q of a chunk: pieces outermost (TM * TN independent accumulators between two MFMAs
    // on the same one), the small pieces first
    constexpr int NM = 3 * TM * TN;
    auto mfma_at = [&](auto s_tag, auto q_tag) {
        constexpr int s = decltype(s_tag)::value, q = decltype(q_tag)::value;
        constexpr int p = 2 - q / (TM * TN), i = (q / TN) % TM, j = q % TN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, af[s][p][i]),
                                                            __builtin_bit_cast(v8bf, bfr[s][j]), acc[i][j], 0, 0, 0);
    };
    using Slot0 = std::integral_constant<int, 0>;
    using Slot1 = std::integral_constant<int, 1>;
    constexpr int kBarrierAt = NM / 4;
    // One K step over LDS stage `buf`: chunk 0 from fragment slot 0 while chunk 1 is read into slot 1
    // and (LOAD) the stage `fill` is requested; chunk 1 from slot 1, the block meets, chunk 0 of
    // stage `next` is read into slot 0 (MORE).
    auto k_step = [&](int buf, int next, int fill, auto load_tag, auto more_tag) {
        constexpr bool LOAD = decltype(load_tag)::value, MORE = decltype(more_tag)::value;
        constexpr int n_loads = LOAD ? kLoads : 0;
        static_for<NM>([&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            mfma_at(Slot0{}, q_tag);
            static_for<kFragOps>([&](auto o_tag) {
                constexpr int o = decltype(o_tag)::value;
                if constexpr ((2 * kFragOps <= NM ? 2 * o + 1 : o * (NM - 2) / kFragOps) == q)
                    frag_op(buf, 1, Slot1{}, o_tag);
            });
            static_for<n_loads>([&](auto o_tag) {
                constexpr int o = decltype(o_tag)::value;
                if constexpr (o * NM / (n_loads > 0 ? n_loads : 1) == q) load_op(fill, o_tag);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (LOAD) {
            a_ptr += BK;
            b_ptr += BK;
        }
        constexpr int room = NM - kBarrierAt - 1;
        static_for<NM>([&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            mfma_at(Slot1{}, q_tag);
            if constexpr (MORE && q == kBarrierAt) {
                // this wavefront has read all of this stage and the next stage has landed; then the
                // block meets
                if constexpr (LOAD)
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 2) * kLoads) : "memory");
                else
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                asm volatile("s_barrier" ::: "memory");
            }
            if constexpr (MORE) {
                static_for<kFragOps>([&](auto o_tag) {
                    constexpr int o = decltype(o_tag)::value;
                    if constexpr (kBarrierAt + 1 + (kFragOps <= room ? o : o * room / kFragOps) == q)
                        frag_op(next, 0, Slot0{}, o_tag);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    if (n_steps > 0) {
        const int pre = n_steps < STAGES - 1 ? n_steps : STAGES - 1;
        for (int s = 0; s < pre; ++s) load_stage(s);
        // stage 0 has landed: everything but the stages requested after it
        if (pre == STAGES - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * kLoads) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        static_for<kFragOps>([&](auto o_tag) { frag_op(0, 0, Slot0{}, o_tag); });
        int buf = 0, fill = STAGES - 1, step = 0;   // fill: the LDS stage the next loads go to
        auto after = [](int stage) { return stage + 1 == STAGES ? 0 : stage + 1; };
        for (; step + STAGES - 1 < n_steps; ++step) {
            k_step(buf, after(buf), fill, std::true_type{}, std::true_type{});
            buf = after(buf);
            fill = after(fill);
        }
        for (; step + 1 < n_steps; ++step) {      // nothing left to request
            k_step(buf, after(buf), fill, std::false_type{}, std::true_type{});
            buf = after(buf);
        }
        k_step(buf, 0, fill, std::false_type{}, std::false_type{});
    }

    float *C = g.c + split * g.slab;
    if constexpr (SWIGLU) {
#pragma unroll
        for (int j = 0; j < TN / 2; ++j) {
            const int col = tile_n * (BN / 2) + wn * (WN / 2) + j * 32 + l32;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * 64 + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    const float gate = acc[i][j][r];
                    const float silu = gate * (1.0f / (1.0f + expf(-gate)));
                    const float act = silu * acc[i][j + TN / 2][r];
                    if (row < g.m) {
                        C[static_cast<int64_t>(row) * g.ldc + col] = act;
                        if (g.act_pieces) {
                            const uint32_t xb = __float_as_uint(act);
                            const uint32_t hb = xb & 0xffff0000u;
                            const bool finite = (xb & 0x7f800000u) != 0x7f800000u;
                            const float r1 = finite ? act - __uint_as_float(hb) : 0.f;
                            const uint32_t mb = __float_as_uint(r1) & 0xffff0000u;
                            const float r2 = r1 - __uint_as_float(mb);
                            uint16_t *pp = g.act_pieces + static_cast<int64_t>(row) * g.n + col;
                            pp[0] = static_cast<uint16_t>(hb >> 16);
                            pp[g.act_plane] = static_cast<uint16_t>(mb >> 16);
                            pp[2 * g.act_plane] = static_cast<uint16_t>(__float_as_uint(r2) >> 16);
                        }
                    }
                }
        }
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int cb = n0 + wn * WN + j * 32;      // first column of this accumulator block
            float *dst = C;
            int64_t ldc = g.ldc;
            int col = cb + l32;
            if (g.n_seg > 0) {
                // (constant indices only: the argument struct stays in scalar registers)
                dst = g.seg_c[0];
                ldc = g.seg_ldc[0];
#pragma unroll
                for (int sgm = 1; sgm < kMaxGroups; ++sgm)
                    if (sgm < g.n_seg && cb >= g.seg_begin[sgm]) {
                        dst = g.seg_c[sgm];
                        ldc = g.seg_ldc[sgm];
                        col = cb - g.seg_begin[sgm] + l32;
                    }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * 64 + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (row < g.m) dst[static_cast<int64_t>(row) * ldc + col] = acc[i][j][r];
                }
        }
    }
}

template <int TN, int STAGES, bool SWIGLU>
int32_t launch_x3(hipStream_t st, X3Args g, int splits) {
    constexpr int BN = 64 * TN;
    constexpr int lds = STAGES * (3 * kTileRows * 64 + BN * 64);
    static_assert(lds <= 160 * 1024, "LDS of a compute unit");
    g.tiles_m = g.m_pad / kTileRows;
    g.tiles_n = g.n / (SWIGLU ? BN / 2 : BN);
    const int64_t tiles = static_cast<int64_t>(g.tiles_m) * g.tiles_n;
    g.per_xcd = static_cast<int32_t>((tiles + 7) / 8);
    auto kern = gemm_bf16x3_kernel<TN, STAGES, SWIGLU>;
    static DynamicLdsGrant grant;
    if (const int32_t st_grant = grant.ensure(kern, lds); st_grant != RMLK_OK) return st_grant;
    kern<<<dim3(g.per_xcd * 8, splits), kThreads, lds, st>>>(g);
    return launch_status();
}

// What the kernels index with 32 bits and fetch in 16-byte units.
bool operands_ok(int64_t m, int64_t k, const void *pieces, const void *wt, int64_t ldw, int64_t w_rows) {
    const int64_t m_pad = padded_rows(m);
    return k % 32 == 0 && ldw >= k && ldw % 8 == 0 && m_pad * k * 6 < ((int64_t)1 << 32) &&
           w_rows * ldw * 2 < ((int64_t)1 << 32) && m_pad < ((int64_t)1 << 30) &&
           reinterpret_cast<uintptr_t>(pieces) % 16 == 0 && reinterpret_cast<uintptr_t>(wt) % 16 == 0;
}

// Slabs of K for a product of `tiles` block tiles: enough blocks for every compute unit where K allows
// (whole K steps, at least eight of them per slab).
int32_t splits_for(int64_t tiles, int64_t k) {
    int32_t s = 1;
    while (s < 8 && tiles * s * 2 <= kNumCU + kNumCU / 4 && k % (64 * s) == 0 && k / (2 * s) >= 256) s *= 2;
    return s;
}

// The plain product: the tile by how many blocks it makes.
int32_t launch_plain(hipStream_t st, const X3Args &g, int32_t splits) {
    const int64_t tiles_m = g.m_pad / kTileRows, n = g.n;
    const bool wide = n % 256 == 0 && tiles_m * (n / 256) * splits >= kNumCU - kNumCU / 8;
    if (wide) {
        // more blocks than compute units: two of them per unit (two stages each) hide more latency
        // than one with three
        if (tiles_m * (n / 256) * splits > 2 * kNumCU) return launch_x3<4, 2, false>(st, g, splits);
        return launch_x3<4, 3, false>(st, g, splits);
    }
    return launch_x3<2, 3, false>(st, g, splits);
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" {

size_t rmlk_hip_bf16x3_pieces_size(int64_t m, int64_t k) {
    if (m <= 0 || k <= 0) return 0;
    return static_cast<size_t>(padded_rows(m)) * static_cast<size_t>(k) * 6;
}

int32_t rmlk_hip_bf16x3_split(rmlk_stream_t stream, int64_t m, int64_t k, const void *a, int64_t lda,
                              void *pieces) {
    hipStream_t st = as_stream(stream);
    if (m < 0 || k < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (m == 0 || k == 0) return RMLK_OK;
    if (!a || !pieces) return RMLK_ERR_NULL_POINTER;
    if (lda < k) return RMLK_ERR_SIZE_MISMATCH;
    const int64_t m_pad = padded_rows(m);
    if (k % 8 != 0 || lda % 4 != 0 || reinterpret_cast<uintptr_t>(a) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(pieces) % 16 != 0 || m_pad >= ((int64_t)1 << 30) || k >= ((int64_t)1 << 30))
        return RMLK_ERR_UNSUPPORTED;
    const int64_t total = m_pad * (k / 8);
    const int64_t blocks = (total + kThreads - 1) / kThreads;
    split_bf16x3_kernel<<<static_cast<uint32_t>(blocks < (1 << 20) ? blocks : (1 << 20)), kThreads, 0, st>>>(
        static_cast<const float *>(a), lda, static_cast<int32_t>(m), static_cast<int32_t>(k),
        static_cast<int32_t>(m_pad), static_cast<uint16_t *>(pieces));
    return launch_status();
}

int32_t rmlk_hip_bf16x3_splits(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || n <= 0 || k <= 0 || k % 32 != 0 || n % 128 != 0) return 0;
    const int64_t tiles_m = padded_rows(m) / kTileRows;
    // (the tile the product will pick: 256 columns where that still gives every unit a block)
    const bool wide = n % 256 == 0 && tiles_m * (n / 256) >= kNumCU - kNumCU / 8;
    return splits_for(tiles_m * (n / (wide ? 256 : 128)), k);
}

int32_t rmlk_hip_matmul_bf16x3(rmlk_stream_t stream, int64_t m, int64_t n, int64_t k, const void *pieces,
                               const void *wt, int64_t ldw, int32_t splits, void *c, int64_t ldc,
                               int64_t slab) {
    hipStream_t st = as_stream(stream);
    if (m < 0 || n < 0 || k < 0 || splits < 1) return RMLK_ERR_INVALID_ARGUMENT;
    if (m == 0 || n == 0) return RMLK_OK;
    if (!pieces || !wt || !c) return RMLK_ERR_NULL_POINTER;
    if (ldc < n || (splits > 1 && slab < m * ldc)) return RMLK_ERR_SIZE_MISMATCH;
    if (k == 0 || n % 128 != 0 || k % (32 * static_cast<int64_t>(splits)) != 0 || n >= ((int64_t)1 << 30) ||
        !operands_ok(m, k, pieces, wt, ldw, n))
        return RMLK_ERR_UNSUPPORTED;
    X3Args g{};
    g.a3 = static_cast<const uint16_t *>(pieces);
    g.b = static_cast<const uint16_t *>(wt);
    g.c = static_cast<float *>(c);
    g.m = static_cast<int32_t>(m);
    g.n = static_cast<int32_t>(n);
    g.k = static_cast<int32_t>(k);
    g.m_pad = static_cast<int32_t>(padded_rows(m));
    g.ldb = ldw;
    g.ldc = ldc;
    g.slab = slab;
    g.k_per_split = static_cast<int32_t>(k / splits);
    return launch_plain(st, g, splits);
}

int32_t rmlk_hip_matmul_bf16x3_grouped(rmlk_stream_t stream, int64_t m, int64_t k, const void *pieces,
                                       const void *wt, int64_t ldw, int32_t groups, const int64_t *widths,
                                       void *const *outs) {
    hipStream_t st = as_stream(stream);
    if (m < 0 || k < 0 || groups < 1 || groups > kMaxGroups || !widths || !outs) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t n = 0;
    for (int i = 0; i < groups; ++i) {
        if (widths[i] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (widths[i] % 32 != 0 || widths[i] == 0) return RMLK_ERR_UNSUPPORTED;
        if (m > 0 && !outs[i]) return RMLK_ERR_NULL_POINTER;
        n += widths[i];
    }
    if (m == 0) return RMLK_OK;
    if (!pieces || !wt) return RMLK_ERR_NULL_POINTER;
    if (k == 0 || n % 128 != 0 || n >= ((int64_t)1 << 30) || !operands_ok(m, k, pieces, wt, ldw, n))
        return RMLK_ERR_UNSUPPORTED;
    X3Args g{};
    g.a3 = static_cast<const uint16_t *>(pieces);
    g.b = static_cast<const uint16_t *>(wt);
    g.m = static_cast<int32_t>(m);
    g.n = static_cast<int32_t>(n);
    g.k = static_cast<int32_t>(k);
    g.m_pad = static_cast<int32_t>(padded_rows(m));
    g.ldb = ldw;
    g.k_per_split = g.k;
    g.n_seg = groups;
    int64_t first = 0;
    for (int i = 0; i < groups; ++i) {
        g.seg_begin[i] = static_cast<int32_t>(first);
        g.seg_c[i] = static_cast<float *>(outs[i]);
        g.seg_ldc[i] = widths[i];
        first += widths[i];
    }
    g.seg_begin[groups] = static_cast<int32_t>(first);
    g.c = g.seg_c[0];
    g.ldc = g.seg_ldc[0];
    return launch_plain(st, g, 1);
}

int32_t rmlk_hip_matmul_bf16x3_swiglu(rmlk_stream_t stream, int64_t m, int64_t n, int64_t k,
                                      const void *pieces, const void *wt, int64_t ldw, int64_t gate_row,
                                      int64_t up_row, void *out, int64_t ldc, void *out_pieces) {
    hipStream_t st = as_stream(stream);
    if (m < 0 || n < 0 || k < 0 || gate_row < 0 || up_row < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (m == 0 || n == 0) return RMLK_OK;
    if (!pieces || !wt || !out) return RMLK_ERR_NULL_POINTER;
    if (ldc < n) return RMLK_ERR_SIZE_MISMATCH;
    const int64_t w_rows = (gate_row > up_row ? gate_row : up_row) + n;
    if (k == 0 || n % 64 != 0 || n >= ((int64_t)1 << 30) || !operands_ok(m, k, pieces, wt, ldw, w_rows))
        return RMLK_ERR_UNSUPPORTED;
    X3Args g{};
    g.a3 = static_cast<const uint16_t *>(pieces);
    g.b = static_cast<const uint16_t *>(wt);
    g.c = static_cast<float *>(out);
    g.m = static_cast<int32_t>(m);
    g.n = static_cast<int32_t>(n);
    g.k = static_cast<int32_t>(k);
    g.m_pad = static_cast<int32_t>(padded_rows(m));
    g.ldb = ldw;
    g.ldc = ldc;
    g.k_per_split = g.k;
    g.gate_row = gate_row;
    g.up_row = up_row;
    if (out_pieces) {
        if (n % 8 != 0 || reinterpret_cast<uintptr_t>(out_pieces) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
        g.act_pieces = static_cast<uint16_t *>(out_pieces);
        g.act_plane = static_cast<int64_t>(g.m_pad) * n;
    }
    const int64_t tiles_m = g.m_pad / kTileRows;
    if (n % 128 == 0 && tiles_m * (n / 128) >= kNumCU - kNumCU / 8) {
        if (tiles_m * (n / 128) > 2 * kNumCU) return launch_x3<4, 2, true>(st, g, 1);
        return launch_x3<4, 3, true>(st, g, 1);
    }
    return launch_x3<2, 3, true>(st, g, 1);
}

}  // extern "C"
