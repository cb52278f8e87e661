// Grouped-query attention over many query rows (prefill) in one kernel for gfx950:
//   out = Softmax(q . k^T * scale + mask) . v,   q [B, G*rep, S, 64], k and v [B, G, L, 64].
// Replaces three launches of the reference's one-kernel-per-node execution (MatMul via
// cublasGemmStridedBatchedEx, cuda/src/kernels/gemm.rs:191-232; Div/Mul and Add,
// cuda/src/kernels/binary.rs:58-100; Softmax, cuda/src/kernels/softmax.rs:5-37; MatMul again) and
// the [rows, L] score and probability matrices they pass through memory.
//
// One block owns 64 query rows of one KV head (the rep query heads that share it lie one after the
// other, so they are rows of ONE matrix) and walks the keys in chunks of 32 * NK, staged in LDS by
// direct global -> LDS loads, two buffers. Wavefront (wq, wk) of the 2 * NK takes query rows
// wq*32.. and keys wk*32.. of every chunk, with its own reference point of the exponents (which
// follows the running maximum), sum and output accumulator (the NK key parts are merged once, at
// the end, through LDS). NK = 2 (four
// wavefronts, 64 KB of LDS, two blocks per CU) when there are blocks enough to fill the chip that
// way; NK = 4 (eight wavefronts, 128 KB) otherwise, so that every SIMD still holds two wavefronts:
// a wavefront's vector instructions do not run under its own MFMAs on this chip, only (in part)
// under another wavefront's.
//
// Everything is computed TRANSPOSED so that a query stays in one lane from the scores to the
// output: S^T = K . Q^T puts query l32 into lane column l32 of the 32x32 MFMA result, with 16 keys
// in the lane's 16 accumulator registers. Those registers, exponentiated, ARE the B operand of
// O^T += V^T . P^T (MFMA k index = lane half, the same key in both operands), and O^T again has the
// query as its lane column. Row maxima and sums are therefore per-lane reductions over registers
// plus one exchange between the two lane halves; no score ever goes through LDS.
#include <cmath>

#include "common.hpp"

namespace rmlk {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));


constexpr int kAttnThreads = 256;                 // of the few-rows kernels
constexpr int kHeadDim = 64;
constexpr int kChunk = 64;                        // keys per block of the few-rows kernel
template <int NK>
struct AttnShape {
    static constexpr int kThreads = 2 * NK * kWave;
    static constexpr int kKeys = 32 * NK;                  // keys per step
    static constexpr int kTile = kKeys * kHeadDim;         // floats of one staged K or V chunk
    static constexpr int kLdsBytes = 2 * 2 * kTile * 4;    // K and V, two buffers each
};
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kSlack = 8.0f / kLog2e;   // how far a score may lie above the point its exponent is taken from

// max / sum of a value over the two lanes (l, l + 32) that share a query, on all 64 lanes: one
// v_permlane32_swap turns x into (lower half twice, upper half twice).
__device__ __forceinline__ void half_pair(float x, float &lo, float &hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

struct AttnArgs {
    const float *q;
    const float *k;
    const float *v;
    const float *mask;
    float *out;
    int32_t rows;      // rep * S query rows per KV head
    int32_t seq;       // S
    int32_t rep;       // query heads per KV head
    int32_t kv_heads;  // G
    int32_t len;       // L keys
    int64_t mask_b, mask_h, mask_s;   // element strides of the mask over batch, head, query
    int64_t out_b, out_h, out_s;      // element strides of out over batch, head, query
    float qscale;      // score scale (folded into the query)
    // Visibility of the mask per (64-query tile, key chunk), one byte each, or null: a chunk whose
    // mask is -inf for all 64 queries of the block is not loaded and not multiplied (its
    // probabilities are exact zeros). Laid out [.., tile, chunk]; tiles_b / tiles_h are the byte
    // strides over batch and head (0 where the mask is broadcast).
    const uint8_t *tiles;
    int64_t tiles_b, tiles_h;
    // With a tile map the blocks differ in work (a causal mask: 1 to L / 64 chunks), and blocks are
    // handed out in order: the grid is then as many blocks as fit the chip at once, each taking the
    // next (query tile, KV head) item from this counter until they run out - last query tiles first,
    // which under a causal mask are the long ones. Null: block (x, y) is item (tile x, KV head y).
    int32_t *queue;
    int32_t items, tiles_per_head;
    // The output also as three bfloat16 pieces whose sum it is exactly (the operand form of
    // rmlk_hip_matmul_bf16x3, for the output projection behind a [B, S, H, D] result): planes of `plane`
    // elements, laid out like `out`. Null: not wanted.
    uint16_t *pieces;
    int64_t plane;
};

// Four floats as three times four bfloat16 (hi, mid, lo: truncate, subtract, truncate, subtract; Inf
// and NaN in hi alone), one 64-bit store per plane.
__device__ __forceinline__ void store_pieces(const v4f &w, uint16_t *at, int64_t plane) {
    uint32_t hi[4], mid[4], lo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t xb = __float_as_uint(w[e]);
        const uint32_t hb = xb & 0xffff0000u;
        const bool finite = (xb & 0x7f800000u) != 0x7f800000u;
        const float r1 = finite ? w[e] - __uint_as_float(hb) : 0.f;
        const uint32_t mb = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(mb);
        hi[e] = hb >> 16;
        mid[e] = mb >> 16;
        lo[e] = __float_as_uint(r2) >> 16;
    }
    *reinterpret_cast<uint2 *>(at) = uint2{hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16)};
    *reinterpret_cast<uint2 *>(at + plane) = uint2{mid[0] | (mid[1] << 16), mid[2] | (mid[3] << 16)};
    *reinterpret_cast<uint2 *>(at + 2 * plane) = uint2{lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16)};
}

// WHOLE: the keys are a multiple of the step's, so every chunk lies inside them.
// PAIRED (with a tile map, one block per compute unit): the two halves of a block's wavefronts take
// 32 rows each of two DIFFERENT query tiles of a head, tile i and tile T - 1 - i. Under a causal mask
// one of them sees many chunks and the other few, and a SIMD holds a wavefront of either half: every
// SIMD of the chip then has the same work, where whole tiles leave the last tile's block to decide
// when the kernel ends. The block walks the chunks that either tile sees; a wavefront sits out the
// ones its own tile does not see (it still fetches its share of them).
template <int NK, bool WHOLE, bool PAIRED>
__global__ __launch_bounds__(AttnShape<NK>::kThreads) void attention_rows_kernel(AttnArgs g) {
    constexpr int kKeys = AttnShape<NK>::kKeys, kTile = AttnShape<NK>::kTile;
    extern __shared__ __align__(16) float smem[];
    float *Ks = smem;               // [2][keys][16 units of 4 floats], unit u of key r at u ^ (r & 15)
    float *Vs = smem + 2 * kTile;   // [2][keys][64], column c of key r at c ^ (32 * ((r >> 2) & 1))

    const int tid = threadIdx.x;
    const int lane = tid % kWave, wave = tid / kWave;
    const int l32 = lane % 32, half = lane / 32;
    const int wq = wave / NK, wk = wave % NK;
    __shared__ int next_item;
    // With a queue a block starts with the item of its own number (no ticket, so the blocks do not
    // all meet at the counter when the kernel starts) and draws a ticket under the last step of
    // every item it works on: ticket t stands for item t + gridDim.x. One ticket per item, so the
    // tickets of a launch are 0 .. items - 1, the last gridDim.x of them for nothing.
    int item = blockIdx.x, drawn = 0;
    // With a queue two blocks share a compute unit, a wavefront of each on every SIMD, and between
    // wavefronts of equal priority the SIMD serves the older one first: left alone, the block that
    // arrived first runs a sixth faster than its neighbour, and the slower blocks decide when the
    // kernel ends. The wavefronts therefore change their priority with every step, the two
    // neighbours (told apart by the wave slot they sit in, bits 3:0 of HW_ID) in opposite phase.
    const int slot_bit = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (3 << 11)) & 1;
    for (;;) {
    int bg = blockIdx.y, tile_x = blockIdx.x;
    if (g.queue) {
        // items by falling query tile; inside one tile index, all the heads of all the KV heads
        const int n_bg = g.items / (g.tiles_per_head * g.rep);
        const int per_tile = n_bg * g.rep;
        const int t = g.tiles_per_head - 1 - item / per_tile, hb = item % per_tile;
        bg = hb / g.rep;
        tile_x = (hb - bg * g.rep) * g.tiles_per_head + t;
    }
    const int b = bg / g.kv_heads, grp = bg - b * g.kv_heads;
    const int r0 = tile_x * 64;
    // the first of this wavefront's 32 query rows, and of the rows of the block's other half
    int rbase = r0 + wq * 32, rbase_other = r0 + (wq ^ 1) * 32;
    if constexpr (PAIRED) {
        // blocks 2 i and 2 i + 1 of a head: rows 0..31 and 32..63 of the tiles T - 1 - i and i
        const int hd = tile_x / g.tiles_per_head, j = tile_x - hd * g.tiles_per_head;
        const int far = (hd * g.tiles_per_head + g.tiles_per_head - 1 - j / 2) * 64 + (j & 1) * 32;
        const int near = (hd * g.tiles_per_head + j / 2) * 64 + (j & 1) * 32;
        rbase = wq == 0 ? far : near;
        rbase_other = wq == 0 ? near : far;
    }
    const float *Kg = g.k + static_cast<int64_t>(bg) * g.len * kHeadDim;
    const float *Vg = g.v + static_cast<int64_t>(bg) * g.len * kHeadDim;
    const int n_chunks = (g.len + kKeys - 1) / kKeys;

    // ---- the chunks this block visits (bit c of active[c / 64]); all of them without a tile map ------
    uint64_t active[2];
    active[0] = n_chunks >= 64 ? ~0ull : ((1ull << n_chunks) - 1);
    active[1] = n_chunks >= 128 ? ~0ull : (n_chunks > 64 ? ((1ull << (n_chunks - 64)) - 1) : 0ull);
    uint64_t mine[2] = {active[0], active[1]};   // PAIRED: the chunks this wavefront's own tile sees
    if (g.tiles) {   // (the launcher gives a map only for n_chunks <= 128 and seq % 64 == 0: a tile lies in one head)
        auto seen_from = [&](int row, uint64_t (&out)[2]) {   // the map's row of the tile that holds query row `row`
            const int head0 = grp * g.rep + row / g.seq, srow0 = row - (row / g.seq) * g.seq;
            const uint8_t *tp =
                g.tiles + b * g.tiles_b + head0 * g.tiles_h + static_cast<int64_t>(srow0 / 64) * n_chunks;
            const bool f0 = lane < n_chunks && tp[min(lane, n_chunks - 1)] != 0;
            const bool f1 = lane + 64 < n_chunks && tp[min(lane + 64, n_chunks - 1)] != 0;
            out[0] = __builtin_amdgcn_ballot_w64(f0);
            out[1] = __builtin_amdgcn_ballot_w64(f1);
            if ((out[0] | out[1]) == 0) out[0] = 1;   // nothing visible at all: chunk 0 gives the NaN rows
        };
        seen_from(rbase, mine);
        active[0] = mine[0];
        active[1] = mine[1];
        if constexpr (PAIRED) {
            uint64_t other[2];
            seen_from(rbase_other, other);
            active[0] |= other[0];
            active[1] |= other[1];
        }
    }
    auto next_active = [&](int c) {   // the first visited chunk after c, -1 when there is none
        const int from = c + 1;
        if (from < 64) {
            const uint64_t m = active[0] & (~0ull << from);
            if (m) return static_cast<int>(__builtin_ctzll(m));
        }
        if (from < 128) {
            const uint64_t m = from <= 64 ? active[1] : (active[1] & (~0ull << (from - 64)));
            if (m) return 64 + static_cast<int>(__builtin_ctzll(m));
        }
        if (from >= 128 && from < n_chunks) return from;   // beyond the map: every chunk
        return -1;
    };

    // ---- staging: piece p * 2 NK + wave of a chunk (4 keys, 1 KiB) is this wavefront's p-th load ---
    const int lrow = wave * 4 + lane / 16;   // key of this lane inside a group of 8 NK keys
    const int lunit = lane % 16;
    const uint32_t k_col = static_cast<uint32_t>((lunit ^ (lrow & 15)) * 4);
    const uint32_t v_col = static_cast<uint32_t>((lunit ^ ((wave & 1) << 3)) * 4);
    const uint32_t lds_k = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(Ks)) + wave * 1024u);
    const uint32_t lds_v = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(Vs)) + wave * 1024u);
    auto direct_load = [&](uint32_t lds_addr, const float *base, uint32_t voff) {
        // (one wait state between a scalar write of M0 and the LDS-bound load that reads it)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(base)
                     : "memory", "m0");
    };
    // Piece p (0..3: K, 4..7: V) of chunk c into buffer buf. WHOLE: the chunk and the piece move
    // only the scalar base address, the lane's offset is the same for all of them, and no vector
    // instruction is spent on addresses (a wavefront's vector ALU instructions do not run under its
    // own fp32 MFMAs on this chip: behind a 64-cycle MFMA each one adds its four cycles, so every
    // such instruction costs matrix time). Otherwise rows past the end are read from the last row.
    const uint32_t k_lane = static_cast<uint32_t>(lrow * kHeadDim + k_col) * 4u;
    const uint32_t v_lane = static_cast<uint32_t>(lrow * kHeadDim + v_col) * 4u;
    auto issue_piece = [&](int p, int c, int buf) {
        const uint32_t lds_at = static_cast<uint32_t>(buf * kTile * 4 + (p & 3) * 2048 * NK);
        if constexpr (WHOLE) {
            const int64_t first = static_cast<int64_t>(c * kKeys + (p & 3) * 8 * NK) * kHeadDim;
            if (p < 4)
                direct_load(lds_k + lds_at, Kg + first, k_lane);
            else
                direct_load(lds_v + lds_at, Vg + first, v_lane);
        } else {
            const int key = min(c * kKeys + (p & 3) * 8 * NK + lrow, g.len - 1);
            if (p < 4)
                direct_load(lds_k + lds_at, Kg, static_cast<uint32_t>(key * kHeadDim + k_col) * 4u);
            else
                direct_load(lds_v + lds_at, Vg, static_cast<uint32_t>(key * kHeadDim + v_col) * 4u);
        }
    };

    // ---- this lane's query: B operand of S^T, scaled once --------------------------------------
    const int qrow = min(rbase + l32, g.rows - 1);
    const float *qp = g.q + (static_cast<int64_t>(bg) * g.rows + qrow) * kHeadDim + half * 4;
    v4f qf[8];
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) {
        const v4f raw = *reinterpret_cast<const v4f *>(qp + kc * 8);
#pragma unroll
        for (int s = 0; s < 4; ++s) qf[kc][s] = raw[s] * g.qscale;
    }
    // The query is in registers before any of the hand-issued loads below starts: the waits the
    // compiler places for its own loads count only those.
#pragma unroll
    for (int kc = 0; kc < 8; ++kc) asm volatile("" : "+v"(qf[kc]));
    const int head = grp * g.rep + qrow / g.seq, srow = qrow - (qrow / g.seq) * g.seq;
    const float *mrow = g.mask + b * g.mask_b + head * g.mask_h + srow * g.mask_s;

    const float kNegInf = -INFINITY;
    float m_run = kNegInf, l_run = 0.f;
    v16f o0, o1;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        o0[r] = 0.f;
        o1[r] = 0.f;
    }

    // The mask of this lane's 16 keys of a chunk (keys 8a + 4*half + 0..3 of the wavefront's 32) is
    // fetched one chunk ahead, together with that chunk's K and V, and everything is awaited at once
    // at the end of a step. These are ordinary loads on purpose: the compiler has to know that the
    // registers are still in flight. (Issued from inline assembly they looked ready at once, and
    // the register allocator copied them to other registers BEFORE the wait, which now and then
    // picked up what the registers held before the data arrived.)
    const float *mlane = mrow + wk * 32 + 4 * half;   // this lane's first key of chunk 0
    auto load_mask = [&](int a, int c) {
        if constexpr (WHOLE) {
            return *reinterpret_cast<const v4f *>(mlane + (c * kKeys + 8 * a));
        } else {
            const int key0 = c * kKeys + wk * 32 + 4 * half;
            return *reinterpret_cast<const v4f *>(mrow + min(key0 + 8 * a, g.len - 4));
        }
    };
    const int first_chunk = next_active(-1);
    v4f mk[4], mk_next[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) mk[a] = load_mask(a, first_chunk);
#pragma unroll
    for (int p = 0; p < 8; ++p) issue_piece(p, first_chunk, 0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier"
                 : "+v"(mk[0]), "+v"(mk[1]), "+v"(mk[2]), "+v"(mk[3])
                 :
                 : "memory");

    const int k_frag = (wk * 32 + l32) * kHeadDim;     // this lane's key row of a staged chunk
    const int k_swz = l32 & 15;
    const int v_frag0 = (wk * 32 + 4 * half) * kHeadDim + (half * 32 + l32);        // d =      l32
    const int v_frag1 = (wk * 32 + 4 * half) * kHeadDim + ((half ^ 1) * 32 + l32);  // d = 32 + l32
    // The LDS byte addresses of this lane's fragment reads, for the buffer the next step reads: kept
    // in registers and moved to the other buffer by ten adds in a row at the end of a step. (Formed
    // from the buffer number in front of every read, each was a vector add that an LDS read waited
    // for between two MFMAs, and such a pair holds the next MFMA back by some 25 cycles.)
    using LdsV4 = const v4f __attribute__((address_space(3))) *;
    using LdsF = const float __attribute__((address_space(3))) *;
    uint32_t k_at[8], v_at[2];
    {
        const uint32_t ks0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(Ks));
        const uint32_t vs0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(Vs));
#pragma unroll
        for (int kc = 0; kc < 8; ++kc)
            k_at[kc] = ks0 + static_cast<uint32_t>(k_frag + (((kc * 2 + half) ^ k_swz) * 4)) * 4u;
        v_at[0] = vs0 + static_cast<uint32_t>(v_frag0) * 4u;
        v_at[1] = vs0 + static_cast<uint32_t>(v_frag1) * 4u;
    }
    int32_t to_other = kTile * 4;   // to the other buffer: +, -, +, ...

    // chunk c from buffer buf; MORE: chunk `next` is fetched into the other buffer meanwhile
    auto step = [&](int c, int next, int buf, auto more_tag) {
        constexpr bool MORE = decltype(more_tag)::value;
        const int key0 = c * kKeys + wk * 32 + 4 * half;
        if (g.queue) {
            if ((c ^ slot_bit) & 1)
                __builtin_amdgcn_s_setprio(1);
            else
                __builtin_amdgcn_s_setprio(0);
        }
        if constexpr (!MORE) {   // the ticket for the item after this one comes back under this step
            if (g.queue && tid == 0) drawn = atomicAdd(g.queue, 1);
        }

        bool here = true;
        if constexpr (PAIRED) here = c >= 128 || ((mine[c >> 6] >> (c & 63)) & 1) != 0;
        if (here) {
        // S^T (32 keys x 32 queries) = K . Q^T over the 64 head dims
        v16f st = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // The next chunk's eight pieces and its mask are requested one after each group of four
        // MFMAs (all at the top of the step they kept the matrix pipe idle for some 1200 cycles of
        // address arithmetic and load issue per step).
        static_for<8>([&](auto kc_tag) {
            constexpr int kc = decltype(kc_tag)::value;
            const v4f kf = *(LdsV4)(k_at[kc]);
#pragma unroll
            for (int s = 0; s < 4; ++s)
                st = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[kc][s], st, 0, 0, 0);
            if constexpr (MORE) {
                if constexpr (kc < 4) mk_next[kc] = load_mask(kc, next);
                issue_piece(kc, next, buf ^ 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // The mask is added to the natural-log scores, as the Add node in front of a Softmax adds it,
        // and only the difference to the running maximum is scaled by log2(e): a mask of the most
        // negative finite float (what exported graphs use for "hidden") stays finite, so a row with
        // nothing else visible comes out uniform like the separate kernels' (scaled by log2(e) first
        // such a mask overflows to -inf and the row turns NaN).
        float t[16];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) t[4 * a + e] = st[4 * a + e] + mk[a][e];
        if (!WHOLE && (c + 1) * kKeys > g.len) {
            // keys past the end (their rows and mask values were read from valid but unrelated places)
#pragma unroll
            for (int a = 0; a < 4; ++a)
                if (key0 + 8 * a >= g.len) {   // L is a multiple of 4: a lane's four keys go together
#pragma unroll
                    for (int e = 0; e < 4; ++e) t[4 * a + e] = kNegInf;
                }
        }
        float mx = t[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(mx, t[r]);
        {
            float lo, hi;
            half_pair(mx, lo, hi);
            mx = fmaxf(lo, hi);
        }
        // m_run is the point the exponents are taken from, not the maximum itself: it follows the
        // maximum only when a score of this chunk lies more than kSlack above it (probabilities then
        // stay below 2^8, far inside the range of a float), so that the 32 accumulator registers
        // and the sum are rescaled in the first chunks of a row and hardly ever afterwards - under a
        // causal mask some query of a wavefront meets a new maximum in most chunks. The quotient
        // of output and sum does not depend on the point. (-inf + kSlack is -inf: the first finite
        // score moves it; a NaN moves nothing and reaches the output through its probability.)
        if (__builtin_amdgcn_ballot_w64(mx > m_run + kSlack) != 0) {
            const float m_new = fmaxf(m_run, mx);
            const float m_to = m_new == kNegInf ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_to) * kLog2e);   // exactly 1 where m_new == m_run
            l_run *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                o0[r] *= alpha;
                o1[r] *= alpha;
            }
            m_run = m_new;
        }
        const float m_safe = m_run == kNegInf ? 0.f : m_run;   // a row with nothing visible so far
        float p[16], psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            p[r] = __builtin_amdgcn_exp2f((t[r] - m_safe) * kLog2e);
            psum += p[r];
        }
        l_run += psum;

        // O^T (64 dims x 32 queries) += V^T . P^T over this wavefront's 32 keys
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key_off = (8 * (r / 4) + (r % 4)) * kHeadDim;
            o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(*(LdsF)(v_at[0] + key_off * 4), p[r], o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(*(LdsF)(v_at[1] + key_off * 4), p[r], o1, 0, 0, 0);
        }
        } else if constexpr (MORE) {   // not this wavefront's chunk: only its share of the next one's loads
#pragma unroll
            for (int a = 0; a < 4; ++a) mk_next[a] = load_mask(a, next);
#pragma unroll
            for (int pc = 0; pc < 8; ++pc) issue_piece(pc, next, buf ^ 1);
        }
        if constexpr (MORE) {   // the next step reads the other buffer
#pragma unroll
            for (int kc = 0; kc < 8; ++kc) asm volatile("v_add_u32 %0, %0, %1" : "+v"(k_at[kc]) : "s"(to_other));
            asm volatile("v_add_u32 %0, %0, %1" : "+v"(v_at[0]) : "s"(to_other));
            asm volatile("v_add_u32 %0, %0, %1" : "+v"(v_at[1]) : "s"(to_other));
            to_other = -to_other;
        }
        // the next chunk and its mask have landed and nobody reads this chunk any more
        if constexpr (MORE) {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier"
                         : "+v"(mk_next[0]), "+v"(mk_next[1]), "+v"(mk_next[2]), "+v"(mk_next[3])
                         :
                         : "memory");
#pragma unroll
            for (int a = 0; a < 4; ++a) mk[a] = mk_next[a];
        } else {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
    };
    {
        int c = first_chunk, buf = 0;
        for (int next = next_active(c); next >= 0; next = next_active(c)) {
            step(c, next, buf, std::true_type{});
            c = next;
            buf ^= 1;
        }
        step(c, -1, buf, std::false_type{});
    }

    // ---- merge the NK key parts of every query tile and write -------------------------------------
    {
        float lo, hi;
        half_pair(l_run, lo, hi);
        l_run = lo + hi;
    }
    // the staging buffers are free after the last barrier: part wk >= 1 of tile wq leaves its
    // maximum, sum and output in slot (wq, wk - 1)
    constexpr int kSlot = 34 * kWave;
    float *cb = smem + wq * ((NK - 1) * kSlot);
    if (wk != 0) {
        float *mine = cb + (wk - 1) * kSlot;
        mine[lane] = m_run;
        mine[kWave + lane] = l_run;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            mine[(2 + r) * kWave + lane] = o0[r];
            mine[(18 + r) * kWave + lane] = o1[r];
        }
    }
    if (g.queue && tid == 0) next_item = drawn + static_cast<int>(gridDim.x);
    __syncthreads();
    const int following = next_item;
    if (wk == 0) {
        float m_f = m_run;
#pragma unroll
        for (int j = 0; j < NK - 1; ++j) m_f = fmaxf(m_f, cb[j * kSlot + lane]);
        const float m_safe = m_f == kNegInf ? 0.f : m_f;
        const float a0 = __builtin_amdgcn_exp2f((m_run - m_safe) * kLog2e);
        float aj[NK - 1], total = l_run * a0;
#pragma unroll
        for (int j = 0; j < NK - 1; ++j) {
            aj[j] = __builtin_amdgcn_exp2f((cb[j * kSlot + lane] - m_safe) * kLog2e);
            total += cb[j * kSlot + kWave + lane] * aj[j];
        }
        const float inv = 1.0f / total;   // nothing visible at all: 0 * inf = NaN, as Softmax
        const int row = rbase + l32;
        if (row < g.rows) {
            float *op = g.out + b * g.out_b + head * g.out_h + srow * g.out_s + 4 * half;   // row == qrow here
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                v4f w0, w1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = 4 * a + e;
                    float s0 = o0[r] * a0, s1 = o1[r] * a0;
#pragma unroll
                    for (int j = 0; j < NK - 1; ++j) {
                        s0 += cb[j * kSlot + (2 + r) * kWave + lane] * aj[j];
                        s1 += cb[j * kSlot + (18 + r) * kWave + lane] * aj[j];
                    }
                    w0[e] = s0 * inv;
                    w1[e] = s1 * inv;
                }
                *reinterpret_cast<v4f *>(op + 8 * a) = w0;
                *reinterpret_cast<v4f *>(op + 32 + 8 * a) = w1;
                if (g.pieces) {
                    uint16_t *pp = g.pieces + (op - g.out);
                    store_pieces(w0, pp + 8 * a, g.plane);
                    store_pieces(w1, pp + 32 + 8 * a, g.plane);
                }
            }
        }
    }
    if (!g.queue) break;
    if (following >= g.items) {
        // the counter only grows; the block that drew the last ticket of the launch leaves it as it
        // found it (zero), so that the map and its counter serve another launch without being made again
        if (tid == 0 && drawn == g.items - 1)
            __hip_atomic_store(g.queue, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
    }
    item = following;
    __syncthreads();   // the merge has read its slots, and thread 0 may write next_item again
    }
}

// ---- which (64-query tile, key chunk) pairs of a mask hold anything but -inf -----------------------
// Block (chunk, tile, batch x head of the mask) looks at 64 x KEYS mask values; a byte per pair.
template <int KEYS>
__global__ __launch_bounds__(256) void attention_mask_tiles_kernel(const float *__restrict__ mask, int64_t mask_b,
                                                                   int64_t mask_h, int64_t mask_s, int32_t heads,
                                                                   int32_t seq, int32_t len,
                                                                   uint8_t *__restrict__ tiles,
                                                                   int32_t *__restrict__ queue) {
    const int chunk = blockIdx.x, tile = blockIdx.y, bh = blockIdx.z;
    if (chunk == 0 && tile == 0 && bh == 0 && threadIdx.x == 0) *queue = 0;   // the item counter of the kernel that follows
    const int b = bh / heads, h = bh - b * heads;
    const float *base = mask + b * mask_b + h * mask_h;
    constexpr int kVecPerRow = KEYS / 4;
    bool seen = false;
    for (int i = threadIdx.x; i < 64 * kVecPerRow; i += 256) {
        const int row = tile * 64 + i / kVecPerRow, key = chunk * KEYS + (i % kVecPerRow) * 4;
        if (row < seq && key < len) {   // len % 4 == 0: a vector is inside or outside
            const v4f m = *reinterpret_cast<const v4f *>(base + row * mask_s + key);
#pragma unroll
            for (int e = 0; e < 4; ++e) seen |= !(m[e] == -INFINITY);
        }
    }
    const int any = __syncthreads_or(seen ? 1 : 0);
    if (threadIdx.x == 0)
        tiles[(static_cast<int64_t>(bh) * gridDim.y + tile) * gridDim.x + chunk] = any ? 1 : 0;
}

// ---- a handful of query rows (a decode step): keys split over blocks ------------------------------
// With one query row per head there is no matrix work to speak of, only the K and V rows to read:
// block (chunk, kv head) takes 64 keys for all the query rows of that KV head (rep * q_len <= 16),
// leaves a partial softmax (maximum, sum, unnormalised output) per row, and a second small kernel
// merges the chunks. B * G * L / 64 blocks instead of B * G keep enough loads in flight.
constexpr int kFewRowsMax = 16;
constexpr int kPartial = kHeadDim + 2;   // floats per (row, chunk): output, maximum, sum

template <bool FRESH>
__device__ __forceinline__ void merge_row(const AttnArgs &g, const float *__restrict__ ws, int n_chunks, int bg,
                                          int r, int lane);
template <bool FRESH>
__device__ __forceinline__ void merge_row_many(const AttnArgs &g, const float *__restrict__ ws, int n_chunks,
                                               int bg, int r, int lane);

// MERGE: the block that finishes last for a KV head (a counter per KV head tells, zero before the
// launch and zero again after it) merges the partial results of all chunks itself; otherwise a
// second kernel does. Blocks of one launch run on different XCDs, whose L2s do not see each other's
// lines; a device-wide fence on both sides would write back and invalidate whole L2s (measured: some
// 6 us per launch, more than the merge launch costs). Instead the partial results alone bypass the
// cache: device-scope stores that go through to memory, awaited before the block counts itself,
// and device-scope loads in the merging block.
template <bool MERGE>
__global__ __launch_bounds__(kAttnThreads) void attention_few_rows_kernel(AttnArgs g, float *__restrict__ ws,
                                                                          float scale, int32_t scale_is_mul,
                                                                          int32_t *__restrict__ counters) {
    __shared__ float Ks[kChunk][kHeadDim + 1];   // +1: lanes read different rows of one column
    __shared__ __align__(16) float Vs[kChunk][kHeadDim];
    __shared__ __align__(16) float qs[kFewRowsMax][kHeadDim];
    __shared__ float ps[kFewRowsMax][kChunk];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int chunk = blockIdx.x, n_chunks = gridDim.x, bg = blockIdx.y;
    const int b = bg / g.kv_heads, grp = bg - b * g.kv_heads;
    const int rows = g.rows;
    const float *Kg = g.k + static_cast<int64_t>(bg) * g.len * kHeadDim;
    const float *Vg = g.v + static_cast<int64_t>(bg) * g.len * kHeadDim;
    const float *Qg = g.q + static_cast<int64_t>(bg) * rows * kHeadDim;
    // stage the chunk (rows past the end: the last valid row, masked below) and the queries
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int idx = tid + i * kAttnThreads;      // 16-byte unit of the 64 x 64 chunk
        const int r = idx / 16, u = idx % 16;
        const int key = min(chunk * kChunk + r, g.len - 1);
        const v4f kv = *reinterpret_cast<const v4f *>(Kg + static_cast<int64_t>(key) * kHeadDim + u * 4);
        const v4f vv = *reinterpret_cast<const v4f *>(Vg + static_cast<int64_t>(key) * kHeadDim + u * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) Ks[r][u * 4 + e] = kv[e];
        *reinterpret_cast<v4f *>(&Vs[r][u * 4]) = vv;
    }
    for (int idx = tid; idx < rows * 16; idx += kAttnThreads)
        *reinterpret_cast<v4f *>(&qs[idx / 16][(idx % 16) * 4]) =
            *reinterpret_cast<const v4f *>(Qg + static_cast<int64_t>(idx) * 4);
    // the mask value of the wavefront's first row: asked for now, on its way with the chunk (after
    // the dot product it would be a trip to memory of its own)
    const int key = chunk * kChunk + lane;
    float mask_first = 0.f;
    if (wave < rows && key < g.len) {
        const int head = grp * g.rep + wave / g.seq, srow = wave - (wave / g.seq) * g.seq;
        mask_first = g.mask[b * g.mask_b + head * g.mask_h + srow * g.mask_s + key];
    }
    __syncthreads();
    for (int r = wave; r < rows; r += kAttnThreads / kWave) {
        const int head = grp * g.rep + r / g.seq, srow = r - (r / g.seq) * g.seq;
        float dot = 0.f;
#pragma unroll 16
        for (int d = 0; d < kHeadDim; ++d) dot = fmaf(qs[r][d], Ks[lane][d], dot);
        float sc = -INFINITY;
        if (key < g.len) {
            const float m = r == wave ? mask_first
                                      : g.mask[b * g.mask_b + head * g.mask_h + srow * g.mask_s + key];
            sc = (scale_is_mul ? dot * scale : dot / scale) + m;
        }
        const float mx = wave_max(sc);
        const float m_safe = mx == -INFINITY ? 0.f : mx;
        const float p = expf(sc - m_safe);
        const float sum = wave_sum(p);
        ps[r][lane] = p;   // read back by this wavefront only
        __builtin_amdgcn_wave_barrier();
        float acc = 0.f;   // lane = head dim
#pragma unroll 16
        for (int j = 0; j < kChunk; ++j) acc = fmaf(ps[r][j], Vs[j][lane], acc);
        float *dst = ws + ((static_cast<int64_t>(bg) * n_chunks + chunk) * rows + r) * kPartial;
        if constexpr (MERGE) {
            __hip_atomic_store(dst + lane, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0) {
                __hip_atomic_store(dst + kHeadDim, mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + kHeadDim + 1, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        } else {
            dst[lane] = acc;
            if (lane == 0) {
                dst[kHeadDim] = mx;
                dst[kHeadDim + 1] = sum;
            }
        }
    }
    if constexpr (MERGE) {
        __shared__ int is_last;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's stores have reached memory ...
        __syncthreads();                                    // ... and so have the block's, before it counts itself done
        if (tid == 0)
            is_last = __hip_atomic_fetch_add(counters + bg, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                      n_chunks - 1;
        __syncthreads();
        if (!is_last) return;
        if (tid == 0) counters[bg] = 0;   // for the next launch
        for (int r = wave; r < rows; r += kAttnThreads / kWave) {
            if (n_chunks <= kWave) merge_row<true>(g, ws, n_chunks, bg, r, lane);
            else merge_row_many<true>(g, ws, n_chunks, bg, r, lane);
        }
    }
}

// out row = sum over chunks of the partial outputs, rescaled to the common maximum, over the
// rescaled sums; a wavefront per (kv head, row), lane = head dim. The kernel is one trip to memory
// long, so it asks for everything at once: lane c the maximum and the sum of chunk c, then every
// lane its element of the first sixteen partial outputs, and only then reduces the maxima (loads
// return in order: the reduction runs while the outputs are on their way). Up to 64 chunks.
constexpr int kMergeGroup = 16;
constexpr int kMergeMaxChunks = kWave;

// FRESH: the partial results were written by other blocks of the SAME launch, possibly through
// another XCD's L2: they are read with device-scope loads, which that cache does not answer from
// what it holds (the writers stored them the same way, see the few-rows kernel).
template <bool FRESH>
__device__ __forceinline__ float partial_load(const float *p) {
    if constexpr (FRESH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *p;
}

// (kv head bg, row r) by one wavefront, n_chunks <= 64
template <bool FRESH>
__device__ __forceinline__ void merge_row(const AttnArgs &g, const float *__restrict__ ws, int n_chunks, int bg,
                                          int r, int lane) {
    const int rows = g.rows;
    const int b = bg / g.kv_heads, grp = bg - b * g.kv_heads;
    const float *src = ws + (static_cast<int64_t>(bg) * n_chunks * rows + r) * kPartial;
    const int64_t step = static_cast<int64_t>(rows) * kPartial;
    const int mine = min(lane, n_chunks - 1);
    const float m_c = partial_load<FRESH>(src + mine * step + kHeadDim);
    const float s_c = partial_load<FRESH>(src + mine * step + kHeadDim + 1);
    float part[kMergeGroup];
#pragma unroll
    for (int j = 0; j < kMergeGroup; ++j) part[j] = partial_load<FRESH>(src + min(j, n_chunks - 1) * step + lane);
    const float m = wave_max(lane < n_chunks ? m_c : -INFINITY);
    const float m_safe = m == -INFINITY ? 0.f : m;
    const float w = lane < n_chunks ? expf(m_c - m_safe) : 0.f;
    const float sum = wave_sum(lane < n_chunks ? s_c * w : 0.f);
    float acc = 0.f;
    for (int c0 = 0; c0 < n_chunks; c0 += kMergeGroup) {
        if (c0 > 0) {
#pragma unroll
            for (int j = 0; j < kMergeGroup; ++j) part[j] = partial_load<FRESH>(src + min(c0 + j, n_chunks - 1) * step + lane);
        }
#pragma unroll
        for (int j = 0; j < kMergeGroup; ++j) {
            // (chunks past the end read the last one again with weight 0: lanes >= n_chunks hold w = 0)
            const float wj = __shfl(w, c0 + j, kWave);
            acc = fmaf(part[j], c0 + j < n_chunks ? wj : 0.f, acc);
        }
    }
    const int head = grp * g.rep + r / g.seq, srow = r - (r / g.seq) * g.seq;
    g.out[b * g.out_b + head * g.out_h + srow * g.out_s + lane] = acc / sum;   // nothing visible: 0 / 0
}

// The same for more chunks than a wavefront has lanes: maxima and sums a chunk per lane in rounds,
// then the outputs chunk by chunk.
template <bool FRESH>
__device__ __forceinline__ void merge_row_many(const AttnArgs &g, const float *__restrict__ ws, int n_chunks,
                                               int bg, int r, int lane) {
    const int rows = g.rows;
    const int b = bg / g.kv_heads, grp = bg - b * g.kv_heads;
    const float *src = ws + (static_cast<int64_t>(bg) * n_chunks * rows + r) * kPartial;
    const int64_t step = static_cast<int64_t>(rows) * kPartial;
    float m = -INFINITY;
    for (int c0 = 0; c0 < n_chunks; c0 += kWave)
        if (c0 + lane < n_chunks) m = fmaxf(m, partial_load<FRESH>(src + (c0 + lane) * step + kHeadDim));
    m = wave_max(m);
    const float m_safe = m == -INFINITY ? 0.f : m;
    float acc = 0.f, sum = 0.f;
    for (int c0 = 0; c0 < n_chunks; c0 += kWave) {
        const int c = c0 + lane;
        const float w = c < n_chunks ? expf(partial_load<FRESH>(src + c * step + kHeadDim) - m_safe) : 0.f;
        if (c < n_chunks) sum = fmaf(partial_load<FRESH>(src + c * step + kHeadDim + 1), w, sum);
        const int here = min(kWave, n_chunks - c0);
#pragma unroll 8
        for (int j = 0; j < here; ++j) acc = fmaf(partial_load<FRESH>(src + (c0 + j) * step + lane), __shfl(w, j, kWave), acc);
    }
    sum = wave_sum(sum);
    const int head = grp * g.rep + r / g.seq, srow = r - (r / g.seq) * g.seq;
    g.out[b * g.out_b + head * g.out_h + srow * g.out_s + lane] = acc / sum;   // nothing visible: 0 / 0
}

__global__ __launch_bounds__(kAttnThreads) void attention_merge_kernel(AttnArgs g, const float *__restrict__ ws,
                                                                       int32_t n_chunks, int32_t total_rows) {
    const int item = blockIdx.x * (kAttnThreads / kWave) + threadIdx.x / kWave;
    if (item >= total_rows) return;
    merge_row<false>(g, ws, n_chunks, item / g.rows, item % g.rows, threadIdx.x % kWave);
}

__global__ __launch_bounds__(kAttnThreads) void attention_merge_many_kernel(AttnArgs g, const float *__restrict__ ws,
                                                                            int32_t n_chunks, int32_t total_rows) {
    const int item = blockIdx.x * (kAttnThreads / kWave) + threadIdx.x / kWave;
    if (item >= total_rows) return;
    merge_row_many<false>(g, ws, n_chunks, item / g.rows, item % g.rows, threadIdx.x % kWave);
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

namespace {

// Argument checks and the argument block shared by both attention entry points; RMLK_OK with
// *empty set when there is nothing to compute.
int32_t attention_args(int32_t dtype, int64_t batch, int64_t kv_heads, int64_t rep, int64_t q_len,
                       int64_t kv_len, int64_t head_dim, const void *q, const void *k, const void *v,
                       const void *mask, const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                       int32_t out_seq_major, void *out, bool vector_mask, AttnArgs *args, bool *empty) {
    *empty = false;
    if (!dims_ok(mask_stride) || mask_stride->rank != 4) return RMLK_ERR_BAD_RANK;
    if (batch < 0 || kv_heads < 0 || rep < 0 || q_len < 0 || kv_len < 0 || head_dim < 0)
        return RMLK_ERR_INVALID_ARGUMENT;
    if (dtype != RMLK_FLOAT || head_dim != kHeadDim) return RMLK_ERR_UNSUPPORTED;
    const int64_t rows = rep * q_len;
    if (batch * kv_heads * rows == 0) {
        *empty = true;
        return RMLK_OK;
    }
    if (kv_len == 0) return RMLK_ERR_UNSUPPORTED;   // Softmax over nothing: left to the separate kernels
    if (!q || !k || !v || !mask || !out) return RMLK_ERR_NULL_POINTER;
    for (int d = 0; d < 4; ++d)
        if (mask_stride->v[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (mask_stride->v[3] != 1) return RMLK_ERR_UNSUPPORTED;
    // 128-bit mask loads where the kernel makes them
    if (vector_mask && (kv_len % 4 != 0 || mask_stride->v[0] % 4 != 0 || mask_stride->v[1] % 4 != 0 ||
                        mask_stride->v[2] % 4 != 0 || reinterpret_cast<uintptr_t>(mask) % 16))
        return RMLK_ERR_UNSUPPORTED;
    // 32-bit byte offsets into one KV head, grid limits
    if (kv_len * kHeadDim >= (1ll << 29) || rows >= (1ll << 30) || batch * kv_heads >= 65536)
        return RMLK_ERR_UNSUPPORTED;
    if (reinterpret_cast<uintptr_t>(q) % 16 || reinterpret_cast<uintptr_t>(k) % 16 ||
        reinterpret_cast<uintptr_t>(v) % 16 || reinterpret_cast<uintptr_t>(out) % 16)
        return RMLK_ERR_UNSUPPORTED;
    if (scale_is_mul == 0 && scale == 0.f) return RMLK_ERR_UNSUPPORTED;   // x / 0: not this kernel's case
    AttnArgs g{};
    g.q = static_cast<const float *>(q);
    g.k = static_cast<const float *>(k);
    g.v = static_cast<const float *>(v);
    g.mask = static_cast<const float *>(mask);
    g.out = static_cast<float *>(out);
    g.rows = static_cast<int32_t>(rows);
    g.seq = static_cast<int32_t>(q_len);
    g.rep = static_cast<int32_t>(rep);
    g.kv_heads = static_cast<int32_t>(kv_heads);
    g.len = static_cast<int32_t>(kv_len);
    g.mask_b = mask_stride->v[0];
    g.mask_h = mask_stride->v[1];
    g.mask_s = mask_stride->v[2];
    g.qscale = scale_is_mul ? scale : 1.0f / scale;
    const int64_t heads = kv_heads * rep;
    if (out_seq_major) {   // [batch, q_len, heads, head_dim]
        g.out_b = q_len * heads * kHeadDim;
        g.out_s = heads * kHeadDim;
        g.out_h = kHeadDim;
    } else {               // [batch, heads, q_len, head_dim]
        g.out_b = heads * q_len * kHeadDim;
        g.out_h = q_len * kHeadDim;
        g.out_s = kHeadDim;
    }
    *args = g;
    return RMLK_OK;
}

}  // namespace

namespace {
// The tile map of masked-chunk skipping: dims and bytes, or 0 bytes when skipping does not apply -
// the blocks must outnumber the compute units (otherwise the block with the most visible chunks
// decides and nothing is gained; it is also the case that runs 64-key chunks), a query tile must
// lie inside one head, and the chunks must fit the kernel's two 64-bit sets.
struct TileMapDims {
    int64_t mask_batches, mask_heads, tiles, chunks;
    int keys;   // keys of a chunk: what the kernel that will run takes per step
    size_t map_bytes, bytes;
};
// shared: the map serves several launches over one mask (the layers of a model), so making it is
// no cost to weigh against what one launch skips: two chunks are enough.
TileMapDims tile_map_dims(int64_t batch, int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                          const rmlk_dims *mask_stride, bool shared = false) {
    TileMapDims d{};
    if (batch <= 0 || kv_heads <= 0 || rep <= 0 || q_len <= 0 || kv_len <= 0 || !dims_ok(mask_stride) ||
        mask_stride->rank != 4)
        return d;
    const int64_t blocks = (rep * q_len + 63) / 64 * batch * kv_heads;
    // More blocks than compute units: the kernel with 64-key steps, its items handed out from a
    // counter. Otherwise the kernel with 128-key steps and one block per tile, which keeps its tile and
    // only skips the chunks it cannot see: that pays where a prompt is much shorter than its cache.
    const bool many_blocks = blocks > kNumCU;
    d.keys = many_blocks ? AttnShape<2>::kKeys : AttnShape<4>::kKeys;
    d.chunks = (kv_len + d.keys - 1) / d.keys;
    if (q_len % 64 != 0 || d.chunks < (shared ? 2 : many_blocks ? 4 : 6) || d.chunks > 128) return d;
    d.mask_batches = mask_stride->v[0] ? batch : 1;
    d.mask_heads = mask_stride->v[1] ? kv_heads * rep : 1;
    d.tiles = q_len / 64;
    if (d.mask_batches * d.mask_heads >= 65536 || d.tiles >= 65536) return d;
    d.map_bytes = static_cast<size_t>(d.mask_batches * d.mask_heads * d.tiles * d.chunks + 15) / 16 * 16;
    d.bytes = d.map_bytes + 16;   // the map, then the item counter
    return d;
}
}  // namespace

extern "C" size_t rmlk_hip_attention_workspace_size(int32_t dtype, int64_t batch, int64_t kv_heads,
                                                    int64_t rep, int64_t q_len, int64_t kv_len,
                                                    int64_t head_dim, const rmlk_dims *mask_stride) {
    if (dtype != RMLK_FLOAT || head_dim != kHeadDim) return 0;
    return tile_map_dims(batch, kv_heads, rep, q_len, kv_len, mask_stride).bytes;
}

namespace {
int32_t attention_many_rows(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads, int64_t rep,
                            int64_t q_len, int64_t kv_len, int64_t head_dim, const void *q, const void *k,
                            const void *v, const void *mask, const rmlk_dims *mask_stride, int32_t scale_is_mul,
                            float scale, int32_t out_seq_major, void *workspace, size_t workspace_bytes, void *out,
                            void *out_pieces, int map_state = 0) {
    // map_state 0: the workspace is room for a map that this call makes and uses; 1: only make the
    // shared map (no attention launch); 2: the workspace holds a shared map made by state 1
    AttnArgs g{};
    bool empty = false;
    const int32_t st = attention_args(dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                                      mask_stride, scale_is_mul, scale, out_seq_major, out, true, &g, &empty);
    if (st || empty) return st;
    if (map_state != 0) {
        const TileMapDims tm = tile_map_dims(batch, kv_heads, rep, q_len, kv_len, mask_stride, true);
        if (!tm.bytes) return RMLK_ERR_UNSUPPORTED;
        if (!workspace || workspace_bytes < tm.bytes || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
            return RMLK_ERR_WORKSPACE;
    }
    if (out_pieces) {
        // the pieces of the [batch * q_len, heads * head_dim] matrix that a [B, S, H, D] result is
        if (!out_seq_major || reinterpret_cast<uintptr_t>(out_pieces) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
        const int64_t rows = batch * q_len, m_pad = (rows + 127) / 128 * 128;
        g.pieces = static_cast<uint16_t *>(out_pieces);
        g.plane = m_pad * kv_heads * rep * head_dim;
    }
    dim3 grid(static_cast<unsigned>((g.rows + 63) / 64), static_cast<unsigned>(batch * kv_heads), 1);
    const bool many_blocks = static_cast<int64_t>(grid.x) * grid.y > kNumCU;
    {
        const TileMapDims tm = tile_map_dims(batch, kv_heads, rep, q_len, kv_len, mask_stride, map_state != 0);
        if (workspace && tm.bytes && workspace_bytes >= tm.bytes && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
            uint8_t *tiles = static_cast<uint8_t *>(workspace);
            const dim3 tgrid(static_cast<unsigned>(tm.chunks), static_cast<unsigned>(tm.tiles),
                             static_cast<unsigned>(tm.mask_batches * tm.mask_heads));
            if (map_state == 2) {
                // made by an earlier call; its counter is zero again
            } else if (tm.keys == 64)
                attention_mask_tiles_kernel<64><<<tgrid, 256, 0, as_stream(stream)>>>(
                    g.mask, g.mask_b, g.mask_h, g.mask_s, static_cast<int32_t>(tm.mask_heads), g.seq, g.len, tiles,
                    reinterpret_cast<int32_t *>(tiles + tm.map_bytes));
            else
                attention_mask_tiles_kernel<128><<<tgrid, 256, 0, as_stream(stream)>>>(
                    g.mask, g.mask_b, g.mask_h, g.mask_s, static_cast<int32_t>(tm.mask_heads), g.seq, g.len, tiles,
                    reinterpret_cast<int32_t *>(tiles + tm.map_bytes));
            const int32_t launched = launch_status();
            if (launched || map_state == 1) return launched;
            g.tiles = tiles;
            g.tiles_h = mask_stride->v[1] ? tm.tiles * tm.chunks : 0;
            g.tiles_b = mask_stride->v[0] ? tm.mask_heads * tm.tiles * tm.chunks : 0;
            if (many_blocks) {
                // (tile, KV head) items handed to a resident grid from a counter, longest first
                g.queue = reinterpret_cast<int32_t *>(tiles + tm.map_bytes);
                g.items = static_cast<int32_t>(static_cast<int64_t>(grid.x) * grid.y);
                g.tiles_per_head = static_cast<int32_t>(tm.tiles);
                grid = dim3(static_cast<unsigned>(std::min<int64_t>(g.items, 2 * kNumCU)), 1, 1);
            }
        }
    }
    // two blocks of four wavefronts per CU when there are that many, else one block of eight
    auto launch = [&](auto nk_tag, auto whole_tag, auto paired_tag) -> int32_t {
        constexpr int NK = decltype(nk_tag)::value;
        constexpr bool WHOLE = decltype(whole_tag)::value, PAIRED = decltype(paired_tag)::value;
        static DynamicLdsGrant grant;
        const int32_t granted = grant.ensure(attention_rows_kernel<NK, WHOLE, PAIRED>, AttnShape<NK>::kLdsBytes);
        if (granted) return granted;
        attention_rows_kernel<NK, WHOLE, PAIRED>
            <<<grid, AttnShape<NK>::kThreads, AttnShape<NK>::kLdsBytes, as_stream(stream)>>>(g);
        return launch_status();
    };
    using Two = std::integral_constant<int, 2>;
    using Four = std::integral_constant<int, 4>;
    const std::true_type yes{};
    const std::false_type no{};
    if (many_blocks) return kv_len % AttnShape<2>::kKeys == 0 ? launch(Two{}, yes, no) : launch(Two{}, no, no);
    // one block per tile and a map: the blocks take halves of two tiles each (an even number of tiles per head)
    if (g.tiles && !g.queue && q_len % 128 == 0) {
        g.tiles_per_head = static_cast<int32_t>(q_len / 64);
        return kv_len % AttnShape<4>::kKeys == 0 ? launch(Four{}, yes, yes) : launch(Four{}, no, yes);
    }
    return kv_len % AttnShape<4>::kKeys == 0 ? launch(Four{}, yes, no) : launch(Four{}, no, no);
}
}  // namespace

extern "C" int32_t rmlk_hip_attention_ws(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                         int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                         int64_t head_dim, const void *q, const void *k, const void *v,
                                         const void *mask, const rmlk_dims *mask_stride,
                                         int32_t scale_is_mul, float scale, int32_t out_seq_major,
                                         void *workspace, size_t workspace_bytes, void *out) {
    return attention_many_rows(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                               mask_stride, scale_is_mul, scale, out_seq_major, workspace, workspace_bytes, out,
                               nullptr);
}

extern "C" int32_t rmlk_hip_attention_ws_pieces(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                                int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                                int64_t head_dim, const void *q, const void *k, const void *v,
                                                const void *mask, const rmlk_dims *mask_stride,
                                                int32_t scale_is_mul, float scale, void *workspace,
                                                size_t workspace_bytes, void *out, void *out_pieces) {
    if (!out_pieces) return RMLK_ERR_NULL_POINTER;
    return attention_many_rows(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                               mask_stride, scale_is_mul, scale, 1, workspace, workspace_bytes, out, out_pieces);
}

extern "C" size_t rmlk_hip_attention_map_size(int32_t dtype, int64_t batch, int64_t kv_heads, int64_t rep,
                                              int64_t q_len, int64_t kv_len, int64_t head_dim,
                                              const rmlk_dims *mask_stride) {
    if (dtype != RMLK_FLOAT || head_dim != kHeadDim) return 0;
    return tile_map_dims(batch, kv_heads, rep, q_len, kv_len, mask_stride, true).bytes;
}

extern "C" int32_t rmlk_hip_attention_map(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                                          int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                                          const void *mask, const rmlk_dims *mask_stride, void *map,
                                          size_t map_bytes) {
    // (q, k, v and out only have to pass the argument checks: the map is made of the mask alone)
    return attention_many_rows(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, mask, mask, mask, mask,
                               mask_stride, 1, 1.0f, 0, map, map_bytes, const_cast<void *>(mask), nullptr, 1);
}

extern "C" int32_t rmlk_hip_attention_mapped(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                                             int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim,
                                             const void *q, const void *k, const void *v, const void *mask,
                                             const rmlk_dims *mask_stride, int32_t scale_is_mul, float scale,
                                             int32_t out_seq_major, const void *map, size_t map_bytes, void *out) {
    return attention_many_rows(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                               mask_stride, scale_is_mul, scale, out_seq_major, const_cast<void *>(map), map_bytes,
                               out, nullptr, 2);
}

extern "C" int32_t rmlk_hip_attention_mapped_pieces(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                                    int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                                    int64_t head_dim, const void *q, const void *k, const void *v,
                                                    const void *mask, const rmlk_dims *mask_stride,
                                                    int32_t scale_is_mul, float scale, const void *map,
                                                    size_t map_bytes, void *out, void *out_pieces) {
    if (!out_pieces) return RMLK_ERR_NULL_POINTER;
    return attention_many_rows(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                               mask_stride, scale_is_mul, scale, 1, const_cast<void *>(map), map_bytes, out,
                               out_pieces, 2);
}

extern "C" int32_t rmlk_hip_attention(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                      int64_t kv_heads, int64_t rep, int64_t q_len, int64_t kv_len,
                                      int64_t head_dim, const void *q, const void *k, const void *v,
                                      const void *mask, const rmlk_dims *mask_stride,
                                      int32_t scale_is_mul, float scale, int32_t out_seq_major,
                                      void *out) {
    return rmlk_hip_attention_ws(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                                 mask_stride, scale_is_mul, scale, out_seq_major, nullptr, 0, out);
}

extern "C" size_t rmlk_hip_attention_few_rows_workspace_size(int32_t dtype, int64_t batch, int64_t kv_heads,
                                                             int64_t rep, int64_t q_len, int64_t kv_len,
                                                             int64_t head_dim) {
    if (dtype != RMLK_FLOAT || head_dim != kHeadDim || batch <= 0 || kv_heads <= 0 || rep <= 0 ||
        q_len <= 0 || kv_len <= 0 || rep * q_len > kFewRowsMax)
        return 0;
    const int64_t chunks = (kv_len + kChunk - 1) / kChunk;
    return static_cast<size_t>(batch * kv_heads * chunks * rep * q_len * kPartial) * sizeof(float);
}

namespace {
int32_t attention_few_rows_launch(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t kv_heads,
                                  int64_t rep, int64_t q_len, int64_t kv_len, int64_t head_dim, const void *q,
                                  const void *k, const void *v, const void *mask, const rmlk_dims *mask_stride,
                                  int32_t scale_is_mul, float scale, int32_t out_seq_major, void *workspace,
                                  size_t workspace_bytes, int32_t *counters, void *out) {
    AttnArgs g{};
    bool empty = false;
    const int32_t st = attention_args(dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                                      mask_stride, scale_is_mul, scale, out_seq_major, out, false, &g, &empty);
    if (st || empty) return st;
    if (g.rows > kFewRowsMax) return RMLK_ERR_UNSUPPORTED;
    const size_t need = rmlk_hip_attention_few_rows_workspace_size(dtype, batch, kv_heads, rep, q_len, kv_len,
                                                                   head_dim);
    if (!workspace || workspace_bytes < need) return RMLK_ERR_WORKSPACE;
    const int64_t chunks = (kv_len + kChunk - 1) / kChunk;
    if (chunks >= (1ll << 31)) return RMLK_ERR_TOO_LARGE;
    hipStream_t s = as_stream(stream);
    float *ws = static_cast<float *>(workspace);
    dim3 grid(static_cast<unsigned>(chunks), static_cast<unsigned>(batch * kv_heads), 1);
    if (counters) {
        attention_few_rows_kernel<true><<<grid, kAttnThreads, 0, s>>>(g, ws, scale, scale_is_mul, counters);
        return launch_status();
    }
    attention_few_rows_kernel<false><<<grid, kAttnThreads, 0, s>>>(g, ws, scale, scale_is_mul, nullptr);
    int32_t launched = launch_status();
    if (launched) return launched;
    const int64_t total_rows = batch * kv_heads * g.rows;
    constexpr int kWaves = kAttnThreads / kWave;
    const unsigned merge_grid = static_cast<unsigned>((total_rows + kWaves - 1) / kWaves);
    if (chunks <= kMergeMaxChunks)
        attention_merge_kernel<<<merge_grid, kAttnThreads, 0, s>>>(g, ws, static_cast<int32_t>(chunks),
                                                                   static_cast<int32_t>(total_rows));
    else
        attention_merge_many_kernel<<<merge_grid, kAttnThreads, 0, s>>>(g, ws, static_cast<int32_t>(chunks),
                                                                        static_cast<int32_t>(total_rows));
    return launch_status();
}
}  // namespace

extern "C" int32_t rmlk_hip_attention_few_rows(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                               int64_t kv_heads, int64_t rep, int64_t q_len,
                                               int64_t kv_len, int64_t head_dim, const void *q,
                                               const void *k, const void *v, const void *mask,
                                               const rmlk_dims *mask_stride, int32_t scale_is_mul,
                                               float scale, int32_t out_seq_major, void *workspace,
                                               size_t workspace_bytes, void *out) {
    return attention_few_rows_launch(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                                     mask_stride, scale_is_mul, scale, out_seq_major, workspace, workspace_bytes,
                                     nullptr, out);
}

extern "C" int32_t rmlk_hip_attention_few_rows_one_launch(rmlk_stream_t stream, int32_t dtype, int64_t batch,
                                                          int64_t kv_heads, int64_t rep, int64_t q_len,
                                                          int64_t kv_len, int64_t head_dim, const void *q,
                                                          const void *k, const void *v, const void *mask,
                                                          const rmlk_dims *mask_stride, int32_t scale_is_mul,
                                                          float scale, int32_t out_seq_major, void *workspace,
                                                          size_t workspace_bytes, int32_t *counters, void *out) {
    if (!counters) return RMLK_ERR_NULL_POINTER;
    return attention_few_rows_launch(stream, dtype, batch, kv_heads, rep, q_len, kv_len, head_dim, q, k, v, mask,
                                     mask_stride, scale_is_mul, scale, out_seq_major, workspace, workspace_bytes,
                                     counters, out);
}
