// Data-movement ops: Transpose, Expand, Slice, Concat, Gather, ScatterND, Trilu.
// All of them are moves of opaque 1/2/4/8-byte elements, so kernels are instantiated per access
// width. The strided N-d copy re-types a contiguous innermost run into the widest unit (up to
// 128 bits) that divides the run, the outer strides and the pointer alignments.
//
// Replaces cuda/src/ptx/{transpose,expand,slice,scatter_nd,trilu}.cu and the host memcpy loops of
// runtime/src/providers/cuda/backend/{gather,concat}.rs in the reference.
#include "batch.hpp"
#include "nd_index.hpp"

namespace rmlk {
namespace {

constexpr int kBlock = 256;

struct alignas(16) U128 {
    uint32_t w[4];
};

// ---------------------------------------------------------------------------------------------
// strided N-d copy: plan operand 0 = in, 1 = out
constexpr int kUnroll = 4;  // independent accesses in flight per lane
constexpr int kChunk = kBlock * kUnroll;      // units a block takes per trip, consecutive in the output

// Sources are read once and results are not found in a cache by whoever reads them next (the L2s of
// the eight XCDs are written back at the end of a kernel): streaming loads and stores.
template <typename U>
__device__ __forceinline__ void put(U *p, const U &v) {
    nt_store(p, v);
}

// REPEATS: the input is read more than once (repeated along some dim, as Expand's): ordinary loads
template <bool REPEATS, typename U>
__device__ __forceinline__ U get(const U *p) {
    if constexpr (REPEATS) return *p;
    else return nt_load(p);
}

template <typename OFF, typename PL>
__device__ __forceinline__ void copy_offsets(const PL &pl, uint32_t i, OFF (&offs)[2]) {
    if constexpr (std::is_same<PL, NdIndex4<2>>::value) nd4_offsets<2>(pl, i, offs);
    else nd_offsets<2>(pl, i, offs);
}

// PL: NdIndex4<2> (at most four dims, 32-bit offsets, a dense side free of index arithmetic) or the
// full NdPlan<2>.
template <typename U, bool REPEATS, typename PL>
__global__ __launch_bounds__(kBlock) void copy_nd_kernel(PL pl, const U *__restrict__ in,
                                                         U *__restrict__ out, uint32_t n) {
    using OFF = std::conditional_t<std::is_same<PL, NdIndex4<2>>::value, int32_t, int64_t>;
    // one trip: the grid covers n in chunks (no loop for the compiler to hoist the index choices out of)
    const uint32_t base = blockIdx.x * kChunk;
    const uint32_t i0 = base + threadIdx.x;
    if (base + kChunk <= n) {
        U r[kUnroll];
        OFF oo[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            OFF offs[2];
            copy_offsets(pl, i0 + j * kBlock, offs);
            r[j] = get<REPEATS>(in + offs[0]);
            oo[j] = offs[1];
        }
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) put(out + oo[j], r[j]);
    } else {
        for (uint32_t i = i0; i < n; i += kBlock) {
            OFF offs[2];
            copy_offsets(pl, i, offs);
            put(out + offs[1], get<REPEATS>(in + offs[0]));
        }
    }
}

// dense flat copy of n units
template <typename U>
__global__ __launch_bounds__(kBlock) void copy_flat_kernel(const U *__restrict__ in,
                                                           U *__restrict__ out, uint32_t n) {
    for (uint32_t base = blockIdx.x * kChunk; base < n; base += gridDim.x * kChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kChunk <= n) {
            U r[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) r[j] = nt_load(in + i0 + j * kBlock);
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) put(out + i0 + j * kBlock, r[j]);
        } else {
            for (uint32_t i = i0; i < n; i += kBlock) put(out + i, nt_load(in + i));
        }
    }
}

// several dense flat copies in one launch: blockIdx.y picks the copy
constexpr int kMaxCopies = 32;
struct CopyMany {
    const U128 *in[kMaxCopies];
    U128 *out[kMaxCopies];
    uint32_t n[kMaxCopies];   // units
};
__global__ __launch_bounds__(kBlock) void copy_many_kernel(CopyMany a) {
    const U128 *__restrict__ in = a.in[blockIdx.y];
    U128 *__restrict__ out = a.out[blockIdx.y];
    const uint32_t n = a.n[blockIdx.y];
    for (uint32_t base = blockIdx.x * kChunk; base < n; base += gridDim.x * kChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kChunk <= n) {
            U128 r[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) r[j] = nt_load(in + i0 + j * kBlock);
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) put(out + i0 + j * kBlock, r[j]);
        } else {
            for (uint32_t i = i0; i < n; i += kBlock) put(out + i, nt_load(in + i));
        }
    }
}

template <typename U>
int32_t launch_copy_units(hipStream_t s, NdPlan<2> &pl, const void *in, void *out) {
    uint32_t n = static_cast<uint32_t>(pl.numel);
    unsigned grid = chunk_grid(n, kChunk);
    if (pl.rank == 1 && pl.stride[0][0] == 1 && pl.stride[1][0] == 1) {
        copy_flat_kernel<U><<<grid, kBlock, 0, s>>>(static_cast<const U *>(in),
                                                    static_cast<U *>(out), n);
    } else {
        bool repeats = false;
        for (int d = 0; d < pl.rank; ++d)
            if (pl.stride[0][d] == 0 && pl.dim64[d] > 1) repeats = true;
        const U *pi = static_cast<const U *>(in);
        U *po = static_cast<U *>(out);
        grid = (n + kChunk - 1) / kChunk;      // one trip
        NdIndex4<2> ix;
        const int unit_shift[2] = {0, 0};
        if (make_index4<2>(ix, pl, unit_shift, -1, 0)) {
            if (repeats) copy_nd_kernel<U, true, NdIndex4<2>><<<grid, kBlock, 0, s>>>(ix, pi, po, n);
            else copy_nd_kernel<U, false, NdIndex4<2>><<<grid, kBlock, 0, s>>>(ix, pi, po, n);
        } else {
            if (repeats) copy_nd_kernel<U, true, NdPlan<2>><<<grid, kBlock, 0, s>>>(pl, pi, po, n);
            else copy_nd_kernel<U, false, NdPlan<2>><<<grid, kBlock, 0, s>>>(pl, pi, po, n);
        }
    }
    return launch_status();
}

// One launch of the strided copy on < 2^30 elements. Byte pointers, element strides.
int32_t strided_copy_piece(hipStream_t s, int esize, int rank, const int64_t *shape,
                           const int64_t (*strides)[kMaxRank], const char *in, char *out) {
    NdPlan<2> pl;
    if (!build_plan<2>(pl, rank, shape, strides)) return RMLK_OK;
    const int last = pl.rank - 1;
    int unit = esize;
    if (pl.stride[0][last] == 1 && pl.stride[1][last] == 1) {
        int64_t run_bytes = pl.dim64[last] * esize;
        for (int cand = 16; cand > esize; cand >>= 1) {
            bool ok = run_bytes % cand == 0 && reinterpret_cast<uintptr_t>(in) % cand == 0 &&
                      reinterpret_cast<uintptr_t>(out) % cand == 0;
            for (int d = 0; d < last && ok; ++d)
                for (int p = 0; p < 2; ++p)
                    if ((static_cast<int64_t>(pl.stride[p][d]) * esize) % cand) ok = false;
            if (ok) { unit = cand; break; }
        }
        if (unit != esize) {
            int f = unit / esize;
            pl.dim64[last] /= f;
            pl.dim[last] = static_cast<uint32_t>(pl.dim64[last]);
            pl.fdiv[last] = FastDiv(pl.dim[last]);
            for (int d = 0; d < last; ++d)
                for (int p = 0; p < 2; ++p) pl.stride[p][d] /= f;
            pl.numel /= f;
        }
    }
    switch (unit) {
        case 1: return launch_copy_units<uint8_t>(s, pl, in, out);
        case 2: return launch_copy_units<uint16_t>(s, pl, in, out);
        case 4: return launch_copy_units<uint32_t>(s, pl, in, out);
        case 8: return launch_copy_units<uint64_t>(s, pl, in, out);
        default: return launch_copy_units<U128>(s, pl, in, out);
    }
}

// Strided copy of any size: pieces that the kernels' 32-bit index math can address.
int32_t strided_copy(hipStream_t s, int esize, int rank, const int64_t *shape,
                     const int64_t (*strides)[kMaxRank], const void *in, void *out) {
    const char *pin = static_cast<const char *>(in);
    char *pout = static_cast<char *>(out);
    int64_t zero[2] = {0, 0};
    return split_pieces<2>(rank, shape, strides, zero,
                           [&](const int64_t *shp, const int64_t *offs) {
                               return strided_copy_piece(s, esize, rank, shp, strides,
                                                         pin + offs[0] * esize,
                                                         pout + offs[1] * esize);
                           });
}

// ---------------------------------------------------------------------------------------------
// Tiled transpose through LDS. The logical space is the OUTPUT shape after coalescing; dim `last`
// is contiguous in the output, dim `q` is contiguous in the input. A block moves a 64 x 64 tile
// over (q, last): wave-wide reads run along q, wave-wide writes run along last, and the tile is
// padded by one column so neither side hits the same LDS bank twice.
struct TilePlan {
    int32_t n_batch_dims;
    uint32_t bdim[kMaxRank];
    FastDiv bdiv[kMaxRank];
    int64_t b_in[kMaxRank];   // in / out element strides of the batch dims
    int64_t b_out[kMaxRank];
    uint32_t q_len, l_len;    // extents of the two tiled dims
    uint32_t q_tiles, l_tiles;
    FastDiv q_tiles_div, l_tiles_div;
    int64_t l_in_stride;      // input stride of dim `last` (input stride of q is 1)
    int64_t q_out_stride;     // output stride of dim q (output stride of last is 1)
};

constexpr int kTile = 64;

template <typename U>
__global__ __launch_bounds__(kBlock) void transpose_tile_kernel(TilePlan tp,
                                                                const U *__restrict__ in,
                                                                U *__restrict__ out) {
    __shared__ U tile[kTile][kTile + 1];
    uint32_t b = blockIdx.x;
    uint32_t t = tp.l_tiles_div.div(b);
    const uint32_t lt = b - t * tp.l_tiles;
    b = t;
    t = tp.q_tiles_div.div(b);
    const uint32_t qt = b - t * tp.q_tiles;
    b = t;
    int64_t in_off = 0, out_off = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; --d) {
        if (d < tp.n_batch_dims) {
            uint32_t qd = tp.bdiv[d].div(b);
            uint32_t i = b - qd * tp.bdim[d];
            b = qd;
            in_off += static_cast<int64_t>(i) * tp.b_in[d];
            out_off += static_cast<int64_t>(i) * tp.b_out[d];
        }
    }
    const uint32_t lane = threadIdx.x & (kTile - 1);
    const uint32_t wrow = threadIdx.x / kTile;  // 0..3
    const uint32_t q0 = qt * kTile, l0 = lt * kTile;
    // read: lane runs along q, rows along last
#pragma unroll 4
    for (uint32_t r = wrow; r < kTile; r += kBlock / kTile) {
        uint32_t l = l0 + r, q = q0 + lane;
        if (l < tp.l_len && q < tp.q_len)
            tile[r][lane] = in[in_off + static_cast<int64_t>(l) * tp.l_in_stride + q];
    }
    __syncthreads();
    // write: lane runs along last, rows along q
#pragma unroll 4
    for (uint32_t r = wrow; r < kTile; r += kBlock / kTile) {
        uint32_t q = q0 + r, l = l0 + lane;
        if (q < tp.q_len && l < tp.l_len)
            out[out_off + static_cast<int64_t>(q) * tp.q_out_stride + l] = tile[lane][r];
    }
}

template <typename U>
int32_t launch_tile(hipStream_t s, const TilePlan &tp, uint64_t blocks, const void *in, void *out) {
    transpose_tile_kernel<U><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(
        tp, static_cast<const U *>(in), static_cast<U *>(out));
    return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Gather rows. Units of `U`; a row is `row_units` units. out row r = (outer, j) takes data row
// (outer * axis_dim + idx[j]).
template <typename U, typename I>
__device__ __forceinline__ U gather_fetch(const U *__restrict__ data, const I *__restrict__ idx,
                                          uint32_t e, uint32_t row_units, FastDiv row_div,
                                          uint32_t n_idx, FastDiv idx_div, int64_t axis_dim,
                                          int32_t *__restrict__ err) {
    const uint32_t row = row_div.div(e);
    const uint32_t c = e - row * row_units;
    const uint32_t outer = idx_div.div(row);
    const uint32_t jj = row - outer * n_idx;
    int64_t ix = static_cast<int64_t>(idx[jj]);
    if (ix < 0) ix += axis_dim;
    if (ix < 0 || ix >= axis_dim) {
        if (err) *err = 1;
        return U{};
    }
    return nt_load(data + (static_cast<int64_t>(outer) * axis_dim + ix) * row_units + c);
}

template <typename U, typename I>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(const U *__restrict__ data,
                                                             const I *__restrict__ idx,
                                                             U *__restrict__ out, uint32_t n_units,
                                                             uint32_t row_units, FastDiv row_div,
                                                             uint32_t n_idx, FastDiv idx_div,
                                                             int64_t axis_dim,
                                                             int32_t *__restrict__ err) {
    for (uint32_t base = blockIdx.x * kChunk; base < n_units; base += gridDim.x * kChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kChunk <= n_units) {
            // the index loads of all kUnroll units, then their data loads, then the stores: each
            // group is in flight together (a fetch at a time would wait for an index, then for its
            // data, kUnroll times over)
            U r[kUnroll];
            I raw[kUnroll];
            uint32_t col[kUnroll], outer[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                const uint32_t e = i0 + j * kBlock;
                const uint32_t row = row_div.div(e);
                col[j] = e - row * row_units;
                outer[j] = idx_div.div(row);
                raw[j] = idx[row - outer[j] * n_idx];
            }
            bool ok[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                int64_t ix = static_cast<int64_t>(raw[j]);
                if (ix < 0) ix += axis_dim;
                ok[j] = ix >= 0 && ix < axis_dim;
                if (!ok[j]) ix = 0;
                r[j] = nt_load(data + (static_cast<int64_t>(outer[j]) * axis_dim + ix) * row_units + col[j]);
            }
#pragma unroll
            for (int j = 0; j < kUnroll; ++j) {
                if (!ok[j]) {
                    r[j] = U{};
                    if (err) *err = 1;
                }
                put(out + i0 + j * kBlock, r[j]);
            }
        } else {
            for (uint32_t i = i0; i < n_units; i += kBlock)
                put(out + i, gather_fetch<U, I>(data, idx, i, row_units, row_div, n_idx, idx_div, axis_dim, err));
        }
    }
}

template <typename U>
int32_t launch_gather(hipStream_t s, int32_t idx_dtype, const void *data, const void *idx,
                      void *out, uint32_t n_units, uint32_t row_units, uint32_t n_idx,
                      int64_t axis_dim, int32_t *err) {
    unsigned grid = chunk_grid(n_units, kChunk);
    FastDiv rd(row_units), id(n_idx);
    if (idx_dtype == RMLK_INT64)
        gather_rows_kernel<U, int64_t><<<grid, kBlock, 0, s>>>(
            static_cast<const U *>(data), static_cast<const int64_t *>(idx), static_cast<U *>(out),
            n_units, row_units, rd, n_idx, id, axis_dim, err);
    else
        gather_rows_kernel<U, int32_t><<<grid, kBlock, 0, s>>>(
            static_cast<const U *>(data), static_cast<const int32_t *>(idx), static_cast<U *>(out),
            n_units, row_units, rd, n_idx, id, axis_dim, err);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------
// ScatterND
struct ScatterPlan {
    int32_t tuple_size;
    int64_t dim[kMaxRank];
    int64_t stride[kMaxRank];  // in units of one slice element
};

template <int RED, typename T>
__device__ __forceinline__ T red_apply(T in, T cur) {
    if constexpr (RED == RMLK_SCATTER_ADD) return cur + in;
    else if constexpr (RED == RMLK_SCATTER_MUL) return cur * in;
    else if constexpr (RED == RMLK_SCATTER_MAX) return in > cur ? in : cur;
    else return in < cur ? in : cur;
}

template <typename T>
struct BitsOf;
template <>
struct BitsOf<float> { using type = unsigned int; };
template <>
struct BitsOf<int32_t> { using type = unsigned int; };
template <>
struct BitsOf<double> { using type = unsigned long long; };
template <>
struct BitsOf<int64_t> { using type = unsigned long long; };

template <int RED, typename T>
__device__ __forceinline__ void atomic_reduce(T *addr, T in) {
    using B = typename BitsOf<T>::type;
    B *baddr = reinterpret_cast<B *>(addr);
    B old = *baddr, assumed;
    do {
        assumed = old;
        T cur;
        __builtin_memcpy(&cur, &assumed, sizeof(T));
        T nv = red_apply<RED, T>(in, cur);
        B nb;
        __builtin_memcpy(&nb, &nv, sizeof(T));
        old = atomicCAS(baddr, assumed, nb);
    } while (old != assumed);
}

// RED == NONE moves units of U; otherwise T is the arithmetic type.
template <int RED, typename T>
__global__ __launch_bounds__(kBlock) void scatter_nd_kernel(ScatterPlan sp,
                                                            const int64_t *__restrict__ idx,
                                                            const T *__restrict__ upd,
                                                            T *__restrict__ out, uint32_t n_units,
                                                            uint32_t slice_units, FastDiv slice_div,
                                                            int32_t *__restrict__ err) {
    const uint32_t step = gridDim.x * kBlock;
    for (uint32_t e = blockIdx.x * kBlock + threadIdx.x; e < n_units; e += step) {
        uint32_t tup = slice_div.div(e);
        uint32_t c = e - tup * slice_units;
        int64_t off = 0;
        bool bad = false;
#pragma unroll
        for (int t = 0; t < kMaxRank; ++t) {
            if (t < sp.tuple_size) {
                int64_t ix = idx[static_cast<int64_t>(tup) * sp.tuple_size + t];
                if (ix < 0) ix += sp.dim[t];
                if (ix < 0 || ix >= sp.dim[t]) bad = true;
                off += ix * sp.stride[t];
            }
        }
        if (bad) {
            if (err) *err = 1;
            continue;
        }
        if constexpr (RED == RMLK_SCATTER_NONE) {
            out[off * slice_units + c] = upd[e];
        } else {
            atomic_reduce<RED, T>(out + off * slice_units + c, upd[e]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// ScatterND with ONNX copy semantics in one launch: out = data, except for the slices the index
// tuples address, which come from `updates`. For few tuples (at most a wavefront's lanes): every
// wavefront lets lane t work out where tuple t lands, a ballot says which of them touch the block's
// chunk (mostly none), and a unit inside such a slice is read from the updates instead of the data.
// Later tuples win over earlier ones, as a sequential scatter would have it.
constexpr uint32_t kMaxFusedTuples = kWave;

__global__ __launch_bounds__(kBlock) void scatter_copy_kernel(ScatterPlan sp,
                                                              const int64_t *__restrict__ idx,
                                                              const U128 *__restrict__ upd,
                                                              const U128 *__restrict__ data,
                                                              U128 *__restrict__ out, uint32_t n,
                                                              uint32_t n_tuples, uint32_t slice_units,
                                                              int32_t *__restrict__ err) {
    const uint32_t base = blockIdx.x * kChunk;
    const uint32_t lane = threadIdx.x % kWave;
    // lane t: first unit of the slice of tuple t
    uint32_t start = 0;
    bool valid = false;
    if (lane < n_tuples) {
        int64_t off = 0;
        bool bad = false;
#pragma unroll
        for (int t = 0; t < kMaxRank; ++t) {
            if (t < sp.tuple_size) {
                int64_t ix = idx[static_cast<int64_t>(lane) * sp.tuple_size + t];
                if (ix < 0) ix += sp.dim[t];
                if (ix < 0 || ix >= sp.dim[t]) bad = true;
                off += ix * sp.stride[t];
            }
        }
        if (bad) {
            if (err && blockIdx.x == 0 && threadIdx.x < kWave) *err = 1;
        } else {
            valid = true;
            start = static_cast<uint32_t>(off) * slice_units;
        }
    }
    const uint32_t chunk_end = base + kChunk < n ? base + kChunk : n;
    const bool touches = valid && start < chunk_end && start + slice_units > base;
    uint64_t hits = __ballot(touches);
    U128 r[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const uint32_t i = base + threadIdx.x + j * kBlock;
        if (i < n) r[j] = nt_load(data + i);
    }
    while (hits) {       // uniform; ascending tuple order, so the last one to address a unit wins
        const int t = __builtin_ctzll(hits);
        hits &= hits - 1;
        const uint32_t s0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(start), t));
#pragma unroll
        for (int j = 0; j < kUnroll; ++j) {
            const uint32_t i = base + threadIdx.x + j * kBlock;
            if (i < n && i >= s0 && i - s0 < slice_units)
                r[j] = upd[static_cast<uint64_t>(t) * slice_units + (i - s0)];
        }
    }
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const uint32_t i = base + threadIdx.x + j * kBlock;
        if (i < n) put(out + i, r[j]);
    }
}

// ---------------------------------------------------------------------------------------------
// Concat of up to kMaxConcatInputs inputs in one launch: blockIdx.y picks the input, blockIdx.x a
// chunk of it (the grid is sized for the largest; blocks past the end of a smaller input leave).
// Input k is [outer, row_units[k]] and lands at column out_off[k] of [outer, out_row_units].
constexpr int kMaxConcatInputs = 8;
struct ConcatArgs {
    const void *in[kMaxConcatInputs];
    uint32_t n_units[kMaxConcatInputs];
    uint32_t row_units[kMaxConcatInputs];
    uint32_t row_mul[kMaxConcatInputs], row_shr[kMaxConcatInputs];
    uint64_t out_off[kMaxConcatInputs];
    uint64_t out_row_units;
};

template <typename U>
__global__ __launch_bounds__(kBlock) void concat_kernel(ConcatArgs a, U *__restrict__ out) {
    const int k = blockIdx.y;
    const uint32_t n = a.n_units[k];
    const uint32_t base = blockIdx.x * kChunk;
    if (base >= n) return;
    const U *__restrict__ in = static_cast<const U *>(a.in[k]);
    const uint32_t row_units = a.row_units[k], mul = a.row_mul[k], shr = a.row_shr[k];
    const uint64_t off = a.out_off[k];
    U r[kUnroll];
    uint64_t dst[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const uint32_t i = base + threadIdx.x + j * kBlock;
        const uint32_t e = i < n ? i : n - 1;
        const uint32_t o = row_units == 1 ? e : (__umulhi(e, mul) >> shr);
        dst[j] = o * a.out_row_units + off + (e - o * row_units);
        r[j] = nt_load(in + e);
    }
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
        const uint32_t i = base + threadIdx.x + j * kBlock;
        if (i < n) put(out + dst[j], r[j]);
    }
}

// ---------------------------------------------------------------------------------------------
// Trilu over [batch, rows, cols]; VEC units along cols
template <typename U, int VEC>
__device__ __forceinline__ Vec<U, VEC> trilu_item(const U *__restrict__ in, uint32_t i, uint32_t cols_v,
                                                  FastDiv cols_div, uint32_t rows, FastDiv rows_div,
                                                  int upper, int64_t k) {
    const uint32_t rq = cols_div.div(i);
    const uint32_t cv = i - rq * cols_v;
    const uint32_t bq = rows_div.div(rq);
    const int64_t row = rq - bq * rows;
    const int64_t c0 = static_cast<int64_t>(cv) * VEC;
    const int64_t diag = row + k;  // upper keeps col >= diag, lower keeps col <= diag
    const bool any = upper ? (c0 + VEC - 1 >= diag) : (c0 <= diag);
    Vec<U, VEC> v;
    if (any) {   // vectors wholly outside the triangle are not read
        v = nt_load(reinterpret_cast<const Vec<U, VEC> *>(in + static_cast<size_t>(i) * VEC));
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const bool keep = upper ? (c0 + j >= diag) : (c0 + j <= diag);
            if (!keep) v.v[j] = U{};
        }
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v.v[j] = U{};
    }
    return v;
}

template <typename U, int VEC>
__global__ __launch_bounds__(kBlock) void trilu_kernel(const U *__restrict__ in,
                                                       U *__restrict__ out, uint32_t n_items,
                                                       uint32_t cols_v, FastDiv cols_div,
                                                       uint32_t rows, FastDiv rows_div, int upper,
                                                       int64_t k) {
    using V = Vec<U, VEC>;
    for (uint32_t base = blockIdx.x * kChunk; base < n_items; base += gridDim.x * kChunk) {
        const uint32_t i0 = base + threadIdx.x;
        if (base + kChunk <= n_items) {
            V r[kUnroll];
#pragma unroll
            for (int j = 0; j < kUnroll; ++j)
                r[j] = trilu_item<U, VEC>(in, i0 + j * kBlock, cols_v, cols_div, rows, rows_div, upper, k);
#pragma unroll
            for (int j = 0; j < kUnroll; ++j)
                put(reinterpret_cast<V *>(out + static_cast<size_t>(i0 + j * kBlock) * VEC), r[j]);
        } else {
            for (uint32_t i = i0; i < n_items; i += kBlock)
                put(reinterpret_cast<V *>(out + static_cast<size_t>(i) * VEC),
                    trilu_item<U, VEC>(in, i, cols_v, cols_div, rows, rows_div, upper, k));
        }
    }
}

template <typename U>
int32_t launch_trilu(hipStream_t s, int64_t batch, int64_t rows, int64_t cols, int upper,
                     int64_t k, const void *in, void *out) {
    constexpr size_t kAlign = sizeof(U) * 4 > 16 ? 16 : sizeof(U) * 4;
    const bool vec_ok = cols % 4 == 0 && reinterpret_cast<uintptr_t>(in) % kAlign == 0 &&
                        reinterpret_cast<uintptr_t>(out) % kAlign == 0;
    const int vec = vec_ok ? 4 : 1;
    const int64_t cols_v = cols / vec;
    constexpr int64_t kLimit = (int64_t)1 << 30;
    if (rows > kLimit / cols_v) return RMLK_ERR_TOO_LARGE;  // one matrix per launch at least
    int64_t mats_per = kLimit / (rows * cols_v);
    for (int64_t b0 = 0; b0 < batch; b0 += mats_per) {
        const int64_t nb = batch - b0 < mats_per ? batch - b0 : mats_per;
        const U *pi = static_cast<const U *>(in) + b0 * rows * cols;
        U *po = static_cast<U *>(out) + b0 * rows * cols;
        const uint32_t n_items = static_cast<uint32_t>(nb * rows * cols_v);
        const unsigned grid = chunk_grid(n_items, kChunk);
        const uint32_t cv = static_cast<uint32_t>(cols_v), rw = static_cast<uint32_t>(rows);
        if (vec == 4)
            trilu_kernel<U, 4><<<grid, kBlock, 0, s>>>(pi, po, n_items, cv, FastDiv(cv), rw,
                                                      FastDiv(rw), upper, k);
        else
            trilu_kernel<U, 1><<<grid, kBlock, 0, s>>>(pi, po, n_items, cv, FastDiv(cv), rw,
                                                      FastDiv(rw), upper, k);
        int32_t st = launch_status();
        if (st) return st;
    }
    return RMLK_OK;
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

// Device-to-device copy with the flat copy kernel when both ends and the length are multiples of 16
// bytes (what the runtime copies: whole tensors from its pool), through the HIP runtime otherwise.
extern "C" int32_t rmlk_hip_memcpy_dtod(rmlk_stream_t stream, void *dst, const void *src,
                                        size_t bytes) {
    if (bytes == 0) return RMLK_OK;
    if (!dst || !src) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    if (bytes % 16 || reinterpret_cast<uintptr_t>(dst) % 16 || reinterpret_cast<uintptr_t>(src) % 16)
        return static_cast<int32_t>(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s));
    constexpr size_t kPieceUnits = static_cast<size_t>(1) << 30;
    const U128 *pi = static_cast<const U128 *>(src);
    U128 *po = static_cast<U128 *>(dst);
    for (size_t done = 0, units = bytes / 16; done < units; done += kPieceUnits) {
        const uint32_t n = static_cast<uint32_t>(units - done < kPieceUnits ? units - done : kPieceUnits);
        copy_flat_kernel<U128><<<chunk_grid(n, kChunk), kBlock, 0, s>>>(pi + done, po + done, n);
        const int32_t st = launch_status();
        if (st) return st;
    }
    return RMLK_OK;
}

// Up to 32 device-to-device copies as ONE launch (16-byte aligned ends and lengths, below 16 GiB
// each; more of them 32 per launch); anything else one call of rmlk_hip_memcpy_dtod per copy.
extern "C" int32_t rmlk_hip_memcpy_dtod_many(rmlk_stream_t stream, int32_t n_copies, void *const *dsts,
                                             const void *const *srcs, const size_t *bytes) {
    if (n_copies < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n_copies == 0) return RMLK_OK;
    if (!dsts || !srcs || !bytes) return RMLK_ERR_NULL_POINTER;
    bool together = n_copies > 1;
    for (int i = 0; i < n_copies; ++i) {
        if (bytes[i] && (!dsts[i] || !srcs[i])) return RMLK_ERR_NULL_POINTER;
        if (bytes[i] % 16 || reinterpret_cast<uintptr_t>(dsts[i]) % 16 || reinterpret_cast<uintptr_t>(srcs[i]) % 16 ||
            bytes[i] / 16 >= (static_cast<size_t>(1) << 30))
            together = false;
    }
    if (!together) {
        for (int i = 0; i < n_copies; ++i) {
            const int32_t st = rmlk_hip_memcpy_dtod(stream, dsts[i], srcs[i], bytes[i]);
            if (st) return st;
        }
        return RMLK_OK;
    }
    for (int first = 0; first < n_copies; first += kMaxCopies) {
        const int count = n_copies - first < kMaxCopies ? n_copies - first : kMaxCopies;
        CopyMany a{};
        size_t longest = 0;
        for (int i = 0; i < count; ++i) {
            a.in[i] = static_cast<const U128 *>(srcs[first + i]);
            a.out[i] = static_cast<U128 *>(dsts[first + i]);
            a.n[i] = static_cast<uint32_t>(bytes[first + i] / 16);
            if (bytes[first + i] > longest) longest = bytes[first + i];
        }
        if (longest == 0) continue;
        dim3 grid(chunk_grid(static_cast<uint32_t>(longest / 16), kChunk), static_cast<unsigned>(count), 1);
        copy_many_kernel<<<grid, kBlock, 0, as_stream(stream)>>>(a);
        const int32_t st = launch_status();
        if (st) return st;
    }
    return RMLK_OK;
}

extern "C" int32_t rmlk_hip_transpose(rmlk_stream_t stream, int32_t dtype,
                                      const rmlk_dims *in_shape, const int64_t *perm,
                                      const void *in, void *out) {
    if (!dims_ok(in_shape)) return RMLK_ERR_BAD_RANK;
    if (!perm) return RMLK_ERR_NULL_POINTER;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    const int rank = in_shape->rank;
    bool seen[kMaxRank] = {false};
    for (int d = 0; d < rank; ++d) {
        if (perm[d] < 0 || perm[d] >= rank || seen[perm[d]]) return RMLK_ERR_INVALID_ARGUMENT;
        seen[perm[d]] = true;
    }
    int64_t numel = dims_numel(in_shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    int64_t in_st[kMaxRank], shape[kMaxRank], st[2][kMaxRank];
    dense_strides(rank, in_shape->v, in_st);
    for (int d = 0; d < rank; ++d) {
        shape[d] = in_shape->v[perm[d]];
        st[0][d] = in_st[perm[d]];
    }
    dense_strides(rank, shape, st[1]);
    hipStream_t s = as_stream(stream);
    NdPlan<2> pl;
    build_plan<2>(pl, rank, shape, st);
    const int last = pl.rank - 1;
    if (pl.stride[0][last] == 1 || numel >= ((int64_t)1 << 31) || (esize != 4 && esize != 8))
        return strided_copy(s, esize, rank, shape, st, in, out);
    // find the dim that is contiguous in the input
    int q = -1;
    for (int d = 0; d < last; ++d)
        if (pl.stride[0][d] == 1) { q = d; break; }
    if (q < 0 || pl.dim64[q] < 8 || pl.dim64[last] < 8)
        return strided_copy(s, esize, rank, shape, st, in, out);
    TilePlan tp{};
    tp.n_batch_dims = 0;
    uint64_t blocks = 1;
    for (int d = 0; d < last; ++d) {
        if (d == q) continue;
        int b = tp.n_batch_dims++;
        tp.bdim[b] = pl.dim[d];
        tp.bdiv[b] = FastDiv(pl.dim[d]);
        tp.b_in[b] = pl.stride[0][d];
        tp.b_out[b] = pl.stride[1][d];
        blocks *= pl.dim[d];
    }
    tp.q_len = pl.dim[q];
    tp.l_len = pl.dim[last];
    tp.q_tiles = (tp.q_len + kTile - 1) / kTile;
    tp.l_tiles = (tp.l_len + kTile - 1) / kTile;
    tp.q_tiles_div = FastDiv(tp.q_tiles);
    tp.l_tiles_div = FastDiv(tp.l_tiles);
    tp.l_in_stride = pl.stride[0][last];
    tp.q_out_stride = pl.stride[1][q];
    blocks *= static_cast<uint64_t>(tp.q_tiles) * tp.l_tiles;
    if (blocks >= (1ull << 31)) return strided_copy(s, esize, rank, shape, st, in, out);
    if (esize == 4) return launch_tile<uint32_t>(s, tp, blocks, in, out);
    return launch_tile<uint64_t>(s, tp, blocks, in, out);
}

extern "C" int32_t rmlk_hip_expand(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                                   const rmlk_dims *out_shape, const void *in, void *out) {
    if (!dims_ok(in_shape) || !dims_ok(out_shape)) return RMLK_ERR_BAD_RANK;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    const int rank = out_shape->rank;
    if (in_shape->rank > rank) return RMLK_ERR_SIZE_MISMATCH;
    int64_t numel = dims_numel(out_shape);
    if (numel < 0 || dims_numel(in_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t in_st[kMaxRank], st[2][kMaxRank];
    dense_strides(in_shape->rank, in_shape->v, in_st);
    const int shift = rank - in_shape->rank;
    for (int d = 0; d < rank; ++d) {
        int di = d - shift;
        if (di < 0) {
            st[0][d] = 0;
        } else if (in_shape->v[di] == out_shape->v[d]) {
            st[0][d] = in_st[di];
        } else if (in_shape->v[di] == 1) {
            st[0][d] = 0;
        } else {
            return RMLK_ERR_SIZE_MISMATCH;
        }
    }
    if (numel == 0) return RMLK_OK;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    dense_strides(rank, out_shape->v, st[1]);
    if (numel <= kBatchMaxElems && batch_collecting()) {
        // (a tiny broadcast copy on a stream that is collecting its launches)
        SmallOp so{};
        so.kind = kSmallCopy;
        so.dt = esize;
        so.in[0] = in;
        so.out = out;
        if (small_op_layout(so, rank, out_shape->v, 1, st) && batch_take(as_stream_collecting(stream), so))
            return RMLK_OK;
    }
    return strided_copy(as_stream(stream), esize, rank, out_shape->v, st, in, out);
}

extern "C" int32_t rmlk_hip_slice(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                                  const rmlk_dims *starts, const rmlk_dims *steps,
                                  const rmlk_dims *out_shape, const void *in, void *out) {
    if (!dims_ok(in_shape) || !dims_ok(starts) || !dims_ok(steps) || !dims_ok(out_shape))
        return RMLK_ERR_BAD_RANK;
    const int rank = in_shape->rank;
    if (starts->rank != rank || steps->rank != rank || out_shape->rank != rank)
        return RMLK_ERR_SIZE_MISMATCH;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    int64_t numel = dims_numel(out_shape);
    if (numel < 0 || dims_numel(in_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    int64_t in_st[kMaxRank], st[2][kMaxRank];
    dense_strides(rank, in_shape->v, in_st);
    int64_t base = 0;
    for (int d = 0; d < rank; ++d) {
        const int64_t step = steps->v[d], start = starts->v[d], n = out_shape->v[d];
        if (step == 0) return RMLK_ERR_INVALID_ARGUMENT;
        const int64_t dim = in_shape->v[d];
        if (start < 0 || start >= dim) return RMLK_ERR_INVALID_ARGUMENT;
        // last addressed index; the magnitudes are bounded by dim so no overflow for valid input
        if (n - 1 > dim) return RMLK_ERR_INVALID_ARGUMENT;
        if (step > dim || step < -dim) {
            if (n > 1) return RMLK_ERR_INVALID_ARGUMENT;
        } else {
            const int64_t lastix = start + (n - 1) * step;
            if (lastix < 0 || lastix >= dim) return RMLK_ERR_INVALID_ARGUMENT;
        }
        base += start * in_st[d];
        st[0][d] = n > 1 ? in_st[d] * step : 0;
    }
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    dense_strides(rank, out_shape->v, st[1]);
    return strided_copy(as_stream(stream), esize, rank, out_shape->v, st,
                        static_cast<const char *>(in) + base * esize, out);
}

extern "C" int32_t rmlk_hip_concat(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *in_shape,
                                   const rmlk_dims *out_shape, int32_t axis, int64_t axis_offset,
                                   const void *in, void *out) {
    if (!dims_ok(in_shape) || !dims_ok(out_shape)) return RMLK_ERR_BAD_RANK;
    const int rank = in_shape->rank;
    if (out_shape->rank != rank) return RMLK_ERR_SIZE_MISMATCH;
    if (axis < 0 || axis >= rank) return RMLK_ERR_INVALID_ARGUMENT;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    for (int d = 0; d < rank; ++d) {
        if (in_shape->v[d] < 0 || out_shape->v[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (d != axis && in_shape->v[d] != out_shape->v[d]) return RMLK_ERR_SIZE_MISMATCH;
    }
    if (axis_offset < 0 || axis_offset + in_shape->v[axis] > out_shape->v[axis])
        return RMLK_ERR_SIZE_MISMATCH;
    int64_t numel = dims_numel(in_shape);
    if (numel < 0 || dims_numel(out_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    int64_t st[2][kMaxRank];
    dense_strides(rank, in_shape->v, st[0]);
    dense_strides(rank, out_shape->v, st[1]);
    const int64_t base = axis_offset * st[1][axis];
    return strided_copy(as_stream(stream), esize, rank, in_shape->v, st, in,
                        static_cast<char *>(out) + base * esize);
}

extern "C" int32_t rmlk_hip_scatter_nd_copy(rmlk_stream_t stream, int32_t dtype,
                                            const rmlk_dims *data_shape, int64_t n_tuples,
                                            int32_t tuple_size, const int64_t *idx, const void *updates,
                                            const void *data, void *out, int32_t *err_flag) {
    if (!dims_ok(data_shape)) return RMLK_ERR_BAD_RANK;
    const int rank = data_shape->rank;
    if (tuple_size < 1 || tuple_size > rank) return RMLK_ERR_INVALID_ARGUMENT;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    const int64_t numel = dims_numel(data_shape);
    if (n_tuples < 0 || numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!data || !out) return RMLK_ERR_NULL_POINTER;
    int64_t slice_len = 1;
    for (int d = tuple_size; d < rank; ++d) slice_len *= data_shape->v[d];
    const int64_t bytes = numel * esize, slice_bytes = slice_len * esize;
    auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool fused = n_tuples >= 1 && n_tuples <= static_cast<int64_t>(kMaxFusedTuples) && idx &&
                       updates && slice_bytes % 16 == 0 && aligned(data) && aligned(out) &&
                       aligned(updates) && bytes / 16 < ((int64_t)1 << 31);
    if (!fused) {
        if (data != out) {
            const int32_t st = rmlk_hip_memcpy_dtod(stream, out, data, static_cast<size_t>(bytes));
            if (st) return st;
        }
        return rmlk_hip_scatter_nd(stream, RMLK_SCATTER_NONE, dtype, data_shape, n_tuples, tuple_size,
                                   idx, updates, out, err_flag);
    }
    ScatterPlan sp{};
    sp.tuple_size = tuple_size;
    int64_t stride = 1;
    for (int t = tuple_size - 1; t >= 0; --t) {
        sp.dim[t] = data_shape->v[t];
        sp.stride[t] = stride;
        stride *= data_shape->v[t];
    }
    const uint32_t n = static_cast<uint32_t>(bytes / 16);
    scatter_copy_kernel<<<(n + kChunk - 1) / kChunk, kBlock, 0, as_stream(stream)>>>(
        sp, idx, static_cast<const U128 *>(updates), static_cast<const U128 *>(data),
        static_cast<U128 *>(out), n, static_cast<uint32_t>(n_tuples),
        static_cast<uint32_t>(slice_bytes / 16), err_flag);
    return launch_status();
}

namespace {
template <typename U>
int32_t launch_concat_units(hipStream_t s, const ConcatArgs &a, int n_in, uint32_t largest, void *out) {
    dim3 grid((largest + kChunk - 1) / kChunk, static_cast<unsigned>(n_in));
    concat_kernel<U><<<grid, kBlock, 0, s>>>(a, static_cast<U *>(out));
    return launch_status();
}
}  // namespace

extern "C" int32_t rmlk_hip_concat_many(rmlk_stream_t stream, int32_t dtype, int32_t n_inputs,
                                        const rmlk_dims *in_shapes, const void *const *ins,
                                        const rmlk_dims *out_shape, int32_t axis, void *out) {
    if (n_inputs < 1 || !in_shapes || !ins) return RMLK_ERR_INVALID_ARGUMENT;
    if (!dims_ok(out_shape)) return RMLK_ERR_BAD_RANK;
    const int rank = out_shape->rank;
    if (axis < 0 || axis >= rank) return RMLK_ERR_INVALID_ARGUMENT;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    int64_t total = 0, outer = 1, inner = 1;
    for (int d = 0; d < axis; ++d) outer *= out_shape->v[d];
    for (int d = axis + 1; d < rank; ++d) inner *= out_shape->v[d];
    for (int k = 0; k < n_inputs; ++k) {
        if (!dims_ok(&in_shapes[k]) || in_shapes[k].rank != rank) return RMLK_ERR_SIZE_MISMATCH;
        for (int d = 0; d < rank; ++d) {
            if (in_shapes[k].v[d] < 0) return RMLK_ERR_INVALID_ARGUMENT;
            if (d != axis && in_shapes[k].v[d] != out_shape->v[d]) return RMLK_ERR_SIZE_MISMATCH;
        }
        total += in_shapes[k].v[axis];
    }
    if (total != out_shape->v[axis]) return RMLK_ERR_SIZE_MISMATCH;
    if (dims_numel(out_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (dims_numel(out_shape) == 0) return RMLK_OK;
    if (!out) return RMLK_ERR_NULL_POINTER;
    if (dims_numel(out_shape) <= kBatchMaxElems && batch_collecting() && n_inputs <= kBatchMaxOps) {
        // a tiny Concat on a stream that is collecting its launches: a copy record per input, each
        // into its columns of the output
        SmallOp recs[kBatchMaxOps];
        int n_rec = 0;
        bool fits = true;
        int64_t out_st[kMaxRank], at = 0;
        dense_strides(rank, out_shape->v, out_st);
        for (int k = 0; k < n_inputs && fits; ++k) {
            const int64_t len = in_shapes[k].v[axis];
            if (len > 0 && outer * inner > 0) {
                if (!ins[k]) return RMLK_ERR_NULL_POINTER;
                int64_t st2[2][kMaxRank];
                dense_strides(rank, in_shapes[k].v, st2[0]);
                for (int d = 0; d < rank; ++d) st2[1][d] = out_st[d];
                SmallOp &so = recs[n_rec];
                so = SmallOp{};
                so.kind = kSmallCopy;
                so.dt = esize;
                so.in[0] = ins[k];
                so.out = static_cast<char *>(out) + at * inner * esize;
                fits = small_op_layout(so, rank, in_shapes[k].v, 1, st2);
                ++n_rec;
            }
            at += len;
        }
        if (fits) {
            hipStream_t sc = as_stream_collecting(stream);
            bool taken = true;
            for (int r = 0; r < n_rec && taken; ++r) taken = batch_take(sc, recs[r]);
            if (taken) return RMLK_OK;
            // (no batch on this stream after all: nothing was taken, the launch below does the work)
        }
    }
    // one launch when every input's rows and landing columns are whole units of one width
    int unit = 16;
    bool one_launch = n_inputs <= kMaxConcatInputs && outer < ((int64_t)1 << 31);
    int64_t col = 0;
    for (int k = 0; k < n_inputs && one_launch; ++k) {
        const int64_t row_bytes = in_shapes[k].v[axis] * inner * esize;
        if (row_bytes == 0) continue;
        if (!ins[k]) return RMLK_ERR_NULL_POINTER;
        if (row_bytes * outer >= ((int64_t)1 << 31) * esize) one_launch = false;
        while (unit > esize && (row_bytes % unit || (col * inner * esize) % unit ||
                                reinterpret_cast<uintptr_t>(ins[k]) % unit))
            unit >>= 1;
        col += in_shapes[k].v[axis];
    }
    while (unit > esize && ((total * inner * esize) % unit || reinterpret_cast<uintptr_t>(out) % unit))
        unit >>= 1;
    if (!one_launch) {
        int64_t off = 0;
        for (int k = 0; k < n_inputs; ++k) {
            const int32_t st = rmlk_hip_concat(stream, dtype, &in_shapes[k], out_shape, axis, off, ins[k], out);
            if (st) return st;
            off += in_shapes[k].v[axis];
        }
        return RMLK_OK;
    }
    ConcatArgs a{};
    a.out_row_units = static_cast<uint64_t>(total * inner * esize / unit);
    uint32_t largest = 0;
    int n_in = 0;
    col = 0;
    for (int k = 0; k < n_inputs; ++k) {
        const int64_t row_units = in_shapes[k].v[axis] * inner * esize / unit;
        if (row_units > 0) {
            const FastDiv fd(static_cast<uint32_t>(row_units));
            a.in[n_in] = ins[k];
            a.row_units[n_in] = static_cast<uint32_t>(row_units);
            a.row_mul[n_in] = fd.mul;
            a.row_shr[n_in] = fd.shr;
            a.n_units[n_in] = static_cast<uint32_t>(row_units * outer);
            a.out_off[n_in] = static_cast<uint64_t>(col * inner * esize / unit);
            if (a.n_units[n_in] > largest) largest = a.n_units[n_in];
            ++n_in;
        }
        col += in_shapes[k].v[axis];
    }
    if (n_in == 0) return RMLK_OK;
    hipStream_t s = as_stream(stream);
    switch (unit) {
        case 1: return launch_concat_units<uint8_t>(s, a, n_in, largest, out);
        case 2: return launch_concat_units<uint16_t>(s, a, n_in, largest, out);
        case 4: return launch_concat_units<uint32_t>(s, a, n_in, largest, out);
        case 8: return launch_concat_units<uint64_t>(s, a, n_in, largest, out);
        default: return launch_concat_units<U128>(s, a, n_in, largest, out);
    }
}

extern "C" int32_t rmlk_hip_gather(rmlk_stream_t stream, int32_t dtype, int32_t idx_dtype,
                                   const rmlk_dims *data_shape, int32_t axis, int64_t n_idx,
                                   const void *data, const void *idx, void *out,
                                   int32_t *err_flag) {
    if (!dims_ok(data_shape)) return RMLK_ERR_BAD_RANK;
    const int rank = data_shape->rank;
    if (axis < 0 || axis >= rank) return RMLK_ERR_INVALID_ARGUMENT;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    if (idx_dtype != RMLK_INT32 && idx_dtype != RMLK_INT64) return RMLK_ERR_UNSUPPORTED;
    if (n_idx < 0 || dims_numel(data_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < axis; ++d) outer *= data_shape->v[d];
    for (int d = axis + 1; d < rank; ++d) inner *= data_shape->v[d];
    const int64_t axis_dim = data_shape->v[axis];
    if (outer == 0 || inner == 0 || n_idx == 0) return RMLK_OK;
    if (!data && axis_dim > 0) return RMLK_ERR_NULL_POINTER;
    if (!idx || !out) return RMLK_ERR_NULL_POINTER;
    // widest unit dividing a row and the alignments
    int64_t row_bytes = inner * esize;
    int unit = esize;
    for (int cand = 16; cand > esize; cand >>= 1) {
        if (row_bytes % cand == 0 && reinterpret_cast<uintptr_t>(data) % cand == 0 &&
            reinterpret_cast<uintptr_t>(out) % cand == 0) {
            unit = cand;
            break;
        }
    }
    const int64_t row_units = row_bytes / unit;
    if (row_units >= ((int64_t)1 << 30) || n_idx >= ((int64_t)1 << 30)) return RMLK_ERR_TOO_LARGE;
    hipStream_t s = as_stream(stream);
    // pieces over `outer` so that units per launch stay below 2^30
    const int64_t units_per_outer = n_idx * row_units;
    if (units_per_outer > ((int64_t)1 << 30)) return RMLK_ERR_TOO_LARGE;
    int64_t outer_per = ((int64_t)1 << 30) / units_per_outer;
    for (int64_t o0 = 0; o0 < outer; o0 += outer_per) {
        int64_t no = outer - o0 < outer_per ? outer - o0 : outer_per;
        const char *pd = static_cast<const char *>(data) + o0 * axis_dim * row_bytes;
        char *po = static_cast<char *>(out) + o0 * n_idx * row_bytes;
        uint32_t n_units = static_cast<uint32_t>(no * units_per_outer);
        int32_t st;
        switch (unit) {
            case 1: st = launch_gather<uint8_t>(s, idx_dtype, pd, idx, po, n_units, (uint32_t)row_units, (uint32_t)n_idx, axis_dim, err_flag); break;
            case 2: st = launch_gather<uint16_t>(s, idx_dtype, pd, idx, po, n_units, (uint32_t)row_units, (uint32_t)n_idx, axis_dim, err_flag); break;
            case 4: st = launch_gather<uint32_t>(s, idx_dtype, pd, idx, po, n_units, (uint32_t)row_units, (uint32_t)n_idx, axis_dim, err_flag); break;
            case 8: st = launch_gather<uint64_t>(s, idx_dtype, pd, idx, po, n_units, (uint32_t)row_units, (uint32_t)n_idx, axis_dim, err_flag); break;
            default: st = launch_gather<U128>(s, idx_dtype, pd, idx, po, n_units, (uint32_t)row_units, (uint32_t)n_idx, axis_dim, err_flag); break;
        }
        if (st) return st;
    }
    return RMLK_OK;
}

namespace {
template <int RED, typename T>
int32_t launch_scatter(hipStream_t s, const ScatterPlan &sp, const int64_t *idx, const void *upd,
                       void *out, uint32_t n_units, uint32_t slice_units, int32_t *err) {
    unsigned grid = grid_for(n_units, kBlock, 16);
    scatter_nd_kernel<RED, T><<<grid, kBlock, 0, s>>>(sp, idx, static_cast<const T *>(upd),
                                                      static_cast<T *>(out), n_units, slice_units,
                                                      FastDiv(slice_units), err);
    return launch_status();
}

template <typename T>
int32_t dispatch_scatter_red(hipStream_t s, int red, const ScatterPlan &sp, const int64_t *idx,
                             const void *upd, void *out, uint32_t n_units, uint32_t slice_units,
                             int32_t *err) {
    switch (red) {
        case RMLK_SCATTER_ADD: return launch_scatter<RMLK_SCATTER_ADD, T>(s, sp, idx, upd, out, n_units, slice_units, err);
        case RMLK_SCATTER_MUL: return launch_scatter<RMLK_SCATTER_MUL, T>(s, sp, idx, upd, out, n_units, slice_units, err);
        case RMLK_SCATTER_MAX: return launch_scatter<RMLK_SCATTER_MAX, T>(s, sp, idx, upd, out, n_units, slice_units, err);
        case RMLK_SCATTER_MIN: return launch_scatter<RMLK_SCATTER_MIN, T>(s, sp, idx, upd, out, n_units, slice_units, err);
        default: return RMLK_ERR_INVALID_ARGUMENT;
    }
}
}  // namespace

extern "C" int32_t rmlk_hip_scatter_nd(rmlk_stream_t stream, int32_t reduction, int32_t dtype,
                                       const rmlk_dims *data_shape, int64_t n_tuples,
                                       int32_t tuple_size, const int64_t *idx, const void *updates,
                                       void *out, int32_t *err_flag) {
    if (!dims_ok(data_shape)) return RMLK_ERR_BAD_RANK;
    const int rank = data_shape->rank;
    if (tuple_size < 1 || tuple_size > rank) return RMLK_ERR_INVALID_ARGUMENT;
    if (reduction < RMLK_SCATTER_NONE || reduction > RMLK_SCATTER_MIN)
        return RMLK_ERR_INVALID_ARGUMENT;
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    if (reduction != RMLK_SCATTER_NONE && dtype != RMLK_FLOAT && dtype != RMLK_DOUBLE &&
        dtype != RMLK_INT32 && dtype != RMLK_INT64)
        return RMLK_ERR_UNSUPPORTED;
    if (n_tuples < 0 || dims_numel(data_shape) < 0) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t slice_len = 1;
    for (int d = tuple_size; d < rank; ++d) slice_len *= data_shape->v[d];
    if (n_tuples == 0 || slice_len == 0) return RMLK_OK;
    if (!idx || !updates || !out) return RMLK_ERR_NULL_POINTER;
    ScatterPlan sp{};
    sp.tuple_size = tuple_size;
    int64_t stride = 1;
    for (int t = tuple_size - 1; t >= 0; --t) {
        sp.dim[t] = data_shape->v[t];
        sp.stride[t] = stride;
        stride *= data_shape->v[t];
    }
    hipStream_t s = as_stream(stream);
    int unit = esize;
    if (reduction == RMLK_SCATTER_NONE) {
        int64_t slice_bytes = slice_len * esize;
        for (int cand = 16; cand > esize; cand >>= 1) {
            if (slice_bytes % cand == 0 && reinterpret_cast<uintptr_t>(updates) % cand == 0 &&
                reinterpret_cast<uintptr_t>(out) % cand == 0) {
                unit = cand;
                break;
            }
        }
    }
    const int64_t slice_units = slice_len * esize / unit;
    if (slice_units >= ((int64_t)1 << 30)) return RMLK_ERR_TOO_LARGE;
    int64_t tuples_per = ((int64_t)1 << 30) / slice_units;
    for (int64_t t0 = 0; t0 < n_tuples; t0 += tuples_per) {
        int64_t nt = n_tuples - t0 < tuples_per ? n_tuples - t0 : tuples_per;
        const int64_t *pidx = idx + t0 * tuple_size;
        const char *pu = static_cast<const char *>(updates) + t0 * slice_len * esize;
        uint32_t n_units = static_cast<uint32_t>(nt * slice_units);
        uint32_t su = static_cast<uint32_t>(slice_units);
        int32_t st;
        if (reduction == RMLK_SCATTER_NONE) {
            switch (unit) {
                case 1: st = launch_scatter<RMLK_SCATTER_NONE, uint8_t>(s, sp, pidx, pu, out, n_units, su, err_flag); break;
                case 2: st = launch_scatter<RMLK_SCATTER_NONE, uint16_t>(s, sp, pidx, pu, out, n_units, su, err_flag); break;
                case 4: st = launch_scatter<RMLK_SCATTER_NONE, uint32_t>(s, sp, pidx, pu, out, n_units, su, err_flag); break;
                case 8: st = launch_scatter<RMLK_SCATTER_NONE, uint64_t>(s, sp, pidx, pu, out, n_units, su, err_flag); break;
                default: st = launch_scatter<RMLK_SCATTER_NONE, U128>(s, sp, pidx, pu, out, n_units, su, err_flag); break;
            }
        } else {
            switch (dtype) {
                case RMLK_FLOAT: st = dispatch_scatter_red<float>(s, reduction, sp, pidx, pu, out, n_units, su, err_flag); break;
                case RMLK_DOUBLE: st = dispatch_scatter_red<double>(s, reduction, sp, pidx, pu, out, n_units, su, err_flag); break;
                case RMLK_INT32: st = dispatch_scatter_red<int32_t>(s, reduction, sp, pidx, pu, out, n_units, su, err_flag); break;
                default: st = dispatch_scatter_red<int64_t>(s, reduction, sp, pidx, pu, out, n_units, su, err_flag); break;
            }
        }
        if (st) return st;
    }
    return RMLK_OK;
}

extern "C" int32_t rmlk_hip_trilu(rmlk_stream_t stream, int32_t dtype, int64_t batch, int64_t rows,
                                  int64_t cols, int32_t upper, int64_t k, const void *in,
                                  void *out) {
    const int esize = dtype_size(dtype);
    if (!esize) return RMLK_ERR_UNSUPPORTED;
    if (batch < 0 || rows < 0 || cols < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (batch == 0 || rows == 0 || cols == 0) return RMLK_OK;
    if (batch > kMaxElems / rows || batch * rows > kMaxElems / cols) return RMLK_ERR_TOO_LARGE;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    // col - row lies in [-(rows-1), cols-1]; clamping k to [-rows, cols] keeps the predicate.
    if (k < -rows) k = -rows;
    if (k > cols) k = cols;
    hipStream_t s = as_stream(stream);
    switch (esize) {
        case 1: return launch_trilu<uint8_t>(s, batch, rows, cols, upper != 0, k, in, out);
        case 2: return launch_trilu<uint16_t>(s, batch, rows, cols, upper != 0, k, in, out);
        case 4: return launch_trilu<uint32_t>(s, batch, rows, cols, upper != 0, k, in, out);
        default: return launch_trilu<uint64_t>(s, batch, rows, cols, upper != 0, k, in, out);
    }
}
