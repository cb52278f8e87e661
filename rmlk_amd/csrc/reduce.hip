// Row reductions: ReduceMean and Softmax.
//
// ReduceMean replaces cuda/src/ptx/reduce_mean.cu:5-9, whose kernel gives every output element to
// one thread that walks the reduced elements serially (aggregation_op_macros.cuh:1-49). Here a
// wavefront (or a block, for few long rows) owns a row, reads it with 128-bit loads, accumulates
// in double like the reference and combines lanes with cross-lane shuffles.
//
// Softmax replaces the cuDNN call of cuda/src/kernels/softmax.rs:5-37. A wavefront keeps its whole
// row in registers (one HBM read, one HBM write), max-subtracted.
#include <type_traits>

#include "nd_index.hpp"

namespace rmlk {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

// sum / n in double. For n a power of two the quotient is the product with 1 / n, exactly (a change
// of exponent), and the multiply is one instruction where the IEEE division is a chain of thirty
// between a wavefront's last load and its first store.
__device__ __forceinline__ double mean_of(double sum, int64_t n) {
    if ((n & (n - 1)) == 0) return sum * (1.0 / static_cast<double>(n));
    return sum / static_cast<double>(n);
}

// ---- ReduceMean over trailing contiguous elements: [rows, cols] -> [rows] ---------------------
// kGroup lanes cooperate on a row: kWave (a wavefront per row) or kBlock (a block per row).
template <typename T, int VEC, int kGroup>
__global__ __launch_bounds__(kBlock) void mean_rows_kernel(const T *__restrict__ in,
                                                           T *__restrict__ out, int64_t rows,
                                                           int64_t cols) {
    __shared__ double partial[kWavesPerBlock];
    constexpr int kRowsPerBlock = kBlock / kGroup;
    const int lane_in_group = threadIdx.x % kGroup;
    const int group = threadIdx.x / kGroup;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + group; row < rows;
         row += static_cast<int64_t>(gridDim.x) * kRowsPerBlock) {
        const T *p = in + row * cols;
        double acc = 0.0;
        if constexpr (VEC == 1) {
            for (int64_t c = lane_in_group; c < cols; c += kGroup) acc += static_cast<double>(p[c]);
        } else {
            using V = Vec<T, VEC>;
            const int64_t nv = cols / VEC;
            const V *pv = reinterpret_cast<const V *>(p);
            int64_t c = lane_in_group;
            // the input is read once: streaming loads, eight in flight per lane while the row lasts
            for (; c + 7 * kGroup < nv; c += 8 * kGroup) {
                V v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = nt_load(pv + c + u * kGroup);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    acc += ((static_cast<double>(v[0].v[j]) + static_cast<double>(v[1].v[j])) +
                            (static_cast<double>(v[2].v[j]) + static_cast<double>(v[3].v[j]))) +
                           ((static_cast<double>(v[4].v[j]) + static_cast<double>(v[5].v[j])) +
                            (static_cast<double>(v[6].v[j]) + static_cast<double>(v[7].v[j])));
            }
            for (; c + 3 * kGroup < nv; c += 4 * kGroup) {
                V v0 = nt_load(pv + c), v1 = nt_load(pv + c + kGroup), v2 = nt_load(pv + c + 2 * kGroup),
                  v3 = nt_load(pv + c + 3 * kGroup);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    acc += (static_cast<double>(v0.v[j]) + static_cast<double>(v1.v[j])) +
                           (static_cast<double>(v2.v[j]) + static_cast<double>(v3.v[j]));
            }
            for (; c < nv; c += kGroup) {
                V v = nt_load(pv + c);
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc += static_cast<double>(v.v[j]);
            }
        }
        acc = wave_sum(acc);
        if constexpr (kGroup == kWave) {
            if (lane_in_group == 0) out[row] = static_cast<T>(mean_of(acc, cols));
        } else {
            const int wave = threadIdx.x / kWave;
            if ((threadIdx.x % kWave) == 0) partial[wave] = acc;
            __syncthreads();
            if (threadIdx.x == 0) {
                double t = 0.0;
#pragma unroll
                for (int w = 0; w < kWavesPerBlock; ++w) t += partial[w];
                out[row] = static_cast<T>(mean_of(t, cols));
            }
            __syncthreads();
        }
    }
}

// ---- ReduceMean, any axes: a wavefront per output element -------------------------------------
// kept / red are single-operand plans over the kept and the reduced dims of the input.
template <typename T>
__global__ __launch_bounds__(kBlock) void mean_generic_kernel(NdPlan<1> kept, NdPlan<1> red,
                                                              const T *__restrict__ in,
                                                              T *__restrict__ out,
                                                              uint32_t n_out, uint32_t n_red) {
    const int lane = threadIdx.x % kWave;
    const uint32_t wave0 = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    for (uint32_t o = wave0; o < n_out; o += gridDim.x * kWavesPerBlock) {
        int64_t base[1];
        nd_offsets<1>(kept, o, base);
        double acc = 0.0;
        for (uint32_t r = lane; r < n_red; r += kWave) {
            int64_t off[1];
            nd_offsets<1>(red, r, off);
            acc += static_cast<double>(in[base[0] + off[0]]);
        }
        acc = wave_sum(acc);
        if (lane == 0) out[o] = static_cast<T>(acc / static_cast<double>(n_red));
    }
}

// ---- Softmax, last axis, row held in registers ------------------------------------------------
template <typename T>
__device__ __forceinline__ T exp_t(T x) {
    if constexpr (std::is_same<T, float>::value) return expf(x);
    else return exp(x);
}
template <typename T>
__device__ __forceinline__ T neg_inf() {
    return -__builtin_huge_val();
}
template <>
__device__ __forceinline__ float neg_inf<float>() {
    return -__builtin_huge_valf();
}

// Where a softmax row comes from: plain memory, or (x / c + mask) resp. (x * c + mask) computed on
// the fly with exactly the roundings of the separate Div (Mul) and Add kernels.
template <typename T>
struct PlainRows {
    static constexpr bool kMasked = false;
    const T *in;
    __device__ __forceinline__ Vec<T, 4> load(int64_t row, int c, int32_t cols) const {
        // (the scores are read once: streaming loads, 196 -> 190 us on 65536 rows of 2048)
        return nt_load(reinterpret_cast<const Vec<T, 4> *>(in + row * cols) + c);
    }
    __device__ __forceinline__ Vec<T, 4> load_mask(int64_t, int) const { return Vec<T, 4>{}; }
    __device__ __forceinline__ void combine(Vec<T, 4> &, const Vec<T, 4> &) const {}
};

// row -> offset into a mask that is broadcast over some of the leading dims
struct RowMap {
    FastDiv d1, d2;       // extents of the two inner row dims
    uint32_t n1, n2;
    int64_t s0, s1, s2;   // mask element strides of the three row dims
    __device__ __forceinline__ int64_t offset(uint32_t row) const {
        const uint32_t t = d2.div(row), i2 = row - t * n2;
        const uint32_t i0 = d1.div(t), i1 = t - i0 * n1;
        return i0 * s0 + i1 * s1 + i2 * s2;
    }
};

template <typename T, bool MUL>
struct ScaledMaskedRows {
    const T *in;
    const T *mask;
    T scale;
    RowMap map;
    static constexpr bool kMasked = true;
    // the kernel issues every load of a row (scores, then mask) before it combines the first pair
    __device__ __forceinline__ Vec<T, 4> load(int64_t row, int c, int32_t cols) const {
        return nt_load(reinterpret_cast<const Vec<T, 4> *>(in + row * cols) + c);
    }
    __device__ __forceinline__ Vec<T, 4> load_mask(int64_t row, int c) const {
        return reinterpret_cast<const Vec<T, 4> *>(mask + map.offset(static_cast<uint32_t>(row)))[c];
    }
    __device__ __forceinline__ void combine(Vec<T, 4> &x, const Vec<T, 4> &m) const {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const T scaled = MUL ? x.v[j] * scale : x.v[j] / scale;
            x.v[j] = scaled + m.v[j];
        }
    }
};

// kGroup lanes own a row of up to kGroup * 4 * NV elements; cols % 4 == 0 and 16-byte aligned rows.
template <typename T, int NV, int kGroup, typename Rows>
__global__ __launch_bounds__(kBlock) void softmax_regs_kernel(Rows src, T *__restrict__ out,
                                                              int64_t rows, int32_t cols) {
    __shared__ T red_buf[2][kWavesPerBlock];
    using V = Vec<T, 4>;
    constexpr int kRowsPerBlock = kBlock / kGroup;
    const int lane_in_group = threadIdx.x % kGroup;
    const int group = threadIdx.x / kGroup;
    const int nv = cols / 4;
    for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock; row0 < rows;
         row0 += static_cast<int64_t>(gridDim.x) * kRowsPerBlock) {
        const bool live = row0 + group < rows;
        const int64_t row = live ? row0 + group : rows - 1;    // idle groups read the last row again
        V x[NV];
        T m = neg_inf<T>();
        // all loads of the row first (columns past the end read the last vector again and are
        // replaced below): a branch per vector would leave one load in flight
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            x[i] = src.load(row, c < nv ? c : nv - 1, cols);
        }
        if constexpr (Rows::kMasked) {
            V mk[NV];
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane_in_group + i * kGroup;
                mk[i] = src.load_mask(row, c < nv ? c : nv - 1);
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) src.combine(x[i], mk[i]);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            if (!(live && c < nv)) {
#pragma unroll
                for (int j = 0; j < 4; ++j) x[i].v[j] = neg_inf<T>();
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) m = x[i].v[j] > m ? x[i].v[j] : m;
        }
        m = wave_max(m);
        if constexpr (kGroup == kBlock) {
            const int wave = threadIdx.x / kWave;
            if ((threadIdx.x % kWave) == 0) red_buf[0][wave] = m;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) m = red_buf[0][w] > m ? red_buf[0][w] : m;
        }
        T sum = 0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // padding lanes hold -inf: exp(-inf - m) = 0 unless m is -inf too (all-masked row),
                // where IEEE gives NaN for real elements; keep padding at 0 in that case.
                T e = exp_t<T>(x[i].v[j] - m);
                const int c = lane_in_group + i * kGroup;
                if (!(live && c < nv)) e = 0;
                x[i].v[j] = e;
                sum += e;
            }
        }
        sum = wave_sum(sum);
        if constexpr (kGroup == kBlock) {
            const int wave = threadIdx.x / kWave;
            if ((threadIdx.x % kWave) == 0) red_buf[1][wave] = sum;
            __syncthreads();
            sum = 0;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) sum += red_buf[1][w];
            __syncthreads();
        }
        const T inv = static_cast<T>(1) / sum;
        V *po = reinterpret_cast<V *>(out + row * cols);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            if (live && c < nv) {
                V y;
#pragma unroll
                for (int j = 0; j < 4; ++j) y.v[j] = x[i].v[j] * inv;
                nt_store(po + c, y);
            }
        }
    }
}

// ---- Softmax fallback: [outer, n, inner], three passes over memory ----------------------------
// inner == 1: a wavefront per row. inner > 1: a thread per (outer, inner) pair (coalesced along
// inner), serial over the axis.
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(const T *__restrict__ in,
                                                              T *__restrict__ out, int64_t rows,
                                                              int64_t cols) {
    const int lane = threadIdx.x % kWave;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
         row < rows; row += static_cast<int64_t>(gridDim.x) * kWavesPerBlock) {
        const T *p = in + row * cols;
        T *q = out + row * cols;
        T m = neg_inf<T>();
        for (int64_t c = lane; c < cols; c += kWave) m = p[c] > m ? p[c] : m;
        m = wave_max(m);
        T sum = 0;
        for (int64_t c = lane; c < cols; c += kWave) sum += exp_t<T>(p[c] - m);
        sum = wave_sum(sum);
        const T inv = static_cast<T>(1) / sum;
        for (int64_t c = lane; c < cols; c += kWave) q[c] = exp_t<T>(p[c] - m) * inv;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_strided_kernel(const T *__restrict__ in,
                                                                 T *__restrict__ out,
                                                                 int64_t outer, int64_t n,
                                                                 int64_t inner) {
    const int64_t total = outer * inner;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < total;
         t += static_cast<int64_t>(gridDim.x) * kBlock) {
        const int64_t o = t / inner, i = t - o * inner;
        const T *p = in + o * n * inner + i;
        T *q = out + o * n * inner + i;
        T m = neg_inf<T>();
        for (int64_t c = 0; c < n; ++c) m = p[c * inner] > m ? p[c * inner] : m;
        T sum = 0;
        for (int64_t c = 0; c < n; ++c) sum += exp_t<T>(p[c * inner] - m);
        const T inv = static_cast<T>(1) / sum;
        for (int64_t c = 0; c < n; ++c) q[c * inner] = exp_t<T>(p[c * inner] - m) * inv;
    }
}

template <typename T, int NV, int kGroup, typename Rows>
int32_t launch_softmax_regs(hipStream_t s, const Rows &src, T *out, int64_t rows, int32_t cols) {
    constexpr int kRowsPerBlock = kBlock / kGroup;
    int64_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
    const int64_t cap = static_cast<int64_t>(kNumCU) * 64;
    if (blocks > cap) blocks = cap;
    softmax_regs_kernel<T, NV, kGroup, Rows><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(
        src, out, rows, cols);
    return launch_status();
}

// Same row-length ladder for the plain and the fused softmax, so both give the same bits.
template <typename T, typename Rows>
int32_t softmax_regs_dispatch(hipStream_t s, const Rows &src, T *out, int64_t rows, int32_t c) {
    if (c <= 256) return launch_softmax_regs<T, 1, kWave>(s, src, out, rows, c);
    if (c <= 512) return launch_softmax_regs<T, 2, kWave>(s, src, out, rows, c);
    if (c <= 1024) return launch_softmax_regs<T, 4, kWave>(s, src, out, rows, c);
    if (c <= 2048) return launch_softmax_regs<T, 8, kWave>(s, src, out, rows, c);
    if (c <= 4096) return launch_softmax_regs<T, 4, kBlock>(s, src, out, rows, c);
    if (c <= 8192) return launch_softmax_regs<T, 8, kBlock>(s, src, out, rows, c);
    return launch_softmax_regs<T, 16, kBlock>(s, src, out, rows, c);
}

template <typename T>
int32_t softmax_typed(hipStream_t s, int64_t outer, int64_t n, int64_t inner, const T *in,
                      T *out) {
    if (inner == 1) {
        const bool vec_ok = n % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                            reinterpret_cast<uintptr_t>(out) % 16 == 0 && n <= 16384 &&
                            sizeof(T) == 4;
        if (vec_ok)
            return softmax_regs_dispatch<T>(s, PlainRows<T>{in}, out, outer, static_cast<int32_t>(n));
        int64_t blocks = (outer + kWavesPerBlock - 1) / kWavesPerBlock;
        const int64_t cap = static_cast<int64_t>(kNumCU) * 32;
        if (blocks > cap) blocks = cap;
        softmax_rows_kernel<T><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(in, out, outer, n);
        return launch_status();
    }
    unsigned grid = grid_for(outer * inner, kBlock, 16);
    softmax_strided_kernel<T><<<grid, kBlock, 0, s>>>(in, out, outer, n, inner);
    return launch_status();
}

// ---- RMSNorm: y = x / sqrt(mean(x^2) + eps) * gamma, one pass, the row held in registers --------
// The fused form of Pow(2) -> ReduceMean(-1) -> Add(eps) -> Sqrt -> Div -> Mul(gamma): squares are
// rounded to float before the double accumulation and every later step rounds like the separate
// kernel does. RECIP selects the exported variant x * (1 / sqrt(..)) * gamma.
// The row may also be formed on the fly as x + add (the residual Add in front of the norm); the
// formed row is then stored to sum_out as well, because the residual stream reads it again later.
struct RmsSource {
    const float *x;       // the row
    const float *add;     // second Add operand, or null
    float *sum_out;       // where the formed row goes (null: nowhere)
    int32_t slabs;        // x is the first of this many partial matrices (split-K), summed in order
    int64_t slab;         // elements from one partial matrix to the next
    // The result also as three bfloat16 pieces whose sum it is exactly (hi, mid, lo: truncate,
    // subtract, truncate, subtract; Inf / NaN in hi alone), the operand form of rmlk_hip_matmul_bf16x3:
    // planes of `plane` elements each, rows of `cols`. Null: not wanted.
    uint16_t *pieces;
    int64_t plane;
};

template <int NV, int kGroup, bool RECIP>
__global__ __launch_bounds__(kBlock) void rmsnorm_kernel(RmsSource src,
                                                         const float *__restrict__ gamma,
                                                         float *__restrict__ out, int64_t rows,
                                                         int32_t cols, float eps) {
    __shared__ double partial[kWavesPerBlock];
    using V = Vec<float, 4>;
    constexpr int kRowsPerBlock = kBlock / kGroup;
    const int lane_in_group = threadIdx.x % kGroup;
    const int group = threadIdx.x / kGroup;
    const int nv = cols / 4;
    for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock; row0 < rows;
         row0 += static_cast<int64_t>(gridDim.x) * kRowsPerBlock) {
        const bool live = row0 + group < rows;
        const int64_t row = live ? row0 + group : rows - 1;    // idle groups read the last row again
        const V *pv = reinterpret_cast<const V *>(src.x + row * cols);
        V xv[NV];
        // every load of the row is issued before the first use (columns past the end read the last
        // vector again and are masked below): a branch per vector would leave one load in flight
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            xv[i] = nt_load(pv + (c < nv ? c : nv - 1));
        }
        // gamma after the row: its requests (the same 8 KB from every wavefront) queue behind the
        // row's, not in front of them
        V g[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            g[i] = reinterpret_cast<const V *>(gamma)[c < nv ? c : nv - 1];
        }
        if (src.slabs > 1) {
            for (int z = 1; z < src.slabs; ++z) {
                const V *pz = reinterpret_cast<const V *>(src.x + z * src.slab + row * cols);
                V more[NV];
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int c = lane_in_group + i * kGroup;
                    more[i] = nt_load(pz + (c < nv ? c : nv - 1));
                }
#pragma unroll
                for (int i = 0; i < NV; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) xv[i].v[j] = xv[i].v[j] + more[i].v[j];
            }
        }
        if (src.add) {
            const V *pa = reinterpret_cast<const V *>(src.add + row * cols);
            V av[NV];
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane_in_group + i * kGroup;
                av[i] = nt_load(pa + (c < nv ? c : nv - 1));
            }
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) xv[i].v[j] = xv[i].v[j] + av[i].v[j];
        }
        if (src.sum_out) {
            V *ps = reinterpret_cast<V *>(src.sum_out + row * cols);
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane_in_group + i * kGroup;
                if (live && c < nv) ps[c] = xv[i];
            }
        }
        double acc = 0.0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float sq = xv[i].v[j] * xv[i].v[j];
                acc += c < nv ? static_cast<double>(sq) : 0.0;
            }
        }
        acc = wave_sum(acc);
        if constexpr (kGroup == kBlock) {
            const int wave = threadIdx.x / kWave;
            if ((threadIdx.x % kWave) == 0) partial[wave] = acc;
            __syncthreads();
            acc = 0.0;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) acc += partial[w];
            __syncthreads();
        }
        const float mean = static_cast<float>(mean_of(acc, cols));
        const float var = mean + eps;
        const float r = sqrtf(var);
        const float inv = 1.0f / r;
        V *po = reinterpret_cast<V *>(out + row * cols);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane_in_group + i * kGroup;
            if (live && c < nv) {
                V y;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float normed = RECIP ? xv[i].v[j] * inv : xv[i].v[j] / r;
                    y.v[j] = normed * g[i].v[j];
                }
                nt_store(po + c, y);
                if (src.pieces) {
                    uint32_t hi[4], mid[4], lo[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t xb = __float_as_uint(y.v[j]);
                        const uint32_t hb = xb & 0xffff0000u;
                        const bool finite = (xb & 0x7f800000u) != 0x7f800000u;
                        const float r1 = finite ? y.v[j] - __uint_as_float(hb) : 0.f;
                        const uint32_t mb = __float_as_uint(r1) & 0xffff0000u;
                        const float r2 = r1 - __uint_as_float(mb);
                        hi[j] = hb >> 16;
                        mid[j] = mb >> 16;
                        lo[j] = __float_as_uint(r2) >> 16;
                    }
                    uint16_t *pp = src.pieces + row * cols + c * 4;
                    *reinterpret_cast<uint2 *>(pp) = uint2{hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16)};
                    *reinterpret_cast<uint2 *>(pp + src.plane) =
                        uint2{mid[0] | (mid[1] << 16), mid[2] | (mid[3] << 16)};
                    *reinterpret_cast<uint2 *>(pp + 2 * src.plane) =
                        uint2{lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16)};
                }
            }
        }
    }
}

template <int NV, int kGroup>
int32_t launch_rmsnorm(hipStream_t s, const RmsSource &src, const float *gamma, float *out,
                       int64_t rows, int32_t cols, float eps, bool recip) {
    constexpr int kRowsPerBlock = kBlock / kGroup;
    int64_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
    const int64_t cap = static_cast<int64_t>(kNumCU) * 32;
    if (blocks > cap) blocks = cap;
    const unsigned grid = static_cast<unsigned>(blocks);
    if (recip) rmsnorm_kernel<NV, kGroup, true><<<grid, kBlock, 0, s>>>(src, gamma, out, rows, cols, eps);
    else rmsnorm_kernel<NV, kGroup, false><<<grid, kBlock, 0, s>>>(src, gamma, out, rows, cols, eps);
    return launch_status();
}

int32_t rmsnorm_dispatch(hipStream_t s, const RmsSource &src, const float *gp, float *op, int64_t rows,
                         int64_t cols, float eps, bool recip) {
    auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool vec_ok = cols % 4 == 0 && aligned(src.x) && aligned(src.add) &&
                        aligned(src.sum_out) && aligned(gp) && aligned(op);
    if (!vec_ok || cols > kBlock * 4 * 8) return RMLK_ERR_UNSUPPORTED;
    const int32_t c = static_cast<int32_t>(cols);
    if (rows >= 1024 && c <= kWave * 4 * 8) {  // many rows: a wavefront per row
        if (c <= 256) return launch_rmsnorm<1, kWave>(s, src, gp, op, rows, c, eps, recip);
        if (c <= 512) return launch_rmsnorm<2, kWave>(s, src, gp, op, rows, c, eps, recip);
        if (c <= 1024) return launch_rmsnorm<4, kWave>(s, src, gp, op, rows, c, eps, recip);
        return launch_rmsnorm<8, kWave>(s, src, gp, op, rows, c, eps, recip);
    }
    if (c <= 1024) return launch_rmsnorm<1, kBlock>(s, src, gp, op, rows, c, eps, recip);
    if (c <= 2048) return launch_rmsnorm<2, kBlock>(s, src, gp, op, rows, c, eps, recip);
    if (c <= 4096) return launch_rmsnorm<4, kBlock>(s, src, gp, op, rows, c, eps, recip);
    return launch_rmsnorm<8, kBlock>(s, src, gp, op, rows, c, eps, recip);
}

template <typename T>
int32_t mean_typed(hipStream_t s, const rmlk_dims *shape, const bool *reduced, const T *in,
                   T *out) {
    const int rank = shape->rank;
    int64_t st[kMaxRank];
    dense_strides(rank, shape->v, st);
    // trailing run of reduced dims?
    int first_red = rank;
    while (first_red > 0 && reduced[first_red - 1]) --first_red;
    bool trailing = true;
    for (int d = 0; d < first_red; ++d)
        if (reduced[d]) trailing = false;
    int64_t n_out = 1, n_red = 1;
    for (int d = 0; d < rank; ++d) (reduced[d] ? n_red : n_out) *= shape->v[d];
    if (trailing) {
        const int64_t rows = n_out, cols = n_red;
        const bool vec_ok = cols % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                            sizeof(T) == 4;
        const bool block_per_row = rows < 2048 && cols >= 8192;
        if (block_per_row) {
            unsigned grid = static_cast<unsigned>(rows < 65536 ? rows : 65536);
            if (vec_ok) mean_rows_kernel<T, 4, kBlock><<<grid, kBlock, 0, s>>>(in, out, rows, cols);
            else mean_rows_kernel<T, 1, kBlock><<<grid, kBlock, 0, s>>>(in, out, rows, cols);
        } else {
            int64_t blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
            const int64_t cap = static_cast<int64_t>(kNumCU) * 32;
            if (blocks > cap) blocks = cap;
            unsigned grid = static_cast<unsigned>(blocks);
            if (vec_ok) mean_rows_kernel<T, 4, kWave><<<grid, kBlock, 0, s>>>(in, out, rows, cols);
            else mean_rows_kernel<T, 1, kWave><<<grid, kBlock, 0, s>>>(in, out, rows, cols);
        }
        return launch_status();
    }
    if (n_out >= ((int64_t)1 << 31) || n_red >= ((int64_t)1 << 31)) return RMLK_ERR_TOO_LARGE;
    int64_t kshape[kMaxRank], kst[1][kMaxRank], rshape[kMaxRank], rst[1][kMaxRank];
    int nk = 0, nr = 0;
    for (int d = 0; d < rank; ++d) {
        if (reduced[d]) {
            rshape[nr] = shape->v[d];
            rst[0][nr++] = st[d];
        } else {
            kshape[nk] = shape->v[d];
            kst[0][nk++] = st[d];
        }
    }
    if (nk == 0) {
        kshape[0] = 1;
        kst[0][0] = 0;
        nk = 1;
    }
    NdPlan<1> kept, red;
    build_plan<1>(kept, nk, kshape, kst);
    build_plan<1>(red, nr, rshape, rst);
    int64_t blocks = (n_out + kWavesPerBlock - 1) / kWavesPerBlock;
    const int64_t cap = static_cast<int64_t>(kNumCU) * 32;
    if (blocks > cap) blocks = cap;
    mean_generic_kernel<T><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(
        kept, red, in, out, static_cast<uint32_t>(n_out), static_cast<uint32_t>(n_red));
    return launch_status();
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_reduce_mean(rmlk_stream_t stream, int32_t dtype,
                                        const rmlk_dims *in_shape, const int64_t *axes,
                                        int32_t n_axes, const void *in, void *out) {
    if (!dims_ok(in_shape)) return RMLK_ERR_BAD_RANK;
    if (dtype != RMLK_FLOAT && dtype != RMLK_DOUBLE) return RMLK_ERR_UNSUPPORTED;
    if (n_axes < 1 || n_axes > in_shape->rank) return RMLK_ERR_INVALID_ARGUMENT;
    if (!axes) return RMLK_ERR_NULL_POINTER;
    bool reduced[kMaxRank] = {false};
    for (int i = 0; i < n_axes; ++i) {
        if (axes[i] < 0 || axes[i] >= in_shape->rank || reduced[axes[i]])
            return RMLK_ERR_INVALID_ARGUMENT;
        reduced[axes[i]] = true;
    }
    int64_t numel = dims_numel(in_shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    int64_t n_out = 1;
    for (int d = 0; d < in_shape->rank; ++d)
        if (!reduced[d]) n_out *= in_shape->v[d];
    if (n_out == 0) return RMLK_OK;
    // A reduced dim of extent 0 leaves outputs that are means of nothing: NaN, as 0/0.
    if (!out) return RMLK_ERR_NULL_POINTER;
    if (numel == 0) {
        if (dtype == RMLK_FLOAT) {
            float nan = __builtin_nanf("");
            return rmlk_hip_fill(stream, dtype, n_out, &nan, out);
        }
        double nan = __builtin_nan("");
        return rmlk_hip_fill(stream, dtype, n_out, &nan, out);
    }
    if (!in) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    if (dtype == RMLK_FLOAT)
        return mean_typed<float>(s, in_shape, reduced, static_cast<const float *>(in),
                                 static_cast<float *>(out));
    return mean_typed<double>(s, in_shape, reduced, static_cast<const double *>(in),
                              static_cast<double *>(out));
}

extern "C" int32_t rmlk_hip_softmax(rmlk_stream_t stream, int32_t dtype, int64_t outer,
                                    int64_t axis_len, int64_t inner, const void *in, void *out) {
    if (dtype != RMLK_FLOAT && dtype != RMLK_DOUBLE) return RMLK_ERR_UNSUPPORTED;
    if (outer < 0 || axis_len < 0 || inner < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (outer == 0 || axis_len == 0 || inner == 0) return RMLK_OK;
    if (outer > kMaxElems / axis_len || outer * axis_len > kMaxElems / inner)
        return RMLK_ERR_TOO_LARGE;
    if (!in || !out) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    if (dtype == RMLK_FLOAT)
        return softmax_typed<float>(s, outer, axis_len, inner, static_cast<const float *>(in),
                                    static_cast<float *>(out));
    return softmax_typed<double>(s, outer, axis_len, inner, static_cast<const double *>(in),
                                 static_cast<double *>(out));
}

extern "C" int32_t rmlk_hip_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows, int64_t cols,
                                    const void *x, const void *gamma, float eps,
                                    int32_t reciprocal_form, void *out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (rows < 0 || cols < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (rows == 0 || cols == 0) return RMLK_OK;
    if (!x || !gamma || !out) return RMLK_ERR_NULL_POINTER;
    if (rows > kMaxElems / cols) return RMLK_ERR_TOO_LARGE;
    RmsSource src{static_cast<const float *>(x), nullptr, nullptr, 1, 0, nullptr, 0};
    return rmsnorm_dispatch(as_stream(stream), src, static_cast<const float *>(gamma),
                            static_cast<float *>(out), rows, cols, eps, reciprocal_form != 0);
}

extern "C" int32_t rmlk_hip_add_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows,
                                        int64_t cols, const void *a, const void *b,
                                        const void *gamma, float eps, int32_t reciprocal_form,
                                        void *sum_out, void *out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (rows < 0 || cols < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (rows == 0 || cols == 0) return RMLK_OK;
    if (!a || !b || !gamma || !sum_out || !out) return RMLK_ERR_NULL_POINTER;
    if (rows > kMaxElems / cols) return RMLK_ERR_TOO_LARGE;
    RmsSource src{static_cast<const float *>(a), static_cast<const float *>(b),
                  static_cast<float *>(sum_out), 1, 0, nullptr, 0};
    return rmsnorm_dispatch(as_stream(stream), src, static_cast<const float *>(gamma),
                            static_cast<float *>(out), rows, cols, eps, reciprocal_form != 0);
}

extern "C" int32_t rmlk_hip_splitk_add_rmsnorm(rmlk_stream_t stream, int32_t dtype, int64_t rows,
                                               int64_t cols, const void *partials, int32_t splits,
                                               int64_t slab, const void *b, const void *gamma,
                                               float eps, int32_t reciprocal_form, void *sum_out,
                                               void *out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (rows < 0 || cols < 0 || splits < 1 || slab < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (rows == 0 || cols == 0) return RMLK_OK;
    if (!partials || !b || !gamma || !sum_out || !out) return RMLK_ERR_NULL_POINTER;
    if (rows > kMaxElems / cols) return RMLK_ERR_TOO_LARGE;
    if (splits > 1 && (slab < rows * cols || slab % 4 != 0)) return RMLK_ERR_SIZE_MISMATCH;
    RmsSource src{static_cast<const float *>(partials), static_cast<const float *>(b),
                  static_cast<float *>(sum_out), splits, slab, nullptr, 0};
    return rmsnorm_dispatch(as_stream(stream), src, static_cast<const float *>(gamma),
                            static_cast<float *>(out), rows, cols, eps, reciprocal_form != 0);
}

extern "C" int32_t rmlk_hip_rmsnorm_pieces(rmlk_stream_t stream, int64_t rows, int64_t cols,
                                           const void *partials, int32_t splits, int64_t slab, const void *b,
                                           const void *gamma, float eps, int32_t reciprocal_form,
                                           void *sum_out, void *out, void *pieces) {
    if (rows < 0 || cols < 0 || splits < 1 || slab < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (rows == 0 || cols == 0) return RMLK_OK;
    if (!partials || !gamma || !out || !pieces || (b && !sum_out)) return RMLK_ERR_NULL_POINTER;
    if (rows > kMaxElems / cols) return RMLK_ERR_TOO_LARGE;
    if (splits > 1 && (slab < rows * cols || slab % 4 != 0)) return RMLK_ERR_SIZE_MISMATCH;
    if (cols % 8 != 0 || reinterpret_cast<uintptr_t>(pieces) % 16 != 0) return RMLK_ERR_UNSUPPORTED;
    const int64_t m_pad = (rows + 127) / 128 * 128;      // (the planes of rmlk_hip_bf16x3_split)
    RmsSource src{static_cast<const float *>(partials), static_cast<const float *>(b),
                  b ? static_cast<float *>(sum_out) : nullptr, splits, slab,
                  static_cast<uint16_t *>(pieces), m_pad * cols};
    return rmsnorm_dispatch(as_stream(stream), src, static_cast<const float *>(gamma),
                            static_cast<float *>(out), rows, cols, eps, reciprocal_form != 0);
}

extern "C" int32_t rmlk_hip_scale_mask_softmax(rmlk_stream_t stream, int32_t dtype,
                                               const rmlk_dims *shape,
                                               const rmlk_dims *mask_stride, int32_t scale_is_mul,
                                               float scale, const void *x, const void *mask,
                                               void *out) {
    if (!dims_ok(shape) || !dims_ok(mask_stride) || mask_stride->rank != shape->rank)
        return RMLK_ERR_BAD_RANK;
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    const int rank = shape->rank;
    const int64_t numel = dims_numel(shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!x || !mask || !out) return RMLK_ERR_NULL_POINTER;
    const int64_t cols = shape->v[rank - 1], rows = numel / cols;
    if (mask_stride->v[rank - 1] != 1 && cols != 1) return RMLK_ERR_UNSUPPORTED;
    if (rows >= ((int64_t)1 << 31) || cols > 16384 || cols % 4 != 0) return RMLK_ERR_UNSUPPORTED;
    // leading dims -> at most three (extent, mask stride) pairs: drop extent 1, merge neighbours
    int64_t ext[kMaxRank], str[kMaxRank];
    int nd = 0;
    for (int d = 0; d < rank - 1; ++d) {
        if (shape->v[d] == 1) continue;
        const int64_t st = mask_stride->v[d];
        if (st < 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (nd > 0 && str[nd - 1] == st * shape->v[d]) {
            ext[nd - 1] *= shape->v[d];
            str[nd - 1] = st;
        } else {
            ext[nd] = shape->v[d];
            str[nd++] = st;
        }
    }
    if (nd > 3) return RMLK_ERR_UNSUPPORTED;
    for (int d = 0; d < nd; ++d)
        if (str[d] % 4 != 0) return RMLK_ERR_UNSUPPORTED;
    if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(mask) % 16 ||
        reinterpret_cast<uintptr_t>(out) % 16)
        return RMLK_ERR_UNSUPPORTED;
    // right-align into (i0, i1, i2)
    int64_t e3[3] = {1, 1, 1}, s3[3] = {0, 0, 0};
    for (int d = 0; d < nd; ++d) {
        e3[3 - nd + d] = ext[d];
        s3[3 - nd + d] = str[d];
    }
    RowMap map;
    map.n1 = static_cast<uint32_t>(e3[1]);
    map.n2 = static_cast<uint32_t>(e3[2]);
    map.d1 = FastDiv(map.n1);
    map.d2 = FastDiv(map.n2);
    map.s0 = s3[0];
    map.s1 = s3[1];
    map.s2 = s3[2];
    hipStream_t s = as_stream(stream);
    const float *xp = static_cast<const float *>(x), *mp = static_cast<const float *>(mask);
    float *op = static_cast<float *>(out);
    const int32_t c = static_cast<int32_t>(cols);
    if (scale_is_mul)
        return softmax_regs_dispatch<float>(s, ScaledMaskedRows<float, true>{xp, mp, scale, map}, op,
                                            rows, c);
    return softmax_regs_dispatch<float>(s, ScaledMaskedRows<float, false>{xp, mp, scale, map}, op,
                                        rows, c);
}
