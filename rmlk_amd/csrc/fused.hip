// Fused element-wise forms of operator chains that exported decoder graphs repeat in every layer.
// The reference runs each ONNX node as its own kernel (runtime/src/providers/cuda/backend/<op>.rs);
// these kernels compute the same chains in one pass over memory, with every intermediate rounded
// exactly like the separate kernel would round it (no contraction into fma), so a graph gives the
// same bits with or without them.
//
//   SwiGLU:  Mul(Mul(g, Sigmoid(g)), u)
//   Rotary:  Add(Mul(x, cos), Mul(Concat(Neg(Slice(x, D/2..D)), Slice(x, 0..D/2)), sin))
#include "common.hpp"

namespace rmlk {
namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__global__ __launch_bounds__(kBlock) void swiglu_kernel(const float *__restrict__ gate,
                                                        const float *__restrict__ up,
                                                        float *__restrict__ out, uint32_t n_vec) {
    using V = Vec<float, 4>;
    const V *g = reinterpret_cast<const V *>(gate);
    const V *u = reinterpret_cast<const V *>(up);
    V *o = reinterpret_cast<V *>(out);
    constexpr uint32_t U = 4;
    const uint32_t stride = gridDim.x * kBlock;
    uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    for (; i + (U - 1) * stride < n_vec; i += U * stride) {
        V gv[U], uv[U];
#pragma unroll
        for (uint32_t k = 0; k < U; ++k) {
            gv[k] = g[i + k * stride];
            uv[k] = u[i + k * stride];
        }
#pragma unroll
        for (uint32_t k = 0; k < U; ++k) {
            V y;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float silu = gv[k].v[j] * sigmoid_f(gv[k].v[j]);
                y.v[j] = silu * uv[k].v[j];
            }
            o[i + k * stride] = y;
        }
    }
    for (; i < n_vec; i += stride) {
        V gv = g[i], uv = u[i], y;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float silu = gv.v[j] * sigmoid_f(gv.v[j]);
            y.v[j] = silu * uv.v[j];
        }
        o[i] = y;
    }
}

__global__ __launch_bounds__(kBlock) void swiglu_tail_kernel(const float *__restrict__ gate,
                                                             const float *__restrict__ up,
                                                             float *__restrict__ out, int64_t begin,
                                                             int64_t n) {
    const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) {
        const float silu = gate[i] * sigmoid_f(gate[i]);
        out[i] = silu * up[i];
    }
}

// SwiGLU whose operands are still split-K partial rows of one GEMV over [gate | up] weights:
// gate_i = sum_z p[z][i], up_i = sum_z p[z][n + i] (z ascending), then as above.
__global__ __launch_bounds__(kBlock) void splitk_swiglu_kernel(const float *__restrict__ partials,
                                                               int32_t splits, int64_t slab,
                                                               float *__restrict__ out,
                                                               uint32_t n_vec, uint32_t up_off) {
    using V = Vec<float, 4>;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_vec; i += gridDim.x * kBlock) {
        const float *pg = partials + static_cast<int64_t>(i) * 4;
        V gv, uv;
#pragma unroll
        for (int j = 0; j < 4; ++j) gv.v[j] = uv.v[j] = 0.f;
        constexpr int kDepth = 8;   // slabs in ascending order, 16 loads in flight
        for (int z0 = 0; z0 < splits; z0 += kDepth) {
            V a[kDepth], b[kDepth];
#pragma unroll
            for (int u = 0; u < kDepth; ++u)
                if (z0 + u < splits) {
                    a[u] = *reinterpret_cast<const V *>(pg + (z0 + u) * slab);
                    b[u] = *reinterpret_cast<const V *>(pg + (z0 + u) * slab + up_off);
                }
#pragma unroll
            for (int u = 0; u < kDepth; ++u)
                if (z0 + u < splits) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        gv.v[j] += a[u].v[j];
                        uv.v[j] += b[u].v[j];
                    }
                }
        }
        V y;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float silu = gv.v[j] * sigmoid_f(gv.v[j]);
            y.v[j] = silu * uv.v[j];
        }
        reinterpret_cast<V *>(out)[i] = y;
    }
}

// Rotary embedding over x [B,H,S,D] read through element strides (the innermost stride is 1), so a
// [B,S,H,D] projection output is rotated and laid out [B,H,S,D] in the same pass. One lane takes W
// neighbouring elements of the first half of a row together with their partners in the second half.
// OFF: the type of element offsets - 32-bit when every operand ends below 2^31 elements (64-bit
// multiplies per dim and operand were most of the kernel's arithmetic). One trip: the grid covers
// the rows; x and the result stream past the caches, the tables (shared by the heads) stay in them.
template <typename OFF>
struct RotaryArgs {
    const float *x, *cos, *sin;
    float *out;
    FastDiv div_s, div_h, div_q;     // S, H, lanes per row
    uint32_t n_s, n_h, n_q, half;
    OFF xs[3], cs[3], ss[3];         // strides of (b, h, s)
    uint32_t total;                  // B * H * S * n_q
};

template <int W, typename OFF>
__global__ __launch_bounds__(kBlock) void rotary_kernel(RotaryArgs<OFF> a) {
    using V = Vec<float, W>;
    // (Four positions per lane, a quarter of the work apart, with all loads of x in front: 16.9 us
    // against the 15.0 us of one position per lane - the index arithmetic per position outweighs
    // what the deeper queue of loads gains.)
    const uint32_t t0 = blockIdx.x * kBlock + threadIdx.x;
    const bool live = t0 < a.total;
    const uint32_t t = live ? t0 : 0;     // (a lane past the end repeats lane 0's loads and stores nothing)
    const uint32_t row = a.div_q.div(t), q = t - row * a.n_q;
    const uint32_t bh = a.div_s.div(row), s = row - bh * a.n_s;
    const uint32_t b = a.div_h.div(bh), h = bh - b * a.n_h;
    const OFF xo = b * a.xs[0] + h * a.xs[1] + s * a.xs[2];
    const OFF co = b * a.cs[0] + h * a.cs[1] + s * a.cs[2];
    const OFF so = b * a.ss[0] + h * a.ss[1] + s * a.ss[2];
    const uint32_t d = q * W;
    const V x1 = nt_load(reinterpret_cast<const V *>(a.x + xo + d));
    const V x2 = nt_load(reinterpret_cast<const V *>(a.x + xo + d + a.half));
    const V c1 = *reinterpret_cast<const V *>(a.cos + co + d);
    const V c2 = *reinterpret_cast<const V *>(a.cos + co + d + a.half);
    const V s1 = *reinterpret_cast<const V *>(a.sin + so + d);
    const V s2 = *reinterpret_cast<const V *>(a.sin + so + d + a.half);
    V y1, y2;
#pragma unroll
    for (int j = 0; j < W; ++j) {
        const float a1 = x1.v[j] * c1.v[j];
        const float r1 = (-x2.v[j]) * s1.v[j];
        y1.v[j] = a1 + r1;
        const float a2 = x2.v[j] * c2.v[j];
        const float r2 = x1.v[j] * s2.v[j];
        y2.v[j] = a2 + r2;
    }
    if (live) {
        float *o = a.out + static_cast<int64_t>(row) * (2 * a.half) + d;
        nt_store(reinterpret_cast<V *>(o), y1);
        nt_store(reinterpret_cast<V *>(o + a.half), y2);
    }
}

// Up to kMaxRowStreams independent streams of head rows in ONE launch (blockIdx.y picks the stream):
// each reads rows of D elements through strides over (b, h, s) like rotary_kernel, rotates them
// (same expressions, same rounding) or moves them unchanged, and writes them either densely as
// [B,H,S,D] or to the rows of a ScatterND destination addressed by one index tuple per row
// (bounds and negative indices as scatter_nd_kernel handles them). That is what a decoder layer
// does behind its joint q/k/v projection: q rotated, k rotated into the key cache, v moved into
// the value cache, five launches otherwise.
constexpr int kMaxRowStreams = 4;
constexpr int kMaxRowTuple = 4;

struct RowStream {
    const float *x, *cos, *sin;      // cos == nullptr: rows are moved unchanged
    float *out;
    const int64_t *idx;              // nullptr: dense output
    FastDiv div_s, div_h;
    uint32_t n_s, n_h;
    uint32_t total;                  // B * H * S * n_q
    int32_t tuple_size;
    int32_t partials;                // x is the sum of this many slabs (split-K partial sums); <= 1: x itself
    int64_t partial_stride;          // elements from one slab to the next
    int64_t xs[3], cs[3], ss[3];     // strides of (b, h, s)
    int64_t dim[kMaxRowTuple], stride[kMaxRowTuple];   // leading dims of the scatter destination, in rows
};

struct RowStreams {
    RowStream s[kMaxRowStreams];
    FastDiv div_q;                   // lanes per row
    uint32_t n_q, half;
    int32_t *err;
};

template <int W>
__global__ __launch_bounds__(kBlock) void head_rows_kernel(RowStreams all) {
    using V = Vec<float, W>;
    const RowStream &a = all.s[blockIdx.y];
    for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < a.total; t += gridDim.x * kBlock) {
        const uint32_t row = all.div_q.div(t), q = t - row * all.n_q;
        const uint32_t bh = a.div_s.div(row), s = row - bh * a.n_s;
        const uint32_t b = a.div_h.div(bh), h = bh - b * a.n_h;
        const int64_t xo = b * a.xs[0] + h * a.xs[1] + s * a.xs[2];
        const uint32_t d = q * W;
        // the index tuple of the row first: its loads are then on their way together with the row's
        // (asked for after the arithmetic, they were a second trip to memory of a 4 us launch)
        int64_t ix[kMaxRowTuple];
        if (a.idx) {
#pragma unroll
            for (int k = 0; k < kMaxRowTuple; ++k)
                ix[k] = k < a.tuple_size ? a.idx[static_cast<int64_t>(row) * a.tuple_size + k] : 0;
        }
        V x1 = *reinterpret_cast<const V *>(a.x + xo + d);
        V x2 = *reinterpret_cast<const V *>(a.x + xo + d + all.half);
        // the rows of a split-K product that was not added up: slab 0 + slab 1 + .., in that order
        // (the order of the combine kernel this replaces)
        for (int z = 1; z < a.partials; ++z) {
            const float *pz = a.x + z * a.partial_stride + xo + d;
            const V p1 = *reinterpret_cast<const V *>(pz);
            const V p2 = *reinterpret_cast<const V *>(pz + all.half);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                x1.v[j] += p1.v[j];
                x2.v[j] += p2.v[j];
            }
        }
        V y1 = x1, y2 = x2;
        if (a.cos) {
            const int64_t co = b * a.cs[0] + h * a.cs[1] + s * a.cs[2];
            const int64_t so = b * a.ss[0] + h * a.ss[1] + s * a.ss[2];
            const V c1 = *reinterpret_cast<const V *>(a.cos + co + d);
            const V c2 = *reinterpret_cast<const V *>(a.cos + co + d + all.half);
            const V s1 = *reinterpret_cast<const V *>(a.sin + so + d);
            const V s2 = *reinterpret_cast<const V *>(a.sin + so + d + all.half);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                const float a1 = x1.v[j] * c1.v[j];
                const float r1 = (-x2.v[j]) * s1.v[j];
                y1.v[j] = a1 + r1;
                const float a2 = x2.v[j] * c2.v[j];
                const float r2 = x1.v[j] * s2.v[j];
                y2.v[j] = a2 + r2;
            }
        }
        int64_t out_row = row;
        if (a.idx) {
            out_row = 0;
            bool bad = false;
#pragma unroll
            for (int k = 0; k < kMaxRowTuple; ++k)
                if (k < a.tuple_size) {
                    int64_t i = ix[k];
                    if (i < 0) i += a.dim[k];
                    if (i < 0 || i >= a.dim[k]) bad = true;
                    out_row += i * a.stride[k];
                }
            if (bad) {
                if (all.err) *all.err = 1;
                continue;
            }
        }
        float *o = a.out + out_row * (2 * all.half) + d;
        *reinterpret_cast<V *>(o) = y1;
        *reinterpret_cast<V *>(o + all.half) = y2;
    }
}

}  // namespace
}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n, const void *gate,
                                   const void *up, void *out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n == 0) return RMLK_OK;
    if (!gate || !up || !out) return RMLK_ERR_NULL_POINTER;
    if (n > kMaxElems) return RMLK_ERR_TOO_LARGE;
    hipStream_t s = as_stream(stream);
    const float *g = static_cast<const float *>(gate), *u = static_cast<const float *>(up);
    float *o = static_cast<float *>(out);
    const bool aligned = reinterpret_cast<uintptr_t>(g) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(u) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(o) % 16 == 0;
    int64_t done = 0;
    if (aligned) {
        // pieces of at most 2^30 vectors keep the 32-bit index arithmetic in range
        const int64_t n_vec = n / 4;
        for (int64_t v0 = 0; v0 < n_vec; v0 += (int64_t)1 << 30) {
            const int64_t cnt = n_vec - v0 < ((int64_t)1 << 30) ? n_vec - v0 : (int64_t)1 << 30;
            swiglu_kernel<<<grid_for(cnt, kBlock * 4, 8), kBlock, 0, s>>>(
                g + v0 * 4, u + v0 * 4, o + v0 * 4, static_cast<uint32_t>(cnt));
        }
        done = n_vec * 4;
    }
    if (done < n) {
        const int64_t rest = n - done;
        const int64_t blocks = (rest + kBlock - 1) / kBlock;
        if (blocks >= ((int64_t)1 << 31)) return RMLK_ERR_TOO_LARGE;
        swiglu_tail_kernel<<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(g, u, o, done, n);
    }
    return launch_status();
}

extern "C" int32_t rmlk_hip_splitk_swiglu(rmlk_stream_t stream, int32_t dtype, int64_t n,
                                          const void *partials, int32_t splits, int64_t slab,
                                          int64_t gate_offset, int64_t up_offset, void *out) {
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    if (n < 0 || splits < 1 || gate_offset < 0 || up_offset < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (n == 0) return RMLK_OK;
    if (!partials || !out) return RMLK_ERR_NULL_POINTER;
    const float *p = static_cast<const float *>(partials) + gate_offset;
    const int64_t rel = up_offset - gate_offset;
    if (n % 4 || slab % 4 || rel % 4 || rel < 0 || n >= ((int64_t)1 << 32) ||
        reinterpret_cast<uintptr_t>(p) % 16 || reinterpret_cast<uintptr_t>(out) % 16)
        return RMLK_ERR_UNSUPPORTED;
    splitk_swiglu_kernel<<<grid_for(n / 4, kBlock, 8), kBlock, 0, as_stream(stream)>>>(
        p, splits, slab, static_cast<float *>(out), static_cast<uint32_t>(n / 4),
        static_cast<uint32_t>(rel));
    return launch_status();
}

extern "C" int32_t rmlk_hip_rotary(rmlk_stream_t stream, int32_t dtype, const rmlk_dims *shape,
                                   const rmlk_dims *x_stride, const rmlk_dims *cos_stride,
                                   const rmlk_dims *sin_stride, const void *x, const void *cos,
                                   const void *sin, void *out) {
    if (!dims_ok(shape) || !dims_ok(x_stride) || !dims_ok(cos_stride) || !dims_ok(sin_stride))
        return RMLK_ERR_BAD_RANK;
    if (shape->rank != 4 || x_stride->rank != 4 || cos_stride->rank != 4 || sin_stride->rank != 4)
        return RMLK_ERR_BAD_RANK;
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    const int64_t numel = dims_numel(shape);
    if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (numel == 0) return RMLK_OK;
    if (!x || !cos || !sin || !out) return RMLK_ERR_NULL_POINTER;
    const int64_t d = shape->v[3];
    if (d % 2 != 0) return RMLK_ERR_INVALID_ARGUMENT;
    if (x_stride->v[3] != 1 || cos_stride->v[3] != 1 || sin_stride->v[3] != 1)
        return RMLK_ERR_UNSUPPORTED;
    const int64_t half = d / 2;
    const int64_t rows = numel / d;
    for (int i = 0; i < 3; ++i)
        if (x_stride->v[i] < 0 || cos_stride->v[i] < 0 || sin_stride->v[i] < 0)
            return RMLK_ERR_INVALID_ARGUMENT;
    // widest lane width that keeps every access aligned
    auto ok = [&](int w) {
        if (half % w) return false;
        const uintptr_t mask = static_cast<uintptr_t>(w) * 4 - 1;
        if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(cos) |
             reinterpret_cast<uintptr_t>(sin) | reinterpret_cast<uintptr_t>(out)) & mask)
            return false;
        for (int i = 0; i < 3; ++i)
            if (x_stride->v[i] % w || cos_stride->v[i] % w || sin_stride->v[i] % w) return false;
        return true;
    };
    const int w = ok(4) ? 4 : ok(2) ? 2 : 1;
    const int64_t total = rows * (half / w);
    if (total >= ((int64_t)1 << 31) || numel >= ((int64_t)1 << 32)) return RMLK_ERR_TOO_LARGE;
    // the last element an operand's strides reach
    auto reach = [&](const rmlk_dims *st) {
        int64_t r = d;
        for (int i = 0; i < 3; ++i) r += (shape->v[i] - 1) * st->v[i];
        return r;
    };
    const bool narrow = reach(x_stride) < (1ll << 31) && reach(cos_stride) < (1ll << 31) &&
                        reach(sin_stride) < (1ll << 31);
    hipStream_t s = as_stream(stream);
    const unsigned grid = static_cast<unsigned>((total + kBlock - 1) / kBlock);   // one trip
    auto launch = [&](auto off_tag) {
        using OFF = decltype(off_tag);
        RotaryArgs<OFF> a;
        a.x = static_cast<const float *>(x);
        a.cos = static_cast<const float *>(cos);
        a.sin = static_cast<const float *>(sin);
        a.out = static_cast<float *>(out);
        a.n_s = static_cast<uint32_t>(shape->v[2]);
        a.n_h = static_cast<uint32_t>(shape->v[1]);
        a.n_q = static_cast<uint32_t>(half / w);
        a.half = static_cast<uint32_t>(half);
        a.div_s = FastDiv(a.n_s);
        a.div_h = FastDiv(a.n_h);
        a.div_q = FastDiv(a.n_q);
        for (int i = 0; i < 3; ++i) {
            a.xs[i] = static_cast<OFF>(x_stride->v[i]);
            a.cs[i] = static_cast<OFF>(cos_stride->v[i]);
            a.ss[i] = static_cast<OFF>(sin_stride->v[i]);
        }
        a.total = static_cast<uint32_t>(total);
        if (w == 4) rotary_kernel<4, OFF><<<grid, kBlock, 0, s>>>(a);
        else if (w == 2) rotary_kernel<2, OFF><<<grid, kBlock, 0, s>>>(a);
        else rotary_kernel<1, OFF><<<grid, kBlock, 0, s>>>(a);
    };
    if (narrow) launch(uint32_t{});
    else launch(int64_t{});
    return launch_status();
}

extern "C" int32_t rmlk_hip_head_rows(rmlk_stream_t stream, int32_t dtype, int32_t n_streams,
                                      const rmlk_row_stream *streams, int32_t *err_flag) {
    if (n_streams < 0 || n_streams > kMaxRowStreams) return RMLK_ERR_INVALID_ARGUMENT;
    if (n_streams == 0) return RMLK_OK;
    if (!streams) return RMLK_ERR_NULL_POINTER;
    if (dtype != RMLK_FLOAT) return RMLK_ERR_UNSUPPORTED;
    RowStreams all{};
    all.err = err_flag;
    int64_t d_common = -1, max_total = 0;
    int w = 4;
    int n_live = 0;
    for (int i = 0; i < n_streams; ++i) {
        const rmlk_row_stream &in = streams[i];
        const bool rotate = in.cos || in.sin;
        if (!dims_ok(&in.shape) || !dims_ok(&in.x_stride) || in.shape.rank != 4 || in.x_stride.rank != 4)
            return RMLK_ERR_BAD_RANK;
        if (rotate && (!dims_ok(&in.cos_stride) || !dims_ok(&in.sin_stride) ||
                       in.cos_stride.rank != 4 || in.sin_stride.rank != 4))
            return RMLK_ERR_BAD_RANK;
        const int64_t numel = dims_numel(&in.shape);
        if (numel < 0) return RMLK_ERR_INVALID_ARGUMENT;
        const int64_t d = in.shape.v[3];
        if (in.idx) {
            if (!dims_ok(&in.data_shape)) return RMLK_ERR_BAD_RANK;
            if (in.tuple_size < 1 || in.tuple_size != in.data_shape.rank - 1)
                return RMLK_ERR_INVALID_ARGUMENT;
            if (in.tuple_size > kMaxRowTuple) return RMLK_ERR_UNSUPPORTED;
            if (in.data_shape.v[in.tuple_size] != d || dims_numel(&in.data_shape) < 0)
                return RMLK_ERR_INVALID_ARGUMENT;
        }
        if (numel == 0) continue;
        if (!in.x || !in.out || (rotate && (!in.cos || !in.sin))) return RMLK_ERR_NULL_POINTER;
        if (d % 2 != 0) return RMLK_ERR_INVALID_ARGUMENT;
        if (d_common >= 0 && d != d_common) return RMLK_ERR_UNSUPPORTED;   // one row length per launch
        d_common = d;
        if (in.x_stride.v[3] != 1 || (rotate && (in.cos_stride.v[3] != 1 || in.sin_stride.v[3] != 1)))
            return RMLK_ERR_UNSUPPORTED;
        for (int k = 0; k < 3; ++k)
            if (in.x_stride.v[k] < 0 || (rotate && (in.cos_stride.v[k] < 0 || in.sin_stride.v[k] < 0)))
                return RMLK_ERR_INVALID_ARGUMENT;
        if (in.idx && dims_numel(&in.data_shape) >= ((int64_t)1 << 40)) return RMLK_ERR_TOO_LARGE;
        // widest lane width that keeps every access of every stream aligned
        auto ok = [&](int lanes) {
            if ((d / 2) % lanes) return false;
            const uintptr_t mask = static_cast<uintptr_t>(lanes) * 4 - 1;
            uintptr_t ptrs = reinterpret_cast<uintptr_t>(in.x) | reinterpret_cast<uintptr_t>(in.out);
            if (rotate) ptrs |= reinterpret_cast<uintptr_t>(in.cos) | reinterpret_cast<uintptr_t>(in.sin);
            if (ptrs & mask) return false;
            for (int k = 0; k < 3; ++k) {
                if (in.x_stride.v[k] % lanes) return false;
                if (rotate && (in.cos_stride.v[k] % lanes || in.sin_stride.v[k] % lanes)) return false;
            }
            return true;
        };
        while (w > 1 && !ok(w)) w /= 2;
        RowStream &a = all.s[n_live++];
        a.x = static_cast<const float *>(in.x);
        a.cos = rotate ? static_cast<const float *>(in.cos) : nullptr;
        a.sin = rotate ? static_cast<const float *>(in.sin) : nullptr;
        a.out = static_cast<float *>(in.out);
        a.idx = in.idx;
        a.n_s = static_cast<uint32_t>(in.shape.v[2]);
        a.n_h = static_cast<uint32_t>(in.shape.v[1]);
        a.div_s = FastDiv(a.n_s);
        a.div_h = FastDiv(a.n_h);
        for (int k = 0; k < 3; ++k) {
            a.xs[k] = in.x_stride.v[k];
            a.cs[k] = rotate ? in.cos_stride.v[k] : 0;
            a.ss[k] = rotate ? in.sin_stride.v[k] : 0;
        }
        a.tuple_size = in.idx ? in.tuple_size : 0;
        if (in.partials < 0 || in.partials > 64 || (in.partials > 1 && in.partial_stride <= 0))
            return RMLK_ERR_INVALID_ARGUMENT;
        if (in.partials > 1 && in.partial_stride % w) {
            while (w > 1 && in.partial_stride % w) w /= 2;
        }
        a.partials = in.partials;
        a.partial_stride = in.partial_stride;
        int64_t stride = 1;
        for (int k = a.tuple_size - 1; k >= 0; --k) {
            a.dim[k] = in.data_shape.v[k];
            a.stride[k] = stride;
            stride *= in.data_shape.v[k];
        }
        if (numel >= ((int64_t)1 << 32)) return RMLK_ERR_TOO_LARGE;
        a.total = static_cast<uint32_t>(numel / d);   // rows for now; lanes per row follow
    }
    if (n_live == 0) return RMLK_OK;
    const int64_t half = d_common / 2;
    all.half = static_cast<uint32_t>(half);
    all.n_q = static_cast<uint32_t>(half / w);
    all.div_q = FastDiv(all.n_q);
    for (int i = 0; i < n_live; ++i) {
        const int64_t total = static_cast<int64_t>(all.s[i].total) * all.n_q;
        if (total >= ((int64_t)1 << 31)) return RMLK_ERR_TOO_LARGE;
        all.s[i].total = static_cast<uint32_t>(total);
        max_total = total > max_total ? total : max_total;
    }
    const dim3 grid(grid_for(max_total, kBlock, 16), static_cast<unsigned>(n_live));
    hipStream_t s = as_stream(stream);
    if (w == 4) head_rows_kernel<4><<<grid, kBlock, 0, s>>>(all);
    else if (w == 2) head_rows_kernel<2><<<grid, kBlock, 0, s>>>(all);
    else head_rows_kernel<1><<<grid, kBlock, 0, s>>>(all);
    return launch_status();
}
