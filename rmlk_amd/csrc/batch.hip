// One launch for a run of operators over tiny tensors (see batch.hpp).
// The reference launches one kernel per operator whatever its size
// (runtime/src/core/instance.rs:100-112); there is no counterpart of the batch there.
#include <mutex>
#include <vector>

#include "batch.hpp"
#include "functors.hpp"

namespace rmlk {

std::atomic<int> g_open_batches{0};

namespace {

constexpr int kBatchThreads = 256;

struct SmallProgram {
    int32_t n_ops;
    int32_t reserved;
    SmallOp ops[kBatchMaxOps];
};
static_assert(sizeof(SmallProgram) <= 4096, "the records travel as kernel arguments");

// Element offsets of output element i in the operands of a record.
struct Offsets {
    int32_t in[3], out;
};
__device__ __forceinline__ Offsets offsets_of(const SmallOp &o, int32_t i) {
    Offsets f{{0, 0, 0}, 0};
    int32_t rem = i;
    for (int d = o.rank - 1; d >= 0; --d) {
        const int32_t c = rem % o.dim[d];
        rem /= o.dim[d];
        f.in[0] += c * o.st[0][d];
        f.in[1] += c * o.st[1][d];
        f.in[2] += c * o.st[2][d];
        f.out += c * o.st[3][d];
    }
    return f;
}

// The lanes that run a record: element i0, then every step-th (one or more wavefronts of the block).
struct Lanes {
    int32_t i0, step;
};

template <template <typename> class F, typename T, typename TO>
__device__ void run_binary(const SmallOp &o, Lanes l) {
    const T *a = static_cast<const T *>(o.in[0]), *b = static_cast<const T *>(o.in[1]);
    TO *out = static_cast<TO *>(o.out);
    for (int32_t i = l.i0; i < o.n; i += l.step) {
        const Offsets f = offsets_of(o, i);
        out[f.out] = F<T>::apply(a[f.in[0]], b[f.in[1]]);
    }
}

template <template <typename> class F, bool kCompare>
__device__ void binary_by_type(const SmallOp &o, Lanes l) {
    switch (o.dt) {
        case RMLK_FLOAT: run_binary<F, float, typename std::conditional<kCompare, uint8_t, float>::type>(o, l); break;
        case RMLK_DOUBLE: run_binary<F, double, typename std::conditional<kCompare, uint8_t, double>::type>(o, l); break;
        case RMLK_INT32: run_binary<F, int32_t, typename std::conditional<kCompare, uint8_t, int32_t>::type>(o, l); break;
        case RMLK_INT64: run_binary<F, int64_t, typename std::conditional<kCompare, uint8_t, int64_t>::type>(o, l); break;
        default: break;
    }
}

template <typename F, typename TI, typename TO>
__device__ void run_map(const SmallOp &o, Lanes l) {
    const TI *in = static_cast<const TI *>(o.in[0]);
    TO *out = static_cast<TO *>(o.out);
    for (int32_t i = l.i0; i < o.n; i += l.step) {
        const Offsets f = offsets_of(o, i);
        out[f.out] = F::apply(in[f.in[0]]);
    }
}

template <template <typename> class F>
__device__ void unary_by_type(const SmallOp &o, Lanes l) {
    if (o.dt == RMLK_FLOAT) run_map<F<float>, float, float>(o, l);
    else if (o.dt == RMLK_DOUBLE) run_map<F<double>, double, double>(o, l);
}

template <typename TI>
__device__ void cast_to(const SmallOp &o, Lanes l) {
    switch (o.dt2) {
        case RMLK_FLOAT: run_map<CastF<TI, float>, TI, float>(o, l); break;
        case RMLK_DOUBLE: run_map<CastF<TI, double>, TI, double>(o, l); break;
        case RMLK_INT32: run_map<CastF<TI, int32_t>, TI, int32_t>(o, l); break;
        case RMLK_INT64: run_map<CastF<TI, int64_t>, TI, int64_t>(o, l); break;
        case RMLK_BOOL: run_map<CastF<TI, BoolTag>, TI, BoolTag>(o, l); break;
        default: break;
    }
}

// Where and the copies move bits: typed by element size.
template <typename U>
__device__ void run_where(const SmallOp &o, Lanes l) {
    const U *x = static_cast<const U *>(o.in[0]), *y = static_cast<const U *>(o.in[1]);
    const uint8_t *cond = static_cast<const uint8_t *>(o.in[2]);
    U *out = static_cast<U *>(o.out);
    for (int32_t i = l.i0; i < o.n; i += l.step) {
        const Offsets f = offsets_of(o, i);
        out[f.out] = cond[f.in[2]] ? x[f.in[0]] : y[f.in[1]];
    }
}

template <typename U>
__device__ void run_copy(const SmallOp &o, Lanes l) {
    const U *in = static_cast<const U *>(o.in[0]);
    U *out = static_cast<U *>(o.out);
    for (int32_t i = l.i0; i < o.n; i += l.step) {
        const Offsets f = offsets_of(o, i);
        out[f.out] = in[f.in[0]];
    }
}

__device__ void run_record(const SmallOp &o, Lanes l) {
    switch (o.kind) {
        case kSmallBinary:
            switch (o.op) {
                case RMLK_ADD: binary_by_type<AddF, false>(o, l); break;
                case RMLK_SUB: binary_by_type<SubF, false>(o, l); break;
                case RMLK_MUL: binary_by_type<MulF, false>(o, l); break;
                case RMLK_DIV: binary_by_type<DivF, false>(o, l); break;
                case RMLK_EQUAL: binary_by_type<EqualF, true>(o, l); break;
                case RMLK_GREATER: binary_by_type<GreaterF, true>(o, l); break;
                default: break;
            }
            break;
        case kSmallUnary:
            switch (o.op) {
                case RMLK_SQRT: unary_by_type<SqrtF>(o, l); break;
                case RMLK_NEG: unary_by_type<NegF>(o, l); break;
                case RMLK_SIN: unary_by_type<SinF>(o, l); break;
                case RMLK_COS: unary_by_type<CosF>(o, l); break;
                case RMLK_SIGMOID: unary_by_type<SigmoidF>(o, l); break;
                default: break;
            }
            break;
        case kSmallCast:
            switch (o.dt) {
                case RMLK_FLOAT: cast_to<float>(o, l); break;
                case RMLK_DOUBLE: cast_to<double>(o, l); break;
                case RMLK_INT32: cast_to<int32_t>(o, l); break;
                case RMLK_INT64: cast_to<int64_t>(o, l); break;
                case RMLK_BOOL: cast_to<BoolTag>(o, l); break;
                default: break;
            }
            break;
        case kSmallWhere:
            switch (o.dt) {
                case 1: run_where<uint8_t>(o, l); break;
                case 2: run_where<uint16_t>(o, l); break;
                case 4: run_where<uint32_t>(o, l); break;
                case 8: run_where<uint64_t>(o, l); break;
                default: break;
            }
            break;
        case kSmallCopy:
            switch (o.dt) {
                case 1: run_copy<uint8_t>(o, l); break;
                case 2: run_copy<uint16_t>(o, l); break;
                case 4: run_copy<uint32_t>(o, l); break;
                case 8: run_copy<uint64_t>(o, l); break;
                default: break;
            }
            break;
        default: break;
    }
}

// One block runs the records in the order the host put them in: groups of records that do not touch
// each other's data, the block meeting after each group. A group's records run side by side: with
// four or more of them a wavefront each (record j on wavefront j % 4), fewer share the block's four
// wavefronts evenly. What a record wrote is complete and visible to the block (one compute unit, one
// L1) after the barrier behind its group.
// The records arrive as kernel arguments. Read one after the other through the argument pointer they
// cost a trip to that memory each (1.4 us per record measured, 17 us for the dozen of a decode step);
// every lane fetches a few words of them at once instead, into LDS, and the records are read there.
__global__ __launch_bounds__(kBatchThreads) void small_program_kernel(SmallProgram) {
    __shared__ SmallProgram sp;
    {
        const uint32_t *src = (const uint32_t *)__builtin_amdgcn_kernarg_segment_ptr();
        uint32_t *dst = reinterpret_cast<uint32_t *>(&sp);
        constexpr int kWords = sizeof(SmallProgram) / 4;
        static_assert(sizeof(SmallProgram) % 4 == 0, "copied in 32-bit words");
#pragma unroll
        for (int i = 0; i < (kWords + kBatchThreads - 1) / kBatchThreads; ++i) {
            const int w = i * kBatchThreads + threadIdx.x;
            if (w < kWords) dst[w] = src[w];
        }
    }
    __syncthreads();
    const int n_ops = sp.n_ops;
    constexpr int kWaves = kBatchThreads / kWave;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    for (int r = 0; r < n_ops; ++r) {
        const SmallOp &o = sp.ops[r];
        const int per_record = o.group_size >= kWaves ? 1 : kWaves / o.group_size;   // wavefronts of one record
        const int first = o.group_size >= kWaves ? o.group_index % kWaves : o.group_index * per_record;
        if (wave >= first && wave < first + per_record)
            run_record(o, Lanes{(wave - first) * kWave + lane, per_record * kWave});
        if (o.sync) __syncthreads();
    }
}

// Bytes an operand of a record may touch.
struct Span {
    uintptr_t lo, hi;   // [lo, hi); lo == hi: no such operand
};
struct Batch {
    hipStream_t stream;
    SmallProgram prog;
    Span reads[kBatchMaxOps][3], writes[kBatchMaxOps];
    int32_t error;
};
std::mutex g_mutex;
std::vector<Batch *> g_batches;

Batch *find_batch(hipStream_t s) {
    for (Batch *b : g_batches)
        if (b->stream == s) return b;
    return nullptr;
}

// Element sizes of the inputs and of the output of a record.
void element_sizes(const SmallOp &o, int (&in)[3], int &out) {
    const int sz = o.kind == kSmallWhere || o.kind == kSmallCopy ? o.dt : dtype_size(o.dt);
    in[0] = in[1] = in[2] = out = sz;
    if (o.kind == kSmallBinary && (o.op == RMLK_EQUAL || o.op == RMLK_GREATER)) out = 1;
    if (o.kind == kSmallCast) out = dtype_size(o.dt2);
    if (o.kind == kSmallWhere) in[2] = 1;
}

Span span_of(const SmallOp &o, int operand, const void *base, int esize) {
    if (!base) return Span{0, 0};
    int64_t last = 0;   // strides of a record are never negative
    for (int d = 0; d < o.rank; ++d) last += static_cast<int64_t>(o.dim[d] - 1) * o.st[operand][d];
    const uintptr_t lo = reinterpret_cast<uintptr_t>(base);
    return Span{lo, lo + static_cast<uintptr_t>(last + 1) * esize};
}

bool overlap(const Span &a, const Span &b) { return a.lo < b.hi && b.lo < a.hi; }

// Order the records for the launch: a record goes one group behind the last earlier record whose
// output it reads or overwrites, or whose inputs it overwrites; records of one group are independent
// of each other and keep their relative order. Groups are numbered within the launch.
void form_groups(Batch &b) {
    const int n = b.prog.n_ops;
    int level[kBatchMaxOps];
    int n_levels = 0;
    for (int r = 0; r < n; ++r) {
        level[r] = 0;
        for (int q = 0; q < r; ++q) {
            bool dep = overlap(b.writes[r], b.writes[q]);
            for (int i = 0; i < 3; ++i)
                dep = dep || overlap(b.reads[r][i], b.writes[q]) || overlap(b.writes[r], b.reads[q][i]);
            if (dep && level[q] + 1 > level[r]) level[r] = level[q] + 1;
        }
        if (level[r] + 1 > n_levels) n_levels = level[r] + 1;
    }
    SmallOp sorted[kBatchMaxOps];
    int at = 0;
    for (int l = 0; l < n_levels; ++l) {
        const int first = at;
        for (int r = 0; r < n; ++r)
            if (level[r] == l) sorted[at++] = b.prog.ops[r];
        for (int r = first; r < at; ++r) {
            sorted[r].group_size = at - first;
            sorted[r].group_index = r - first;
            sorted[r].sync = r == at - 1 ? 1 : 0;
        }
    }
    for (int r = 0; r < n; ++r) b.prog.ops[r] = sorted[r];
}

void send(Batch &b) {
    if (b.prog.n_ops == 0) return;
    form_groups(b);
    small_program_kernel<<<1, kBatchThreads, 0, b.stream>>>(b.prog);
    const int32_t st = launch_status();
    if (st && !b.error) b.error = st;
    b.prog.n_ops = 0;
}

}  // namespace

int32_t batch_flush_stream(hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_mutex);
    Batch *b = find_batch(s);
    if (!b) return RMLK_OK;
    send(*b);
    return b->error;
}

bool batch_take(hipStream_t s, const SmallOp &op) {
    std::lock_guard<std::mutex> lock(g_mutex);
    Batch *b = find_batch(s);
    if (!b) return false;
    if (b->prog.n_ops == kBatchMaxOps) send(*b);
    const int r = b->prog.n_ops++;
    b->prog.ops[r] = op;
    int in_size[3], out_size;
    element_sizes(op, in_size, out_size);
    for (int i = 0; i < 3; ++i) b->reads[r][i] = span_of(op, i, op.in[i], in_size[i]);
    b->writes[r] = span_of(op, 3, op.out, out_size);
    return true;
}

bool small_op_layout(SmallOp &op, int rank, const int64_t *shape, int n_in, const int64_t (*strides)[kMaxRank]) {
    int64_t n = 1;
    for (int d = 0; d < rank; ++d) n *= shape[d];
    if (n <= 0 || n > kBatchMaxElems || n_in < 1 || n_in > 3) return false;
    // operand rows of the record: inputs 0 .. n_in - 1, the output last
    const int rows[4] = {0, 1, 2, n_in};
    int64_t dim[kMaxRank], st[4][kMaxRank];
    int r = 0;
    for (int d = 0; d < rank; ++d) {
        if (shape[d] == 1) continue;
        dim[r] = shape[d];
        for (int p = 0; p < 4; ++p) st[p][r] = (p < n_in || p == 3) ? strides[rows[p]][d] : 0;
        ++r;
    }
    // merge dim d + 1 into d where every operand walks the two as one run
    for (int d = r - 2; d >= 0; --d) {
        bool one_run = true;
        for (int p = 0; p < 4; ++p) one_run = one_run && st[p][d] == st[p][d + 1] * dim[d + 1];
        if (!one_run) continue;
        dim[d] *= dim[d + 1];
        for (int p = 0; p < 4; ++p) st[p][d] = st[p][d + 1];
        for (int e = d + 1; e + 1 < r; ++e) {
            dim[e] = dim[e + 1];
            for (int p = 0; p < 4; ++p) st[p][e] = st[p][e + 1];
        }
        --r;
    }
    if (r == 0) {
        r = 1;
        dim[0] = 1;
        for (int p = 0; p < 4; ++p) st[p][0] = 0;
    }
    if (r > kBatchMaxRank) return false;
    // the kernel adds offsets up in 32 bits: the farthest element of every operand must stay below 2^31
    for (int p = 0; p < 4; ++p) {
        int64_t reach = 0;
        for (int d = 0; d < r; ++d) {
            const int64_t a = st[p][d] < 0 ? -st[p][d] : st[p][d];
            if (a > (1ll << 30)) return false;
            reach += (dim[d] - 1) * a;
        }
        if (reach >= (1ll << 31)) return false;
    }
    op.n = static_cast<int32_t>(n);
    op.rank = r;
    for (int d = 0; d < kBatchMaxRank; ++d) {
        op.dim[d] = d < r ? static_cast<int32_t>(dim[d]) : 1;
        for (int p = 0; p < 4; ++p) {
            const int64_t v = d < r ? st[p][d] : 0;
            if (v < -(1ll << 30) || v > (1ll << 30)) return false;
            op.st[p][d] = static_cast<int32_t>(v);
        }
    }
    return true;
}

}  // namespace rmlk

using namespace rmlk;

extern "C" int32_t rmlk_hip_batch_collects(const rmlk_dims *shape, int32_t n_in, const rmlk_dims *strides) {
    if (!shape || !strides || n_in < 1 || n_in > 3) return 0;
    if (shape->rank < 1 || shape->rank > kMaxRank) return 0;
    int64_t st[4][kMaxRank] = {};
    for (int p = 0; p <= n_in; ++p) {
        if (strides[p].rank != shape->rank) return 0;
        for (int d = 0; d < shape->rank; ++d) st[p][d] = strides[p].v[d];
    }
    SmallOp op{};
    return small_op_layout(op, shape->rank, shape->v, n_in, st) ? 1 : 0;
}

extern "C" int32_t rmlk_hip_batch_begin(rmlk_stream_t stream) {
    hipStream_t s = as_stream_collecting(stream);
    std::lock_guard<std::mutex> lock(g_mutex);
    if (find_batch(s)) return RMLK_ERR_INVALID_ARGUMENT;   // already collecting
    Batch *b = new Batch{};
    b->stream = s;
    g_batches.push_back(b);
    g_open_batches.fetch_add(1, std::memory_order_relaxed);
    return RMLK_OK;
}

extern "C" int32_t rmlk_hip_batch_flush(rmlk_stream_t stream) {
    return batch_flush_stream(as_stream_collecting(stream));
}

extern "C" int32_t rmlk_hip_batch_end(rmlk_stream_t stream) {
    hipStream_t s = as_stream_collecting(stream);
    std::lock_guard<std::mutex> lock(g_mutex);
    Batch *b = find_batch(s);
    if (!b) return RMLK_ERR_INVALID_ARGUMENT;
    send(*b);
    const int32_t st = b->error;
    for (size_t i = 0; i < g_batches.size(); ++i)
        if (g_batches[i] == b) {
            g_batches.erase(g_batches.begin() + i);
            break;
        }
    delete b;
    g_open_batches.fetch_sub(1, std::memory_order_relaxed);
    return st;
}
