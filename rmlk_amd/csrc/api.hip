// Memory, stream and device helpers of the C ABI, plus status strings.
// What the reference's provider reaches through cudarc: allocation
// (runtime/src/providers/cuda/allocator.rs:96-139), host/device copies
// (runtime/src/providers/cuda/store.rs:385-416) and the blocking readback of outputs
// (runtime/src/core/execution_state.rs:201-225).
#include <cstring>

#include "common.hpp"

using namespace rmlk;

extern "C" int32_t rmlk_hip_malloc(void **ptr, size_t bytes) {
    if (!ptr) return RMLK_ERR_NULL_POINTER;
    *ptr = nullptr;
    if (bytes == 0) return RMLK_OK;
    return static_cast<int32_t>(hipMalloc(ptr, bytes));
}

extern "C" int32_t rmlk_hip_free(void *ptr) {
    if (!ptr) return RMLK_OK;
    return static_cast<int32_t>(hipFree(ptr));
}

extern "C" int32_t rmlk_hip_memcpy_htod(rmlk_stream_t stream, void *dst, const void *src,
                                        size_t bytes) {
    if (bytes == 0) return RMLK_OK;
    if (!dst || !src) return RMLK_ERR_NULL_POINTER;
    return static_cast<int32_t>(
        hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
}

extern "C" int32_t rmlk_hip_memcpy_dtoh(rmlk_stream_t stream, void *dst, const void *src,
                                        size_t bytes) {
    if (bytes == 0) return RMLK_OK;
    if (!dst || !src) return RMLK_ERR_NULL_POINTER;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream));
    if (e != hipSuccess) return static_cast<int32_t>(e);
    return static_cast<int32_t>(hipStreamSynchronize(as_stream(stream)));
}

// Byte fill through the fill kernels (never hipMemsetAsync): safe to record into a HIP graph, where
// memset nodes have given wrong results on replays after the first. Head and tail bytes go one by one,
// the 8-byte aligned middle as 64-bit words.
extern "C" int32_t rmlk_hip_memset(rmlk_stream_t stream, void *dst, int32_t byte, size_t bytes) {
    if (bytes == 0) return RMLK_OK;
    if (!dst) return RMLK_ERR_NULL_POINTER;
    const uint8_t b = static_cast<uint8_t>(byte);
    uint8_t *p = static_cast<uint8_t *>(dst);
    size_t head = (8 - reinterpret_cast<uintptr_t>(p) % 8) % 8;
    if (head > bytes) head = bytes;
    const size_t words = (bytes - head) / 8;
    const size_t tail = bytes - head - words * 8;
    const uint64_t word = 0x0101010101010101ull * b;
    int32_t st = RMLK_OK;
    if (head) st = rmlk_hip_fill(stream, RMLK_UINT8, static_cast<int64_t>(head), &b, p);
    if (!st && words) st = rmlk_hip_fill(stream, RMLK_UINT64, static_cast<int64_t>(words), &word, p + head);
    if (!st && tail) st = rmlk_hip_fill(stream, RMLK_UINT8, static_cast<int64_t>(tail), &b, p + head + words * 8);
    return st;
}

// ---- streaming yardsticks --------------------------------------------------------------------------
// The least a kernel can do with N bytes on this chip: every lane requests all its 128-bit units up
// front (streaming loads), the grid covers the bytes in one trip. Benchmarks time these next to the
// operators of the same traffic; with `stamps` a block also notes the constant 100 MHz clock when it
// starts and when it ends, so that the time between the first block's start and the last block's
// end (what the memory system needs) can be told from what a trace adds around it (dispatch).
namespace rmlk {
namespace {
using U128 = Vec<uint32_t, 4>;

__device__ __forceinline__ void note(uint64_t *stamps, uint64_t t0) {
    if (stamps && threadIdx.x == 0) {
        stamps[2 * blockIdx.x] = t0;
        stamps[2 * blockIdx.x + 1] = wall_clock64();
    }
}

// 32 KiB per block: 8 units per lane
__global__ __launch_bounds__(256) void yardstick_read_kernel(const U128 *__restrict__ in, uint32_t *__restrict__ out,
                                                             uint64_t *stamps) {
    const uint64_t t0 = stamps ? wall_clock64() : 0;
    const size_t base = static_cast<size_t>(blockIdx.x) * 2048 + threadIdx.x;
    U128 r[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) r[u] = nt_load(in + base + u * 256);
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += r[u].v[0] ^ r[u].v[1] ^ r[u].v[2] ^ r[u].v[3];
    if (acc == 0x9e3779b9u && out) out[blockIdx.x] = acc;   // keeps the loads alive; writes next to nothing
    note(stamps, t0);
}

// 16 KiB in and 16 KiB out per block: 4 units per lane
__global__ __launch_bounds__(256) void yardstick_copy_kernel(const U128 *__restrict__ in, U128 *__restrict__ out,
                                                             uint64_t *stamps) {
    const uint64_t t0 = stamps ? wall_clock64() : 0;
    const size_t base = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
    U128 r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) r[u] = nt_load(in + base + u * 256);
#pragma unroll
    for (int u = 0; u < 4; ++u) nt_store(out + base + u * 256, r[u]);
    note(stamps, t0);
}
}  // namespace
}  // namespace rmlk

extern "C" int32_t rmlk_hip_stream_yardstick(rmlk_stream_t stream, int32_t kind, size_t bytes, const void *src,
                                             void *dst, uint64_t *stamps) {
    if (kind != RMLK_YARDSTICK_READ && kind != RMLK_YARDSTICK_COPY) return RMLK_ERR_INVALID_ARGUMENT;
    const size_t chunk = kind == RMLK_YARDSTICK_READ ? 32768 : 16384;
    if (bytes == 0 || bytes % chunk != 0 || bytes / chunk > 0x7fffffffu) return RMLK_ERR_INVALID_ARGUMENT;
    if (!src || !dst) return RMLK_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(dst) % 16) return RMLK_ERR_INVALID_ARGUMENT;
    const unsigned grid = static_cast<unsigned>(bytes / chunk);
    hipStream_t s = as_stream(stream);
    if (kind == RMLK_YARDSTICK_READ)
        yardstick_read_kernel<<<grid, 256, 0, s>>>(static_cast<const U128 *>(src), static_cast<uint32_t *>(dst), stamps);
    else
        yardstick_copy_kernel<<<grid, 256, 0, s>>>(static_cast<const U128 *>(src), static_cast<U128 *>(dst), stamps);
    return launch_status();
}

// ---- issue yardstick -------------------------------------------------------------------------------
// What a SIMD does with other instructions beside fp32 MFMAs. A block of eight wavefronts, two per
// SIMD: wavefronts 0..3 issue v_mfma_f32_32x32x2_f32 with something between them, wavefronts 4..7
// (when asked) run a chain of dependent v_fma_f32 meanwhile; every wavefront notes the shader clock
// cycles it took. Kinds 0, 4, 8, 12, 16: ONE chain of MFMAs, that many independent v_fma_f32 behind
// each. Kinds 100..103: four accumulators in turn (independent MFMAs, as in a GEMM step) and behind
// every fourth MFMA nothing / one v_add_u32 / one ds_read_b128 / a v_add_u32 and the ds_read_b128
// that takes its result as the address. Benchmarks read from it which instructions of a kernel run
// in the shadow of its MFMAs and which add to them.
namespace rmlk {
namespace {
typedef float IssueAcc __attribute__((ext_vector_type(16)));
typedef float IssueFrag __attribute__((ext_vector_type(4)));

template <int KIND>
__global__ __launch_bounds__(512) void yardstick_issue_kernel(int second, int iterations, uint64_t *cycles) {
    __shared__ float lds[4096];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if constexpr (KIND >= 102) {
        for (int i = threadIdx.x; i < 4096; i += 512) lds[i] = i * 0.001f;
        __syncthreads();
    }
    long long t0 = 0, t1 = 0;
    float res = 0.f;
    const float m = 0.999f, c = 0.0001f;
    if (wave < 4) {
        IssueAcc acc[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[k][j] = 0.f;
        const float a = lane * 0.001f, b = 1.0f + lane * 0.002f;
        float x[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) x[j] = lane * 0.01f + j;
        uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + lane * 16;
        const uint32_t step = 1024;
        IssueFrag frag = {0.f, 0.f, 0.f, 0.f};
        t0 = clock64();
        for (int i = 0; i < iterations; ++i) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                constexpr int kAccs = KIND >= 100 ? 4 : 1;
                acc[j % kAccs] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j % kAccs], 0, 0, 0);
                if constexpr (KIND < 100) {
#pragma unroll
                    for (int v = 0; v < KIND; ++v) x[v % 16] = __builtin_fmaf(x[v % 16], m, c);
                } else if (j % 4 == 0) {
                    // (the address walks over 4 KiB of the 16 KiB array and comes back)
                    if constexpr (KIND == 101 || KIND == 103)
                        asm volatile("v_add_u32 %0, %0, %1" : "+v"(addr) : "s"(j == 12 ? 0u - 3u * step : step));
                    if constexpr (KIND == 102 || KIND == 103)
                        asm volatile("ds_read_b128 %0, %1" : "=v"(frag) : "v"(addr));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        res = frag[0] + frag[3];
#pragma unroll
        for (int j = 0; j < 16; ++j) res += acc[0][j] + acc[1][j] + acc[2][j] + acc[3][j] + x[j];
        asm volatile("" : "+v"(res));
        t1 = clock64();
    } else if (second) {
        float x0 = lane * 0.001f;
        t0 = clock64();
        for (int i = 0; i < iterations; ++i) {
#pragma unroll
            for (int j = 0; j < 64; ++j) x0 = __builtin_fmaf(x0, m, c);
        }
        res = x0;
        asm volatile("" : "+v"(res));
        t1 = clock64();
    }
    if (lane == 0) cycles[blockIdx.x * 8 + wave] = static_cast<uint64_t>(t1 - t0) + (res == 12345.678f ? 1 : 0);
}
}  // namespace
}  // namespace rmlk

extern "C" int32_t rmlk_hip_issue_yardstick(rmlk_stream_t stream, int32_t kind, int32_t second_wavefront,
                                            int32_t iterations, int32_t blocks, uint64_t *cycles) {
    if (iterations <= 0 || iterations > (1 << 20) || blocks <= 0 || blocks > 65535) return RMLK_ERR_INVALID_ARGUMENT;
    if (!cycles) return RMLK_ERR_NULL_POINTER;
    hipStream_t s = as_stream(stream);
    const int second = second_wavefront ? 1 : 0;
    switch (kind) {
        case 0: yardstick_issue_kernel<0><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 4: yardstick_issue_kernel<4><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 8: yardstick_issue_kernel<8><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 12: yardstick_issue_kernel<12><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 16: yardstick_issue_kernel<16><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 100: yardstick_issue_kernel<100><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 101: yardstick_issue_kernel<101><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 102: yardstick_issue_kernel<102><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        case 103: yardstick_issue_kernel<103><<<blocks, 512, 0, s>>>(second, iterations, cycles); break;
        default: return RMLK_ERR_INVALID_ARGUMENT;
    }
    return launch_status();
}

extern "C" int32_t rmlk_hip_stream_sync(rmlk_stream_t stream) {
    return static_cast<int32_t>(hipStreamSynchronize(as_stream(stream)));
}

extern "C" int32_t rmlk_hip_device_info(int32_t device, rmlk_device_info *info) {
    if (!info) return RMLK_ERR_NULL_POINTER;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return static_cast<int32_t>(e);
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->name, prop.name, sizeof(info->name) - 1);
    std::strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->lds_bytes_per_block = static_cast<int32_t>(prop.sharedMemPerBlock);
    info->clock_khz = prop.clockRate;
    info->total_mem_bytes = static_cast<int64_t>(prop.totalGlobalMem);
    return RMLK_OK;
}

extern "C" const char *rmlk_hip_status_string(int32_t status) {
    switch (status) {
        case RMLK_OK: return "ok";
        case RMLK_ERR_BAD_RANK: return "rank outside 1..8";
        case RMLK_ERR_UNSUPPORTED: return "unsupported data type";
        case RMLK_ERR_NULL_POINTER: return "null pointer with non-zero length";
        case RMLK_ERR_SIZE_MISMATCH: return "size mismatch";
        case RMLK_ERR_INVALID_ARGUMENT: return "invalid argument";
        case RMLK_ERR_WORKSPACE: return "workspace too small";
        case RMLK_ERR_TOO_LARGE: return "tensor too large";
        case RMLK_ERR_SCRATCH_LIMIT: return "problem needs more scratch memory than the no-allocation entry point holds";
        default:
            if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
            return "unknown status";
    }
}

extern "C" const char *rmlk_hip_version(void) { return "0.1.0"; }
