// What the tests, the benchmark and the C++ host mirror need around the paged-KV library and an
// integration does not (include/breccia_kv_bench.h): device allocation, copies, streams, events,
// graph capture, and the bandwidth probes.  A library of its own, libbreccia_kv_bench.so; nothing
// here touches a pool.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/breccia_kv_bench.h"

namespace {

thread_local std::string g_bench_error;

bkv_status fail(bkv_status st, const std::string& msg) {
    g_bench_error = msg;
    return st;
}
bkv_status hip_fail(hipError_t e, const char* what) {
    g_bench_error = std::string(what) + " failed: " + hipGetErrorString(e);
    (void)hipGetLastError();
    return BKV_ERR_HIP;
}
#define BKV_HIP(call)                                     \
    do {                                                  \
        hipError_t e__ = (call);                          \
        if (e__ != hipSuccess) return hip_fail(e__, #call); \
    } while (0)

std::string sfmt(const char* f, long long a = 0, long long b = 0) {
    char buf[256];
    std::snprintf(buf, sizeof(buf), f, a, b);
    return buf;
}
inline hipStream_t S(void* s) { return reinterpret_cast<hipStream_t>(s); }
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kBlock = 256;

__global__ __launch_bounds__(kBlock) void copy_probe_kernel(uint4* __restrict__ dst,
                                                            const uint4* __restrict__ src,
                                                            uint64_t n_vec) {
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride],
                    d = src[i + 3 * stride];
        dst[i] = a;
        dst[i + stride] = b;
        dst[i + 2 * stride] = c;
        dst[i + 3 * stride] = d;
    }
    for (; i < n_vec; i += stride) dst[i] = src[i];
}

// Read-only bandwidth probe: every wave reads 8 KiB chunks (8 wave-loads of 1 KiB, the shape of
// one (page, kv head) run of a pool) and folds them into a value nothing depends on.  Chunk c of
// the walk is chunk c of the buffer, or, scattered, chunk (c * odd) mod n_chunks of it (n_chunks a
// power of two: a bijection), which is how a shuffled pool looks to the attention kernels.
typedef unsigned probe_v4u __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(kBlock) void read_probe_kernel(const probe_v4u* __restrict__ src, uint32_t n_chunks,
                                                            uint32_t scatter_mul, uint32_t* __restrict__ sink) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) >> 6;
    const uint32_t n_waves = gridDim.x * (kBlock / 64);
    probe_v4u acc = probe_v4u{0u, 0u, 0u, 0u};
    for (uint32_t c = wave; c < n_chunks; c += 2 * n_waves) {
        const uint32_t c1 = c + n_waves < n_chunks ? c + n_waves : c;
        const probe_v4u* a = src + (size_t)((c * scatter_mul) & (n_chunks - 1u)) * 512u + lane;
        const probe_v4u* b = src + (size_t)((c1 * scatter_mul) & (n_chunks - 1u)) * 512u + lane;
        probe_v4u r[16];
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = __builtin_nontemporal_load(a + i * 64);
#pragma unroll
        for (int i = 0; i < 8; ++i) r[8 + i] = __builtin_nontemporal_load(b + i * 64);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc ^= r[i];
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;  // keeps the loads alive
}

// The scattered walk again, every chunk fetched with 16-byte global->LDS loads instead of loads into
// registers (two 8 KiB slots per wave, the next chunk in flight while one word a lane of the landed
// one is folded): the mechanism the quantised attention kernels used first.  It streams about a tenth
// slower than the register path on this chip, which is why they moved off it; the probe keeps that
// comparison reproducible.
__global__ __launch_bounds__(kBlock) void read_probe_lds_kernel(const probe_v4u* __restrict__ src, uint32_t n_chunks,
                                                                uint32_t scatter_mul, uint32_t* __restrict__ sink) {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    __shared__ __attribute__((aligned(16))) probe_v4u stage[(kBlock / 64) * 2 * 512];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wv = threadIdx.x >> 6;
    const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) >> 6;
    const uint32_t n_waves = gridDim.x * (kBlock / 64);
    probe_v4u* const mine = stage + wv * 2 * 512;
    const auto request = [&](uint32_t c, uint32_t slot) {
        const probe_v4u* a = src + (size_t)((c * scatter_mul) & (n_chunks - 1u)) * 512u + lane;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            __builtin_amdgcn_global_load_lds((gptr)(a + i * 64), (lptr)(mine + slot * 512 + i * 64), 16, 0, 0);
    };
    probe_v4u acc = probe_v4u{0u, 0u, 0u, 0u};
    uint32_t slot = 0;
    if (wave < n_chunks) request(wave, 0);
    for (uint32_t c = wave; c < n_chunks; c += n_waves) {
        // the next chunk (or this one again past the end: the count of loads in flight stays 16)
        const uint32_t nx = c + n_waves < n_chunks ? c + n_waves : c;
        request(nx, slot ^ 1u);
        __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): the older eight have landed
        acc ^= mine[slot * 512 + lane];
        slot ^= 1u;
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): nothing may land in LDS after the wave has gone
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;
}

hipError_t launch_copy_probe(void* dst, const void* src, uint64_t bytes, hipStream_t stream) {
    const uint64_t n_vec = bytes / 16;
    if (n_vec == 0) return hipSuccess;
    uint64_t blocks = (n_vec + 4 * kBlock - 1) / (4 * kBlock);
    if (blocks > 8192) blocks = 8192;
    copy_probe_kernel<<<(unsigned)blocks, kBlock, 0, stream>>>((uint4*)dst, (const uint4*)src, n_vec);
    return hipGetLastError();
}

hipError_t launch_read_probe(const void* src, uint64_t bytes, int32_t mode, void* sink, int32_t n_cu,
                             hipStream_t stream) {
    const uint32_t n_chunks = (uint32_t)(bytes / 8192);
    if (n_chunks == 0) return hipSuccess;
    if (mode == 2) {
        // the decode kernels' launch shape: two 4-wave work-groups per compute unit, all resident
        uint32_t blocks = (uint32_t)(n_cu > 0 ? n_cu : 256) * 2u;
        if (blocks * (kBlock / 64) > n_chunks) blocks = (n_chunks + kBlock / 64 - 1) / (kBlock / 64);
        read_probe_lds_kernel<<<blocks, kBlock, 0, stream>>>((const probe_v4u*)src, n_chunks, 0x9e3779b1u, (uint32_t*)sink);
        return hipGetLastError();
    }
    // two resident generations of 4-wave work-groups at the decode kernels' occupancy
    uint32_t blocks = (uint32_t)(n_cu > 0 ? n_cu : 256) * 4u;
    if (blocks * (kBlock / 64) > n_chunks) blocks = (n_chunks + kBlock / 64 - 1) / (kBlock / 64);
    read_probe_kernel<<<blocks, kBlock, 0, stream>>>((const probe_v4u*)src, n_chunks, mode ? 0x9e3779b1u : 1u,
                                                     (uint32_t*)sink);
    return hipGetLastError();
}

}  // namespace

extern "C" {

const char* bkv_bench_last_error(void) { return g_bench_error.c_str(); }

bkv_status bkv_dev_alloc(uint64_t bytes, void** dev_out) {
    if (!dev_out) return fail(BKV_ERR_INVALID, "dev_alloc: NULL out pointer");
    BKV_HIP(hipMalloc(dev_out, bytes ? bytes : 16));
    return BKV_OK;
}
bkv_status bkv_dev_free(void* dev) {
    if (dev) BKV_HIP(hipFree(dev));
    return BKV_OK;
}
bkv_status bkv_memcpy_h2d(void* dev, const void* host, uint64_t bytes, void* stream) {
    BKV_HIP(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, S(stream)));
    return BKV_OK;
}
bkv_status bkv_memcpy_d2h(void* host, const void* dev, uint64_t bytes, void* stream) {
    BKV_HIP(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, S(stream)));
    return BKV_OK;
}
bkv_status bkv_graph_begin_capture(void* stream) {
    if (!stream) return fail(BKV_ERR_INVALID, "graph_begin_capture: the NULL stream cannot be captured");
    BKV_HIP(hipStreamBeginCapture(S(stream), hipStreamCaptureModeThreadLocal));
    return BKV_OK;
}

bkv_status bkv_graph_end_capture(void* stream, void** graph_exec_out) {
    if (!stream || !graph_exec_out) return fail(BKV_ERR_INVALID, "graph_end_capture: NULL argument");
    *graph_exec_out = nullptr;
    hipGraph_t graph = nullptr;
    BKV_HIP(hipStreamEndCapture(S(stream), &graph));
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate");
    *graph_exec_out = exec;
    return BKV_OK;
}

bkv_status bkv_graph_launch(void* graph_exec, void* stream) {
    if (!graph_exec) return fail(BKV_ERR_INVALID, "graph_launch: NULL graph");
    BKV_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), S(stream)));
    return BKV_OK;
}

bkv_status bkv_graph_destroy(void* graph_exec) {
    if (!graph_exec) return fail(BKV_ERR_INVALID, "graph_destroy: NULL graph");
    BKV_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return BKV_OK;
}

bkv_status bkv_stream_create(void** stream_out) {
    if (!stream_out) return fail(BKV_ERR_INVALID, "stream_create: NULL out pointer");
    hipStream_t s;
    BKV_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream_out = s;
    return BKV_OK;
}
bkv_status bkv_stream_destroy(void* stream) {
    if (stream) BKV_HIP(hipStreamDestroy(S(stream)));
    return BKV_OK;
}
bkv_status bkv_device_sync(void) {
    BKV_HIP(hipDeviceSynchronize());
    return BKV_OK;
}
bkv_status bkv_event_create(void** event_out) {
    if (!event_out) return fail(BKV_ERR_INVALID, "event_create: NULL out pointer");
    hipEvent_t e;
    BKV_HIP(hipEventCreate(&e));
    *event_out = e;
    return BKV_OK;
}
bkv_status bkv_event_destroy(void* event) {
    if (event) BKV_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return BKV_OK;
}
bkv_status bkv_event_record(void* event, void* stream) {
    BKV_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), S(stream)));
    return BKV_OK;
}
bkv_status bkv_event_sync(void* event) {
    BKV_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return BKV_OK;
}
bkv_status bkv_event_elapsed_ms(void* start, void* stop, float* ms_out) {
    if (!ms_out) return fail(BKV_ERR_INVALID, "event_elapsed_ms: NULL out pointer");
    BKV_HIP(hipEventElapsedTime(ms_out, reinterpret_cast<hipEvent_t>(start),
                                reinterpret_cast<hipEvent_t>(stop)));
    return BKV_OK;
}
bkv_status bkv_device_info(char* name_out, int32_t name_cap, int32_t* cu_out,
                           uint64_t* mem_bytes_out) {
    int dev = 0;
    BKV_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    BKV_HIP(hipGetDeviceProperties(&prop, dev));
    if (name_out && name_cap > 0) {
        std::snprintf(name_out, (size_t)name_cap, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (cu_out) *cu_out = prop.multiProcessorCount;
    if (mem_bytes_out) *mem_bytes_out = prop.totalGlobalMem;
    return BKV_OK;
}
bkv_status bkv_device_mem_info(uint64_t* free_out, uint64_t* total_out) {
    size_t f = 0, t = 0;
    BKV_HIP(hipMemGetInfo(&f, &t));
    if (free_out) *free_out = f;
    if (total_out) *total_out = t;
    return BKV_OK;
}
bkv_status bkv_copy_probe(void* dst_dev, const void* src_dev, uint64_t bytes, void* stream) {
    if (!dst_dev || !src_dev || !aligned16(dst_dev) || !aligned16(src_dev) || bytes % 16)
        return fail(BKV_ERR_INVALID, "copy_probe: pointers and size must be 16-byte multiples");
    BKV_HIP(launch_copy_probe(dst_dev, src_dev, bytes, S(stream)));
    return BKV_OK;
}

bkv_status bkv_read_probe(const void* src_dev, uint64_t bytes, int32_t scattered, void* sink_dev, void* stream) {
    if (!src_dev || !sink_dev || !aligned16(src_dev) || ((uintptr_t)sink_dev & 3u))
        return fail(BKV_ERR_INVALID, "read_probe: NULL or misaligned pointer");
    const uint64_t chunks = bytes / 8192;
    if (bytes % 8192 != 0 || chunks == 0 || chunks > 0x7fffffffull || (chunks & (chunks - 1)) != 0)
        return fail(BKV_ERR_INVALID, sfmt("read_probe: %lld bytes; need a power-of-two number of 8 KiB chunks",
                                          (long long)bytes));
    if (scattered < 0 || scattered > 2)
        return fail(BKV_ERR_INVALID, sfmt("read_probe: order %lld (0 = address order, 1 = scattered, 2 = scattered "
                                          "through global->LDS loads)", scattered));
    int dev = 0, n_cu = 0;
    BKV_HIP(hipGetDevice(&dev));
    BKV_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    BKV_HIP(launch_read_probe(src_dev, bytes, scattered, sink_dev, n_cu, S(stream)));
    return BKV_OK;
}

// The host polls the stream for a few milliseconds before it blocks: a thread that sleeps in
// hipStreamSynchronize is woken some tens of microseconds after the stream has drained.  (The
// product's own bounded wait is bkv_stream_wait.)
bkv_status bkv_stream_sync(void* stream) {
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
        const hipError_t e = hipStreamQuery(S(stream));
        if (e == hipSuccess) return BKV_OK;
        if (e != hipErrorNotReady) return hip_fail(e, "hipStreamQuery");
        (void)hipGetLastError();
        if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(4)) break;
        __builtin_ia32_pause();
    }
    BKV_HIP(hipStreamSynchronize(S(stream)));
    return BKV_OK;
}

}  // extern "C"
