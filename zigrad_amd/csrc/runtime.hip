// Context, memory API and the caching allocator of the gfx950 backend.
//
// Mirrors the memory half of the reference's device interface
// (src/device/device_reference.zig:29-131, src/device/host_device.zig:876-958) and supplies the
// DataHandler primitives src/allocators/caching_allocator.zig expects from a device.
#include "common.h"

#include <cmath>
#include <mutex>

namespace zg {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

void* workspace(zg_hip_ctx* ctx, size_t bytes) {
    if (bytes <= ctx->ws_bytes) return ctx->ws;
    if (ctx->capturing) {
        set_error("workspace: needs to grow to %zu bytes while an execution graph is being captured; run the same "
                  "ops once eagerly first", bytes);
        return nullptr;
    }
    // grow: nothing may still be reading the old buffer
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
        set_error("workspace: stream synchronize failed");
        return nullptr;
    }
    size_t want = ctx->ws_bytes ? ctx->ws_bytes : (size_t)1 << 20;
    while (want < bytes) want *= 2;
    void* p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) {
        (void)hipGetLastError();
        set_error("workspace: hipMalloc(%zu) failed", want);
        return nullptr;
    }
    ctx->n_device_allocs++;
    if (ctx->ws) {
        // an instantiated graph may have recorded the old address: keep it alive until the context goes
        if (ctx->live_graphs > 0) ctx->retired_ws.push_back(ctx->ws);
        else (void)hipFree(ctx->ws);
    }
    ctx->ws = p;
    ctx->ws_bytes = want;
    return p;
}

// ------------------------------------------------------------------------------------------------
// Block pool: a coalescing free-list allocator over device segments obtained with hipMalloc.
// Counterpart of src/allocators/block_pool.zig:103-412 (split on alloc, fuse with free neighbours on
// free); segments are added on demand instead of mapping one region of the whole device up front, so
// steady-state training never reaches hipMalloc once the working set has been seen.
// ------------------------------------------------------------------------------------------------
struct Block {
    char* ptr;
    size_t size;
    bool free;
    int segment;
};

struct BlockPool {
    size_t segment_bytes;
    size_t min_split;
    std::vector<void*> segments;
    std::map<char*, Block> blocks;                 // by address
    std::multimap<size_t, char*> free_by_size;     // free blocks by size
    size_t in_use = 0;
    size_t mapped = 0;

    void erase_free(const Block& b) {
        auto range = free_by_size.equal_range(b.size);
        for (auto it = range.first; it != range.second; ++it) {
            if (it->second == b.ptr) {
                free_by_size.erase(it);
                return;
            }
        }
    }

    bool add_segment(zg_hip_ctx* ctx, size_t at_least) {
        if (ctx->capturing) return false;  // no driver allocation inside a graph capture
        size_t bytes = segment_bytes;
        while (bytes < at_least) bytes *= 2;
        void* p = nullptr;
        if (hipMalloc(&p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            // retry with exactly what is needed
            bytes = (at_least + min_split - 1) / min_split * min_split;
            if (hipMalloc(&p, bytes) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
        }
        ctx->n_device_allocs++;
        int seg = (int)segments.size();
        segments.push_back(p);
        mapped += bytes;
        Block b{(char*)p, bytes, true, seg};
        blocks[b.ptr] = b;
        free_by_size.insert({bytes, b.ptr});
        return true;
    }

    void* alloc(zg_hip_ctx* ctx, size_t bytes) {
        size_t need = (bytes + min_split - 1) / min_split * min_split;
        auto it = free_by_size.lower_bound(need);
        if (it == free_by_size.end()) {
            if (!add_segment(ctx, need)) return nullptr;
            it = free_by_size.lower_bound(need);
            if (it == free_by_size.end()) return nullptr;
        }
        char* p = it->second;
        free_by_size.erase(it);
        Block& b = blocks[p];
        if (b.size - need >= min_split) {
            Block rest{p + need, b.size - need, true, b.segment};
            b.size = need;
            blocks[rest.ptr] = rest;
            free_by_size.insert({rest.size, rest.ptr});
        }
        b.free = false;
        in_use += b.size;
        return p;
    }

    bool release(void* ptr) {
        auto it = blocks.find((char*)ptr);
        if (it == blocks.end() || it->second.free) return false;
        Block& b = it->second;
        in_use -= b.size;
        b.free = true;
        // fuse with the next block of the same segment
        auto nx = std::next(it);
        if (nx != blocks.end() && nx->second.free && nx->second.segment == b.segment &&
            nx->second.ptr == b.ptr + b.size) {
            erase_free(nx->second);
            b.size += nx->second.size;
            blocks.erase(nx);
        }
        // fuse with the previous block
        if (it != blocks.begin()) {
            auto pv = std::prev(it);
            if (pv->second.free && pv->second.segment == b.segment && pv->second.ptr + pv->second.size == b.ptr) {
                erase_free(pv->second);
                pv->second.size += b.size;
                blocks.erase(it);
                it = pv;
            }
        }
        free_by_size.insert({it->second.size, it->second.ptr});
        return true;
    }

    bool owns(void* ptr) const {
        return blocks.find((char*)ptr) != blocks.end();
    }
    bool owns_live(void* ptr) const {
        auto it = blocks.find((char*)ptr);
        return it != blocks.end() && !it->second.free;
    }

    void destroy() {
        for (void* s : segments) (void)hipFree(s);
        segments.clear();
        blocks.clear();
        free_by_size.clear();
        in_use = mapped = 0;
    }
};

constexpr size_t kLargeThreshold = (size_t)1 << 20;  // src/allocators/caching_allocator.zig:20

static BlockPool* make_pool(size_t segment_bytes) {
    BlockPool* p = new BlockPool();
    p->segment_bytes = segment_bytes;
    p->min_split = kPoolAlign;
    return p;
}

// ------------------------------------------------------------------------------------------------
// small device kernels of the memory API
// ------------------------------------------------------------------------------------------------
template <class T>
__global__ void copy_kernel(T* __restrict__ dst, const T* __restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += nt) dst[i] = src[i];
}

template <typename T>
__global__ void fill_kernel(T* __restrict__ x, size_t n, T v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) x[i] = v;
}

__global__ void fill4_kernel(float4* __restrict__ x, size_t n4, float v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    float4 w = make_float4(v, v, v, v);
    for (; i < n4; i += stride) x[i] = w;
}

__global__ void sequence_kernel(float* __restrict__ x, size_t n, float initial, float step) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) x[i] = __fadd_rn(initial, __fmul_rn((float)i, step));
}

__global__ void take_kernel(const float* __restrict__ src, const uint64_t* __restrict__ idxs, size_t n,
                            float* __restrict__ dst, size_t src_len, int* __restrict__ oob) {
    size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; j < n; j += stride) {
        uint64_t i = idxs[j];
        if (i < src_len) dst[j] = src[i];
        else if (oob) *oob = 1;
    }
}

static int grid_for(zg_hip_ctx* ctx, size_t work_items, int block) {
    size_t blocks = ceil_div_sz(work_items, (size_t)block);
    size_t cap = (size_t)ctx->n_cu * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

// host generator for mem_random: splitmix64-seeded xoshiro256++; uniform = top 24 bits * 2^-24;
// normal = Box-Muller (cosine branch) in fp32
struct Rng {
    uint64_t s[4];
    explicit Rng(uint64_t seed) {
        uint64_t z = seed;
        for (int i = 0; i < 4; i++) {
            z += 0x9e3779b97f4a7c15ULL;
            uint64_t v = z;
            v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ULL;
            v = (v ^ (v >> 27)) * 0x94d049bb133111ebULL;
            s[i] = v ^ (v >> 31);
        }
    }
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t next() {
        uint64_t result = rotl(s[0] + s[3], 23) + s[0];
        uint64_t t = s[1] << 17;
        s[2] ^= s[0];
        s[3] ^= s[1];
        s[1] ^= s[2];
        s[0] ^= s[3];
        s[2] ^= t;
        s[3] = rotl(s[3], 45);
        return result;
    }
    float uniform() { return (float)(next() >> 40) * (1.0f / 16777216.0f); }
    float normal() {
        float u1 = 1.0f - uniform();
        float u2 = uniform();
        return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
    }
};

}  // namespace zg

using namespace zg;

// ------------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------------
ZG_API const char* zg_hip_last_error(void) {
    return zg::g_err;
}

ZG_API int zg_hip_device_count(int* count) {
    ZG_REQUIRE(count != nullptr, "device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return ZG_HIP_OK;
}

static int init_resources(zg_hip_ctx* ctx) {
    hipDeviceProp_t prop;
    ZG_HIP_TRY(hipGetDeviceProperties(&prop, ctx->device));
    ctx->n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    ctx->total_mem = prop.totalGlobalMem;
    // one stream, default priority, in-order: the reference's device model (src/device/cuda_device.zig:126-144)
    ZG_HIP_TRY(hipStreamCreateWithFlags(&ctx->stream, hipStreamDefault));
    ZG_HIP_TRY(hipMalloc((void**)&ctx->scalar_slot, 256));
    ZG_HIP_TRY(hipMalloc(&ctx->partials, 64 << 10));
    return noalloc_setup(ctx);
}

ZG_API int zg_hip_init(int device_id, zg_hip_ctx** out) {
    ZG_REQUIRE(out != nullptr, "init: null output");
    *out = nullptr;
    int n = 0;
    ZG_HIP_TRY(hipGetDeviceCount(&n));
    ZG_REQUIRE(device_id >= 0 && device_id < n, "init: device %d not present (%d devices)", device_id, n);
    ZG_HIP_TRY(hipSetDevice(device_id));
    zg_hip_ctx* ctx = new zg_hip_ctx();
    ctx->device = device_id;
    ctx->small_pool_bytes = (size_t)64 << 20;
    ctx->large_pool_bytes = (size_t)1 << 30;
    if (int rc = init_resources(ctx)) {
        // a context that failed part-way owns whatever it got so far
        if (ctx->scalar_slot) (void)hipFree(ctx->scalar_slot);
        if (ctx->partials) (void)hipFree(ctx->partials);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_deinit(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->small_pool) {
        ctx->small_pool->destroy();
        delete ctx->small_pool;
    }
    if (ctx->large_pool) {
        ctx->large_pool->destroy();
        delete ctx->large_pool;
    }
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->ws) (void)hipFree(ctx->ws);
    for (void* w : ctx->retired_ws) (void)hipFree(w);
    if (ctx->scalar_slot) (void)hipFree(ctx->scalar_slot);
    if (ctx->partials) (void)hipFree(ctx->partials);
    for (auto& kv : ctx->raw_allocs) (void)hipFree(kv.first);
    for (auto& kv : ctx->host_allocs) (void)hipHostFree(kv.first);
    if (ctx->copy_stream) {
        (void)hipStreamSynchronize(ctx->copy_stream);
        (void)hipEventDestroy(ctx->ev_compute);
        (void)hipEventDestroy(ctx->ev_copy);
        (void)hipStreamDestroy(ctx->copy_stream);
    }
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_sync(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "sync");
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// input staging: a copy stream beside the compute stream, ordered against it with events
// ------------------------------------------------------------------------------------------------
static int ensure_copy_stream(zg_hip_ctx* ctx) {
    if (ctx->copy_stream) return ZG_HIP_OK;
    ZG_HIP_TRY(hipStreamCreateWithFlags(&ctx->copy_stream, hipStreamNonBlocking));  // default priority
    ZG_HIP_TRY(hipEventCreateWithFlags(&ctx->ev_compute, hipEventDisableTiming));
    ZG_HIP_TRY(hipEventCreateWithFlags(&ctx->ev_copy, hipEventDisableTiming));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_staged_h2d(zg_hip_ctx* ctx, void* dst, const void* src_host, size_t bytes) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "staged_h2d");
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(dst && src_host, "staged_h2d: null pointer");
    // a pageable source would make the copy synchronous and let the caller reuse it too early
    bool pinned = false;
    for (auto& kv : ctx->host_allocs) {
        const char* lo = (const char*)kv.first;
        if ((const char*)src_host >= lo && (const char*)src_host + bytes <= lo + kv.second) pinned = true;
    }
    ZG_REQUIRE(pinned, "staged_h2d: the source must lie inside a zg_hip_host_alloc allocation");
    if (int rc = ensure_copy_stream(ctx)) return rc;
    ZG_HIP_TRY(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, ctx->copy_stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_staging_after_compute(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "staging_after_compute");
    if (int rc = ensure_copy_stream(ctx)) return rc;
    ZG_HIP_TRY(hipEventRecord(ctx->ev_compute, ctx->stream));
    ZG_HIP_TRY(hipStreamWaitEvent(ctx->copy_stream, ctx->ev_compute, 0));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_compute_after_staging(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "compute_after_staging");
    if (!ctx->copy_stream) return ZG_HIP_OK;  // nothing was ever staged
    ZG_HIP_TRY(hipEventRecord(ctx->ev_copy, ctx->copy_stream));
    ZG_HIP_TRY(hipStreamWaitEvent(ctx->stream, ctx->ev_copy, 0));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_staging_wait(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "staging_wait");
    if (!ctx->copy_stream) return ZG_HIP_OK;
    ZG_HIP_TRY(hipStreamSynchronize(ctx->copy_stream));
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// execution graphs (src/device/cuda_device.zig:558-611: open / save / run / free)
// ------------------------------------------------------------------------------------------------
struct zg_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<void*, uint64_t>> parked;  // cache blocks freed inside the capture
};

static void unpark(zg_hip_ctx* ctx, std::vector<std::pair<void*, uint64_t>>& parked) {
    for (auto& pb : parked) {
        BlockPool* pool = pb.second == 2 ? ctx->large_pool : ctx->small_pool;
        if (pool) (void)pool->release(pb.first);
    }
    parked.clear();
}

ZG_API int zg_hip_graph_open(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "graph_open");
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    ZG_HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_graph_save(zg_hip_ctx* ctx, zg_hip_graph** out) {
    ZG_CTX(ctx);
    ZG_REQUIRE(out != nullptr, "graph_save: null output");
    *out = nullptr;
    if (!ctx->capturing) {
        set_error("graph_save: no capture in progress");
        return ZG_HIP_ECAPTURE;
    }
    ctx->capturing = false;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g);
    if (e != hipSuccess || g == nullptr) {
        (void)hipGetLastError();
        unpark(ctx, ctx->capture_parked);
        set_error("graph_save: hipStreamEndCapture failed: %s", hipGetErrorString(e));
        return ZG_HIP_ERUNTIME;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(g);
        unpark(ctx, ctx->capture_parked);
        set_error("graph_save: hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return ZG_HIP_ERUNTIME;
    }
    zg_hip_graph* gr = new zg_hip_graph();
    gr->graph = g;
    gr->exec = exec;
    gr->parked.swap(ctx->capture_parked);
    ctx->live_graphs++;
    *out = gr;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_graph_run(zg_hip_ctx* ctx, zg_hip_graph* graph) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "graph_run");
    ZG_REQUIRE(graph != nullptr && graph->exec != nullptr, "graph_run: null or unsaved graph");
    ZG_HIP_TRY(hipGraphLaunch(graph->exec, ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_graph_free(zg_hip_ctx* ctx, zg_hip_graph* graph) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "graph_free");
    if (!graph) return ZG_HIP_OK;
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));  // a replay may still be running
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    unpark(ctx, graph->parked);
    ctx->live_graphs--;
    delete graph;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_total_memory(zg_hip_ctx* ctx, size_t* bytes) {
    ZG_CTX(ctx);
    ZG_REQUIRE(bytes != nullptr, "total_memory: null output");
    *bytes = ctx->total_mem;
    return ZG_HIP_OK;
}

ZG_API void* zg_hip_stream(zg_hip_ctx* ctx) {
    return ctx ? (void*)ctx->stream : nullptr;
}

ZG_API int zg_hip_event_create(zg_hip_ctx* ctx, zg_hip_event** out) {
    ZG_CTX(ctx);
    ZG_REQUIRE(out != nullptr, "event_create: null output");
    zg_hip_event* e = new zg_hip_event();
    hipError_t err = hipEventCreate(&e->ev);
    if (err != hipSuccess) {
        delete e;
        set_error("hipEventCreate failed: %s", hipGetErrorString(err));
        return ZG_HIP_ERUNTIME;
    }
    *out = e;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_event_record(zg_hip_ctx* ctx, zg_hip_event* ev) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "event_record");
    ZG_REQUIRE(ev != nullptr, "event_record: null event");
    ZG_HIP_TRY(hipEventRecord(ev->ev, ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_event_elapsed_ms(zg_hip_event* start, zg_hip_event* stop, float* ms) {
    ZG_REQUIRE(start && stop && ms, "event_elapsed_ms: null argument");
    ZG_HIP_TRY(hipEventSynchronize(stop->ev));
    ZG_HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_event_destroy(zg_hip_event* ev) {
    if (!ev) return ZG_HIP_OK;
    (void)hipEventDestroy(ev->ev);
    delete ev;
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// DataHandler primitives
// ------------------------------------------------------------------------------------------------
ZG_API int zg_hip_page_size(zg_hip_ctx* ctx, size_t* bytes) {
    ZG_CTX(ctx);
    ZG_REQUIRE(bytes != nullptr, "page_size: null output");
    *bytes = (size_t)2 << 20;  // device allocations are backed by 2 MiB fragments
    return ZG_HIP_OK;
}

static int raw_alloc(zg_hip_ctx* ctx, size_t bytes, void** out, const char* who) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "alloc");
    ZG_REQUIRE(out != nullptr, "%s: null output", who);
    *out = nullptr;
    if (bytes == 0) return ZG_HIP_OK;
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("%s: hipMalloc(%zu) failed: %s", who, bytes, hipGetErrorString(e));
        return ZG_HIP_EOOM;
    }
    ctx->n_device_allocs++;
    ctx->raw_allocs[p] = bytes;
    *out = p;
    return ZG_HIP_OK;
}

static int raw_free(zg_hip_ctx* ctx, void* ptr, const char* who) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "free");
    if (!ptr) return ZG_HIP_OK;
    auto it = ctx->raw_allocs.find(ptr);
    ZG_REQUIRE(it != ctx->raw_allocs.end(), "%s: pointer %p was not allocated by this context", who, ptr);
    // in-order stream: work that still uses the buffer must finish first
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    ZG_HIP_TRY(hipFree(ptr));
    ctx->raw_allocs.erase(it);
    return ZG_HIP_OK;
}

ZG_API int zg_hip_pool_map(zg_hip_ctx* ctx, size_t bytes, void** out) {
    return raw_alloc(ctx, bytes, out, "pool_map");
}
ZG_API int zg_hip_pool_unmap(zg_hip_ctx* ctx, void* ptr) {
    return raw_free(ctx, ptr, "pool_unmap");
}
ZG_API int zg_hip_alloc(zg_hip_ctx* ctx, size_t bytes, void** out) {
    return raw_alloc(ctx, bytes, out, "alloc");
}
ZG_API int zg_hip_free(zg_hip_ctx* ctx, void* ptr) {
    return raw_free(ctx, ptr, "free");
}

ZG_API int zg_hip_host_alloc(zg_hip_ctx* ctx, size_t bytes, void** out) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "host_alloc");
    ZG_REQUIRE(out != nullptr, "host_alloc: null output");
    *out = nullptr;
    if (bytes == 0) return ZG_HIP_OK;
    void* p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("host_alloc: hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        return ZG_HIP_EOOM;
    }
    ctx->host_allocs[p] = bytes;
    *out = p;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_host_free(zg_hip_ctx* ctx, void* ptr) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "host_free");
    if (!ptr) return ZG_HIP_OK;
    auto it = ctx->host_allocs.find(ptr);
    ZG_REQUIRE(it != ctx->host_allocs.end(), "host_free: pointer %p was not allocated by this context", ptr);
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (ctx->copy_stream) ZG_HIP_TRY(hipStreamSynchronize(ctx->copy_stream));
    ZG_HIP_TRY(hipHostFree(ptr));
    ctx->host_allocs.erase(it);
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// caching allocator
// ------------------------------------------------------------------------------------------------
ZG_API int zg_hip_cache_configure(zg_hip_ctx* ctx, size_t small_pool_bytes, size_t large_pool_bytes) {
    ZG_CTX(ctx);
    ZG_REQUIRE(ctx->small_pool == nullptr && ctx->large_pool == nullptr,
               "cache_configure: pools already in use; call clear_cache first");
    ZG_REQUIRE(small_pool_bytes >= kPoolAlign && large_pool_bytes >= kPoolAlign, "cache_configure: pool too small");
    ctx->small_pool_bytes = small_pool_bytes;
    ctx->large_pool_bytes = large_pool_bytes;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_cache_alloc(zg_hip_ctx* ctx, size_t bytes, void** out, uint64_t* block) {
    ZG_CTX(ctx);
    ZG_REQUIRE(out != nullptr && block != nullptr, "mem_cache_alloc: null output");
    *out = nullptr;
    *block = 0;
    if (bytes == 0) return ZG_HIP_OK;  // src/allocators/caching_allocator.zig:81-85
    bool large = bytes > kLargeThreshold;
    BlockPool*& pool = large ? ctx->large_pool : ctx->small_pool;
    if (!pool) pool = make_pool(large ? ctx->large_pool_bytes : ctx->small_pool_bytes);
    void* p = pool->alloc(ctx, bytes);
    if (!p) {
        if (ctx->capturing) {
            set_error("mem_cache_alloc: the pool would have to grow for %zu bytes while an execution graph is being "
                      "captured; run the same ops once eagerly first", bytes);
            return ZG_HIP_ECAPTURE;
        }
        set_error("mem_cache_alloc: out of device memory for %zu bytes", bytes);
        return ZG_HIP_EOOM;
    }
    *out = p;
    *block = large ? 2 : 1;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_cache_free(zg_hip_ctx* ctx, void* ptr, uint64_t block) {
    ZG_CTX(ctx);
    if (!ptr || block == 0) return ZG_HIP_OK;  // views and empty data: src/allocators/caching_allocator.zig:111-112
    ZG_REQUIRE(block == 1 || block == 2, "mem_cache_free: bad block handle %llu", (unsigned long long)block);
    BlockPool* pool = block == 2 ? ctx->large_pool : ctx->small_pool;
    if (ctx->capturing) {
        // the graph being recorded names this address: the block stays out of the pool until the graph is freed
        ZG_REQUIRE(pool && pool->owns_live(ptr), "mem_cache_free: %p is not a live block of this pool", ptr);
        ctx->capture_parked.push_back({ptr, block});
        return ZG_HIP_OK;
    }
    // Stream order makes reuse safe: a later op that receives this block runs after every op
    // already enqueued on the same stream.
    ZG_REQUIRE(pool && pool->release(ptr), "mem_cache_free: %p is not a live block of this pool", ptr);
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_scratch(zg_hip_ctx* ctx, size_t bytes, void** out) {
    ZG_CTX(ctx);
    ZG_REQUIRE(out != nullptr, "mem_scratch: null output");
    if (bytes > ctx->scratch_bytes) {
        ZG_NOT_CAPTURING(ctx, "mem_scratch (growing)");
        ZG_REQUIRE(ctx->live_graphs == 0, "mem_scratch: cannot grow while an execution graph may name the old buffer");
        ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
        if (ctx->scratch) ZG_HIP_TRY(hipFree(ctx->scratch));
        ctx->scratch = nullptr;
        ctx->scratch_bytes = 0;
        size_t want = (bytes + kPoolAlign - 1) / kPoolAlign * kPoolAlign;
        hipError_t e = hipMalloc(&ctx->scratch, want);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("mem_scratch: hipMalloc(%zu) failed", want);
            return ZG_HIP_EOOM;
        }
        ctx->n_device_allocs++;
        ctx->scratch_bytes = want;
    }
    *out = bytes ? ctx->scratch : nullptr;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_clear_cache(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "clear_cache");
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    for (BlockPool** pp : {&ctx->small_pool, &ctx->large_pool}) {
        if (*pp) {
            ZG_REQUIRE((*pp)->in_use == 0, "clear_cache: %zu bytes still in use", (*pp)->in_use);
            (*pp)->destroy();
            delete *pp;
            *pp = nullptr;
        }
    }
    if (ctx->scratch) {
        (void)hipFree(ctx->scratch);
        ctx->scratch = nullptr;
        ctx->scratch_bytes = 0;
    }
    return ZG_HIP_OK;
}

ZG_API int zg_hip_cache_stats(zg_hip_ctx* ctx, size_t* bytes_in_use, size_t* bytes_mapped, uint64_t* n_device_allocs) {
    ZG_CTX(ctx);
    size_t u = 0, m = 0;
    for (BlockPool* p : {ctx->small_pool, ctx->large_pool}) {
        if (p) {
            u += p->in_use;
            m += p->mapped;
        }
    }
    if (bytes_in_use) *bytes_in_use = u;
    if (bytes_mapped) *bytes_mapped = m;
    if (n_device_allocs) *n_device_allocs = ctx->n_device_allocs;
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// memory ops
// ------------------------------------------------------------------------------------------------
ZG_API int zg_hip_memcpy_h2d(zg_hip_ctx* ctx, void* dst, const void* src_host, size_t bytes) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "memcpy_h2d");
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(dst && src_host, "memcpy_h2d: null pointer");
    // The caller may reuse or free a pageable source right after the call, so wait for the copy.
    // hipMemcpyDefault: the destination may also be pinned host memory from zg_hip_host_alloc
    ZG_HIP_TRY(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyDefault, ctx->stream));
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_memcpy_d2h(zg_hip_ctx* ctx, void* dst_host, const void* src, size_t bytes) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "memcpy_d2h");
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(dst_host && src, "memcpy_d2h: null pointer");
    ZG_HIP_TRY(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDefault, ctx->stream));
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_memcpy_d2d(zg_hip_ctx* ctx, void* dst, const void* src, size_t bytes) {
    ZG_CTX(ctx);
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(dst && src, "memcpy_d2d: null pointer");
    if (ctx->capturing) {
        // recorded as a kernel node like everything else in the graph
        const bool v16 = aligned16(dst) && aligned16(src) && bytes % 16 == 0;
        const size_t units = v16 ? bytes / 16 : bytes;
        if (v16)
            hipLaunchKernelGGL(copy_kernel<uint4>, dim3(grid_for(ctx, units, kBlock)), dim3(kBlock), 0, ctx->stream,
                               (uint4*)dst, (const uint4*)src, units);
        else
            hipLaunchKernelGGL(copy_kernel<uint8_t>, dim3(grid_for(ctx, units, kBlock)), dim3(kBlock), 0, ctx->stream,
                               (uint8_t*)dst, (const uint8_t*)src, units);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    ZG_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_fill(zg_hip_ctx* ctx, float* x, size_t n, float value) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_fill: null pointer");
    if (aligned16(x) && n >= 4) {
        size_t n4 = n / 4;
        hipLaunchKernelGGL(fill4_kernel, dim3(grid_for(ctx, n4, kBlock)), dim3(kBlock), 0, ctx->stream, (float4*)x, n4,
                           value);
        ZG_LAUNCH_CHECK();
        size_t tail = n - n4 * 4;
        if (tail) {
            hipLaunchKernelGGL(fill_kernel<float>, dim3(1), dim3(64), 0, ctx->stream, x + n4 * 4, tail, value);
            ZG_LAUNCH_CHECK();
        }
    } else {
        hipLaunchKernelGGL(fill_kernel<float>, dim3(grid_for(ctx, n, kBlock)), dim3(kBlock), 0, ctx->stream, x, n,
                           value);
        ZG_LAUNCH_CHECK();
    }
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_fill_u8(zg_hip_ctx* ctx, void* x, size_t n, uint8_t value) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_fill_u8: null pointer");
    hipLaunchKernelGGL(fill_kernel<uint8_t>, dim3(grid_for(ctx, n, kBlock)), dim3(kBlock), 0, ctx->stream,
                       (uint8_t*)x, n, value);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_fill_u64(zg_hip_ctx* ctx, uint64_t* x, size_t n, uint64_t value) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_fill_u64: null pointer");
    hipLaunchKernelGGL(fill_kernel<uint64_t>, dim3(grid_for(ctx, n, kBlock)), dim3(kBlock), 0, ctx->stream, x, n,
                       value);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_sequence(zg_hip_ctx* ctx, float* x, size_t n, float initial, float step) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_sequence: null pointer");
    hipLaunchKernelGGL(sequence_kernel, dim3(grid_for(ctx, n, kBlock)), dim3(kBlock), 0, ctx->stream, x, n, initial,
                       step);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_take(zg_hip_ctx* ctx, const float* src, size_t src_len, const uint64_t* idxs, size_t n,
                           float* dst) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(src && idxs && dst, "mem_take: null pointer");
    // out-of-range indices are skipped rather than dereferenced
    hipLaunchKernelGGL(take_kernel, dim3(grid_for(ctx, n, kBlock)), dim3(kBlock), 0, ctx->stream, src, idxs, n, dst,
                       src_len, (int*)nullptr);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_random(zg_hip_ctx* ctx, float* x, size_t n, int kind, uint64_t fan, uint64_t seed) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_random: null pointer");
    ZG_REQUIRE(kind >= ZG_RAND_UNIFORM && kind <= ZG_RAND_KAIMING, "mem_random: unknown kind %d", kind);
    ZG_REQUIRE(kind != ZG_RAND_KAIMING || fan > 0, "mem_random: kaiming needs fan > 0");
    std::vector<float> host(n);
    Rng r(seed);
    if (kind == ZG_RAND_UNIFORM) {
        for (size_t i = 0; i < n; i++) host[i] = r.uniform();
    } else if (kind == ZG_RAND_NORMAL) {
        for (size_t i = 0; i < n; i++) host[i] = r.normal();
    } else {
        float sd = sqrtf(2.0f / (float)fan);
        for (size_t i = 0; i < n; i++) host[i] = r.normal() * sd;
    }
    return zg_hip_memcpy_h2d(ctx, x, host.data(), n * sizeof(float));
}
