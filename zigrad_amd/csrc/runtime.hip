// Context, memory API and the caching allocator of the gfx950 backend.
//
// Mirrors the memory half of the reference's device interface
// (src/device/device_reference.zig:29-131, src/device/host_device.zig:876-958) and supplies the
// DataHandler primitives src/allocators/caching_allocator.zig expects from a device.
#include "common.h"

#include <algorithm>
#include <cmath>

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
// Block pool: a coalescing allocator over device segments obtained with hipMalloc, with every operation in
// constant time.  Counterpart of src/allocators/block_pool.zig:103-412 (split on alloc, fuse with free
// neighbours on free, free blocks filed by size order); segments are added on demand instead of mapping
// one region of the whole device up front, so steady-state training never reaches hipMalloc once the
// working set has been seen.
//
// A block is a node of two doubly linked lists: the blocks of its segment in address order (for fusing)
// and the free blocks of its size class.  Size classes are exact up to 7 units of 256 bytes and four per
// power of two above that; a bitmap of the non-empty classes finds the first class whose blocks all fit.
// The handle the caller keeps (DeviceData.ctx in the reference, src/allocators/device_data.zig:32-40) is
// the node's address, so freeing looks nothing up; nodes live in slabs, which makes a stale or foreign
// handle detectable by a range test.
// ------------------------------------------------------------------------------------------------
struct Block {
    char* ptr;
    size_t size;
    Block *prev, *next;    // neighbours in address order within the segment
    Block *fprev, *fnext;  // neighbours in the free list of the size class (fnext also chains unused nodes)
    BlockPool* pool;
    uint8_t state;         // kNodeUnused, kFree, kLive
};
enum : uint8_t { kNodeUnused = 0, kFree = 1, kLive = 2 };

struct Segment {
    char* base;
    size_t bytes;
    Block* first;
};

struct BlockPool {
    static constexpr int kClasses = 8 + 4 * 48;
    static constexpr int kSlabNodes = 1024;
    size_t segment_bytes = 0;
    size_t min_split = kPoolAlign;
    std::vector<Segment> segments;
    std::vector<Block*> slabs;
    Block* unused_nodes = nullptr;
    Block* free_head[kClasses] = {};
    uint64_t class_bits[(kClasses + 63) / 64] = {};
    size_t in_use = 0;
    size_t mapped = 0;

    // ---- nodes ----
    Block* new_node() {
        if (!unused_nodes) {
            Block* slab = new Block[kSlabNodes]();
            slabs.push_back(slab);
            for (int i = kSlabNodes - 1; i >= 0; i--) {
                slab[i].state = kNodeUnused;
                slab[i].fnext = unused_nodes;
                unused_nodes = &slab[i];
            }
        }
        Block* b = unused_nodes;
        unused_nodes = b->fnext;
        *b = Block{};
        b->pool = this;
        return b;
    }
    void drop_node(Block* b) {
        b->state = kNodeUnused;
        b->fnext = unused_nodes;
        unused_nodes = b;
    }
    bool is_node(const void* h) const {
        for (Block* slab : slabs) {
            const char* lo = (const char*)slab;
            const char* p = (const char*)h;
            if (p >= lo && p < lo + sizeof(Block) * kSlabNodes) return (size_t)(p - lo) % sizeof(Block) == 0;
        }
        return false;
    }

    // ---- size classes ----
    // class of a block of `units` (largest class whose lower bound is <= units)
    static int class_floor(size_t units) {
        if (units < 8) return (int)units;
        const int fl = 63 - __builtin_clzll((unsigned long long)units);
        const int sl = (int)((units >> (fl - 2)) & 3);
        return 8 + (fl - 3) * 4 + sl;
    }
    // smallest class all of whose blocks hold `units`
    static int class_ceil(size_t units) {
        if (units < 8) return (int)units;
        const int fl = 63 - __builtin_clzll((unsigned long long)units);
        return class_floor(units + (((size_t)1 << (fl - 2)) - 1));
    }
    void push_free(Block* b) {
        const int c = class_floor(b->size / min_split);
        b->state = kFree;
        b->fprev = nullptr;
        b->fnext = free_head[c];
        if (free_head[c]) free_head[c]->fprev = b;
        free_head[c] = b;
        class_bits[c >> 6] |= (uint64_t)1 << (c & 63);
    }
    void pop_free(Block* b) {
        const int c = class_floor(b->size / min_split);
        if (b->fprev) b->fprev->fnext = b->fnext;
        else free_head[c] = b->fnext;
        if (b->fnext) b->fnext->fprev = b->fprev;
        if (!free_head[c]) class_bits[c >> 6] &= ~((uint64_t)1 << (c & 63));
        b->fprev = b->fnext = nullptr;
    }
    int first_class_from(int c) const {
        constexpr int kWords = (kClasses + 63) / 64;
        if (c >= kClasses) return -1;
        int w = c >> 6;
        uint64_t bits = class_bits[w] & (~(uint64_t)0 << (c & 63));
        while (true) {
            if (bits) return (w << 6) + __builtin_ctzll(bits);
            if (++w >= kWords) return -1;
            bits = class_bits[w];
        }
    }

    // ---- segments ----
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
        mapped += bytes;
        Block* b = new_node();
        b->ptr = (char*)p;
        b->size = bytes;
        segments.push_back(Segment{(char*)p, bytes, b});
        push_free(b);
        return true;
    }

    // the tail of `b` beyond `keep` bytes becomes a block of its own, filed as free
    void split_tail(Block* b, size_t keep) {
        Block* rest = new_node();
        rest->ptr = b->ptr + keep;
        rest->size = b->size - keep;
        rest->prev = b;
        rest->next = b->next;
        if (b->next) b->next->prev = rest;
        b->next = rest;
        b->size = keep;
        push_free(rest);
    }

    Block* alloc(zg_hip_ctx* ctx, size_t bytes) {
        const size_t need = (bytes + min_split - 1) / min_split * min_split;
        const size_t units = need / min_split;
        Block* b = nullptr;
        // a block of the request's own class may fit (it does when it was freed by the same caller a step ago)
        const int cf = class_floor(units);
        int tries = 0;
        for (Block* c = free_head[cf]; c && tries < 4; c = c->fnext, tries++)
            if (c->size >= need) {
                b = c;
                break;
            }
        if (!b) {
            int c = first_class_from(class_ceil(units));
            if (c < 0) {
                if (!add_segment(ctx, need)) return nullptr;
                c = first_class_from(class_ceil(units));
                if (c < 0) return nullptr;
            }
            b = free_head[c];
        }
        pop_free(b);
        if (b->size - need >= min_split) split_tail(b, need);
        b->state = kLive;
        in_use += b->size;
        return b;
    }

    // `b` must be a live block of this pool
    void release(Block* b) {
        in_use -= b->size;
        Block* nx = b->next;
        if (nx && nx->state == kFree) {
            pop_free(nx);
            b->size += nx->size;
            b->next = nx->next;
            if (nx->next) nx->next->prev = b;
            drop_node(nx);
        }
        Block* pv = b->prev;
        if (pv && pv->state == kFree) {
            pop_free(pv);
            pv->size += b->size;
            pv->next = b->next;
            if (b->next) b->next->prev = pv;
            drop_node(b);
            b = pv;
        }
        push_free(b);
    }

    bool owns_live(const void* handle, const void* ptr) const {
        if (!is_node(handle)) return false;
        const Block* b = (const Block*)handle;
        return b->pool == this && b->state == kLive && b->ptr == (const char*)ptr;
    }

    bool contains(const void* p) const {
        for (const Segment& s : segments)
            if ((const char*)p >= s.base && (const char*)p < s.base + s.bytes) return true;
        return false;
    }

    // Takes every free byte of [lo, hi) out of circulation (as live blocks appended to `held`): the part of the
    // range that callers still own is left alone.  Used when a recorded graph keeps naming addresses.
    void reserve_range(char* lo, char* hi, std::vector<Block*>& held) {
        for (Segment& s : segments) {
            if (hi <= s.base || lo >= s.base + s.bytes) continue;
            for (Block* b = s.first; b && b->ptr < hi; b = b->next) {
                if (b->ptr + b->size <= lo || b->state != kFree) continue;
                pop_free(b);
                if (b->ptr < lo) {  // keep the front free, continue with the part inside the range
                    const size_t front = (size_t)(lo - b->ptr);
                    split_tail(b, front);  // files the tail as free
                    push_free(b);
                    b = b->next;
                    pop_free(b);
                }
                if (b->ptr + b->size > hi) split_tail(b, (size_t)(hi - b->ptr));
                b->state = kLive;
                in_use += b->size;
                held.push_back(b);
            }
        }
    }

    void destroy() {
        for (Segment& s : segments) (void)hipFree(s.base);
        segments.clear();
        for (Block* slab : slabs) delete[] slab;
        slabs.clear();
        unused_nodes = nullptr;
        for (auto& h : free_head) h = nullptr;
        for (auto& w : class_bits) w = 0;
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

// A fill of x[0 .. n) with v and a copy of n_copy floats to x + off in one pass: a zero-filled gradient whose leading rows
// are then overwritten (MaskLayer.backward, examples/gcn/src/model.zig:343-348).
__global__ void fill_and_copy_kernel(float* __restrict__ x, size_t n, float v, size_t off, const float* __restrict__ src,
                                     size_t n_copy) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += nt) x[i] = (i >= off && i - off < n_copy) ? src[i - off] : v;
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

// capped = 16 workgroups per compute unit, threads looping over the rest: the better choice where a thread moves four
// bytes per trip (sequence on 134 M elements: 99 us capped, 116 us with a thread per element); kernels whose threads move
// 8 or 16 bytes per trip take a workgroup per chunk at any size (fill of 134 M 64-bit words: 208 -> 163 us)
static int grid_for(zg_hip_ctx* ctx, size_t work_items, int block, bool capped = true) {
    size_t blocks = ceil_div_sz(work_items, (size_t)block);
    size_t cap = capped ? (size_t)ctx->n_cu * 16 : 0x7fffffffull;
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

constexpr size_t kSmallD2H = 4096;  // device-to-host copies up to this size go through the context's pinned slot
static int init_resources(zg_hip_ctx* ctx) {
    hipDeviceProp_t prop;
    ZG_HIP_TRY(hipGetDeviceProperties(&prop, ctx->device));
    ctx->n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    ctx->total_mem = prop.totalGlobalMem;
    // one stream, default priority, in-order: the reference's device model (src/device/cuda_device.zig:126-144)
    ZG_HIP_TRY(hipStreamCreateWithFlags(&ctx->stream, hipStreamDefault));
    ZG_HIP_TRY(hipMalloc((void**)&ctx->scalar_slot, 256));
    ZG_HIP_TRY(hipMalloc(&ctx->partials, 64 << 10));
    ZG_HIP_TRY(hipHostMalloc(&ctx->d2h_slot, kSmallD2H, hipHostMallocDefault));
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
        if (ctx->d2h_slot) (void)hipHostFree(ctx->d2h_slot);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_deinit(zg_hip_ctx* ctx) {
    ZG_REQUIRE(ctx != nullptr, "null context");
    // held work is launched first; if that fails the error is returned, but the context is torn down all the same
    int held_rc = ctx->late_error;
    if (anything_waits(ctx))
        if (int rc = flush_pending(ctx)) held_rc = held_rc ? held_rc : rc;
    (void)hipStreamSynchronize(ctx->stream);
    gemm_plans_destroy(ctx);
    plan_cache_destroy(ctx);  // its device memory is in raw_allocs; this frees the host side
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
    if (ctx->d2h_slot) (void)hipHostFree(ctx->d2h_slot);
    for (auto& kv : ctx->raw_allocs) (void)hipFree(kv.first);
    for (auto& kv : ctx->host_allocs) (void)hipHostFree(kv.first);
    for (auto& b : ctx->host_free_blocks) {
        (void)hipEventDestroy(b.done);
        (void)hipHostFree(b.ptr);
    }
    if (ctx->copy_stream) {
        (void)hipStreamSynchronize(ctx->copy_stream);
        (void)hipEventDestroy(ctx->ev_compute);
        (void)hipEventDestroy(ctx->ev_copy);
        (void)hipStreamDestroy(ctx->copy_stream);
    }
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return held_rc;
}

// Launches whatever waits in the context, without waiting for the stream (no counterpart in the reference).
ZG_API int zg_hip_flush(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    return ZG_HIP_OK;
}

// Whether calls may leave work waiting in the context for the calls that follow (default) or launch their own work
// before they return.
ZG_API int zg_hip_set_holding(zg_hip_ctx* ctx, int enable) {
    ZG_CTX(ctx);  // what waits now goes out either way
    ctx->hold_work = enable != 0;
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
    std::vector<Block*> held;  // the cache memory the recorded ops name, kept out of the pools while the graph lives
    std::vector<PlanUse> plan_uses;  // cached segment plans the recorded kernels read, and the index arrays they stand for
};

static void release_held(std::vector<Block*>& held) {
    for (Block* b : held) b->pool->release(b);
    held.clear();
}

// The address ranges of every cache block handed out or returned while recording, merged; whatever part of
// them is free when the recording ends belongs to the graph from then on.
static void hold_touched_ranges(zg_hip_ctx* ctx, std::vector<Block*>& held) {
    auto& r = ctx->capture_touched;
    std::sort(r.begin(), r.end());
    size_t i = 0;
    while (i < r.size()) {
        char* lo = r[i].first;
        char* hi = lo + r[i].second;
        size_t j = i + 1;
        while (j < r.size() && r[j].first <= hi) {
            if (r[j].first + r[j].second > hi) hi = r[j].first + r[j].second;
            j++;
        }
        for (BlockPool* pool : {ctx->small_pool, ctx->large_pool})
            if (pool) pool->reserve_range(lo, hi, held);
        i = j;
    }
    r.clear();
}

ZG_API int zg_hip_graph_open(zg_hip_ctx* ctx) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "graph_open");
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    ZG_HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capture_touched.clear();
    ctx->plan_uses.clear();
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
        ctx->capture_touched.clear();
        ctx->plan_uses.clear();
        set_error("graph_save: hipStreamEndCapture failed: %s", hipGetErrorString(e));
        return ZG_HIP_ERUNTIME;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(g);
        ctx->capture_touched.clear();
        ctx->plan_uses.clear();
        set_error("graph_save: hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return ZG_HIP_ERUNTIME;
    }
    zg_hip_graph* gr = new zg_hip_graph();
    gr->graph = g;
    gr->exec = exec;
    hold_touched_ranges(ctx, gr->held);
    gr->plan_uses.swap(ctx->plan_uses);
    plan_uses_retain(gr->plan_uses, +1);
    ctx->live_graphs++;
    *out = gr;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_graph_run(zg_hip_ctx* ctx, zg_hip_graph* graph) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "graph_run");
    ZG_REQUIRE(graph != nullptr && graph->exec != nullptr, "graph_run: null or unsaved graph");
    if (!graph->plan_uses.empty())
        if (int rc = plan_uses_validate(ctx, graph->plan_uses)) return rc;
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
    release_held(graph->held);
    plan_uses_retain(graph->plan_uses, -1);
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
    if (!ctx) return nullptr;
    // work the caller queues on the stream itself must find everything already there; if what waits cannot be launched
    // the stream is not handed out (zg_hip_last_error says why)
    if (flush_pending(ctx) != ZG_HIP_OK) return nullptr;
    return (void*)ctx->stream;
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

// Pinned host memory.  Size classes are powers of two from 256 bytes; blocks of up to 16 MiB that are given back are
// kept (up to 256 MiB in all) and handed out again to requests of the same class.
constexpr size_t kHostBlockKeepMax = (size_t)16 << 20;
constexpr size_t kHostCacheMax = (size_t)256 << 20;
static size_t host_size_class(size_t bytes) {
    size_t cap = 256;
    while (cap < bytes) cap <<= 1;
    return cap;
}

ZG_API int zg_hip_host_alloc(zg_hip_ctx* ctx, size_t bytes, void** out) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "host_alloc");
    ZG_REQUIRE(out != nullptr, "host_alloc: null output");
    *out = nullptr;
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(bytes <= ((size_t)1 << 62), "host_alloc: %zu bytes", bytes);
    const size_t cap = host_size_class(bytes);
    void* p = nullptr;
    for (size_t i = 0; i < ctx->host_free_blocks.size() && !p; i++) {
        if (ctx->host_free_blocks[i].cap != cap) continue;
        zg_hip_ctx::HostBlock b = ctx->host_free_blocks[i];
        // kernels queued before the block was given back may still read it: wait for that point of the stream
        ZG_HIP_TRY(hipEventSynchronize(b.done));
        (void)hipEventDestroy(b.done);
        ctx->host_free_blocks.erase(ctx->host_free_blocks.begin() + (long)i);
        ctx->host_cached_bytes -= cap;
        p = b.ptr;
    }
    if (!p) {
        hipError_t e = hipHostMalloc(&p, cap, hipHostMallocDefault);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("host_alloc: hipHostMalloc(%zu) failed: %s", cap, hipGetErrorString(e));
            return ZG_HIP_EOOM;
        }
    }
    ctx->host_allocs[p] = bytes;
    ctx->host_caps[p] = cap;
    *out = p;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_host_free(zg_hip_ctx* ctx, void* ptr) {
    ZG_CTX(ctx);  // whatever waits in the context may read the block: it is launched first
    ZG_NOT_CAPTURING(ctx, "host_free");
    if (!ptr) return ZG_HIP_OK;
    auto it = ctx->host_allocs.find(ptr);
    ZG_REQUIRE(it != ctx->host_allocs.end(), "host_free: pointer %p was not allocated by this context", ptr);
    const size_t cap = ctx->host_caps[ptr];
    if (ctx->copy_stream) ZG_HIP_TRY(hipStreamSynchronize(ctx->copy_stream));
    if (cap <= kHostBlockKeepMax && ctx->host_cached_bytes + cap <= kHostCacheMax) {
        hipEvent_t done = nullptr;
        ZG_HIP_TRY(hipEventCreateWithFlags(&done, hipEventDisableTiming));
        hipError_t e = hipEventRecord(done, ctx->stream);
        if (e != hipSuccess) {
            (void)hipEventDestroy(done);
            ZG_HIP_TRY(e);
        }
        ctx->host_free_blocks.push_back(zg_hip_ctx::HostBlock{ptr, cap, done});
        ctx->host_cached_bytes += cap;
    } else {
        ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
        ZG_HIP_TRY(hipHostFree(ptr));
    }
    ctx->host_allocs.erase(it);
    ctx->host_caps.erase(ptr);
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
    ZG_ENTER(ctx, kWaitAll);
    // waiting fills stay (a block that is handed out is free, so no waiting fill names it), and so do waiting
    // elementwise ops: a new block holds no operand of theirs, and a caller allocates each op's output just before it
    if (ctx->scatter_wait.active)
        if (int rc = flush_scatter(ctx)) return rc;
    if (ctx->graddeg_wait.active)
        if (int rc = flush_graddeg(ctx)) return rc;
    // what a waiting product waits for comes right after it, not after an allocation; a bias gradient that waits
    // alone stays (the input gradient its layer's products write is allocated next, and a new block holds no operand)
    if (ctx->deferred.active)
        if (int rc = flush_deferred_gemm(ctx)) return rc;
    if (ctx->steps.count)
        if (int rc = flush_steps(ctx)) return rc;
    ZG_REQUIRE(out != nullptr && block != nullptr, "mem_cache_alloc: null output");
    *out = nullptr;
    *block = 0;
    if (bytes == 0) return ZG_HIP_OK;  // src/allocators/caching_allocator.zig:81-85
    bool large = bytes > kLargeThreshold;
    BlockPool*& pool = large ? ctx->large_pool : ctx->small_pool;
    if (!pool) pool = make_pool(large ? ctx->large_pool_bytes : ctx->small_pool_bytes);
    Block* b = pool->alloc(ctx, bytes);
    if (!b) {
        if (ctx->capturing) {
            set_error("mem_cache_alloc: the pool would have to grow for %zu bytes while an execution graph is being "
                      "captured; run the same ops once eagerly first", bytes);
            return ZG_HIP_ECAPTURE;
        }
        set_error("mem_cache_alloc: out of device memory for %zu bytes", bytes);
        return ZG_HIP_EOOM;
    }
    if (ctx->capturing) ctx->capture_touched.push_back({b->ptr, b->size});
    *out = b->ptr;
    *block = (uint64_t)(uintptr_t)b;
    return ZG_HIP_OK;
}

static void release_block(zg_hip_ctx* ctx, Block* b) {
    // While recording, the block goes back to the pool like any other, so a later allocation of the same recording
    // may reuse it (the graph keeps the stream's order); its range is noted, and whatever part of the noted ranges is
    // free when the recording ends stays with the graph.  Outside a recording, stream order makes reuse safe: a
    // later op that receives this block runs after every op already enqueued on the same stream.
    if (ctx->capturing) ctx->capture_touched.push_back({b->ptr, b->size});
    b->pool->release(b);
}

namespace zg {
void run_deferred_frees(zg_hip_ctx* ctx) {
    const int n = ctx->n_deferred_frees;
    ctx->n_deferred_frees = 0;
    for (int i = 0; i < n; i++) release_block(ctx, (Block*)(uintptr_t)ctx->deferred_frees[i].block);
}
}  // namespace zg

ZG_API int zg_hip_mem_cache_free(zg_hip_ctx* ctx, void* ptr, uint64_t block) {
    ZG_ENTER(ctx, kWaitAll);
    // Waiting elementwise ops stay: the pool keeps the block's memory, so they may still read and write it when they
    // are launched, and whoever receives the block next either joins them (in call order, element by element) or sends
    // them out first.
    if (ctx->scatter_wait.active)
        if (int rc = flush_scatter(ctx)) return rc;
    if (ctx->graddeg_wait.active) {
        // a waiting degree gradient whose whole output lies in the block that is given back has no reader left and is
        // dropped (the reference's layer frees it unread); any other free sends it out first
        const zg_waiting_graddeg& w = ctx->graddeg_wait;
        const Block* gb = (const Block*)(uintptr_t)block;
        bool dead = false;
        if (ptr && block)
            for (BlockPool* p : {ctx->small_pool, ctx->large_pool})
                if (p && p->owns_live(const_cast<Block*>(gb), ptr))
                    dead = gb->ptr <= (const char*)w.grad_deg && (const char*)(w.grad_deg + w.n_nodes) <= gb->ptr + gb->size;
        if (dead) ctx->graddeg_wait.active = false;
        else if (int rc = flush_graddeg(ctx)) return rc;
    }
    if (ctx->steps.count)
        if (int rc = flush_steps(ctx)) return rc;
    if (!ptr || block == 0) {  // views and empty data: src/allocators/caching_allocator.zig:111-112
        if (int rc = flush_fills(ctx)) return rc;
        if (gemm_group_waiting(ctx)) return flush_deferred_gemm(ctx);
        return ZG_HIP_OK;
    }
    Block* b = (Block*)(uintptr_t)block;
    BlockPool* pool = nullptr;
    for (BlockPool* p : {ctx->small_pool, ctx->large_pool})
        if (p && p->owns_live(b, ptr)) pool = p;
    if (pool == nullptr) (void)flush_fills(ctx);
    ZG_REQUIRE(pool != nullptr, "mem_cache_free: %p with handle %llx is not a live block of this context's pools", ptr,
               (unsigned long long)block);
    if (ctx->n_pending_fills) {
        // A fill must not land on the block's next owner.  One that lies wholly inside the block that is given back
        // has no reader left (the block's contents are nobody's once it is free) and is dropped: the upstream gradient
        // of a loss is filled, never read by the fused loss backward, and freed.  One that straddles the block's end
        // sends all waiting fills out instead; the others keep waiting.
        const char *lo = b->ptr, *hi = b->ptr + b->size;
        bool straddles = false;
        for (int i = 0; i < ctx->n_pending_fills; i++) {
            const char* x0 = (const char*)ctx->pending_fills[i].x;
            const char* x1 = x0 + ctx->pending_fills[i].n * sizeof(float);
            straddles = straddles || (x0 < hi && lo < x1 && !(lo <= x0 && x1 <= hi));
        }
        if (straddles) {
            if (int rc = flush_fills(ctx)) return rc;
        } else {
            int kept = 0;
            for (int i = 0; i < ctx->n_pending_fills; i++) {
                const char* x0 = (const char*)ctx->pending_fills[i].x;
                if (!(lo <= x0 && x0 < hi)) ctx->pending_fills[kept++] = ctx->pending_fills[i];
            }
            ctx->n_pending_fills = kept;
        }
    }
    if (gemm_group_waiting(ctx)) {
        // An input-gradient product that waits for its mask outlives the frees of the backward pass it belongs to
        // (the layer's output, the output gradient), and so do the bias gradient and the weight-gradient product
        // that wait with it.  A block none of their operands lies in goes back at once; one that holds an operand
        // goes back when they have been launched.
        const bool keep_waiting = !ctx->deferred.active || ctx->deferred.kind == 2;
        for (int i = 0; i < ctx->n_deferred_frees; i++)
            ZG_REQUIRE(ctx->deferred_frees[i].block != block, "mem_cache_free: %p was already given back", ptr);
        if (keep_waiting) {
            if (!gemm_group_touches(ctx, b->ptr, b->ptr + b->size)) {
                release_block(ctx, b);
                return ZG_HIP_OK;
            }
            if (ctx->n_deferred_frees < 4) {
                ctx->deferred_frees[ctx->n_deferred_frees].ptr = ptr;
                ctx->deferred_frees[ctx->n_deferred_frees].block = block;
                ctx->n_deferred_frees++;
                return ZG_HIP_OK;
            }
        }
        if (int rc = flush_deferred_gemm(ctx)) return rc;
    }
    release_block(ctx, b);
    return ZG_HIP_OK;
}

// Whether `ptr` lies in memory this context handed out as device memory (cache pools, raw allocations, scratch):
// what a binding needs to tell a device slice from a host scalar (the reference's callers pass both through the
// same parameter: src/ndarray.zig:251, src/nn/optim.zig:117 against src/ndtensor.zig:1146-1150).
ZG_API int zg_hip_is_device_ptr(zg_hip_ctx* ctx, const void* ptr, int* yes) {
    ZG_ENTER(ctx, kWaitAll);  // a lookup in host tables: a binding asks before every op with a one-float operand
    ZG_REQUIRE(yes != nullptr, "is_device_ptr: null output");
    *yes = 0;
    if (!ptr) return ZG_HIP_OK;
    for (BlockPool* p : {ctx->small_pool, ctx->large_pool})
        if (p && p->contains(ptr)) *yes = 1;
    if (!*yes && ctx->scratch && (const char*)ptr >= (const char*)ctx->scratch &&
        (const char*)ptr < (const char*)ctx->scratch + ctx->scratch_bytes)
        *yes = 1;
    if (!*yes && !ctx->raw_allocs.empty()) {
        auto it = ctx->raw_allocs.upper_bound(const_cast<void*>(ptr));
        if (it != ctx->raw_allocs.begin()) {
            --it;
            if ((const char*)ptr < (const char*)it->first + it->second) *yes = 1;
        }
    }
    return ZG_HIP_OK;
}

ZG_API int zg_hip_mem_scratch(zg_hip_ctx* ctx, size_t bytes, void** out) {
    ZG_CTX(ctx);
    ZG_REQUIRE(out != nullptr, "mem_scratch: null output");
    if (bytes > ctx->scratch_bytes) {
        ZG_NOT_CAPTURING(ctx, "mem_scratch (growing)");
        ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
        if (ctx->scratch) {
            // an instantiated graph may have recorded the old address: keep it alive until the context goes
            if (ctx->live_graphs > 0) ctx->retired_ws.push_back(ctx->scratch);
            else ZG_HIP_TRY(hipFree(ctx->scratch));
        }
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
    for (auto& b : ctx->host_free_blocks) {  // the stream has been waited for: nothing reads them any more
        (void)hipEventDestroy(b.done);
        (void)hipHostFree(b.ptr);
    }
    ctx->host_free_blocks.clear();
    ctx->host_cached_bytes = 0;
    return ZG_HIP_OK;
}

namespace zg {
std::atomic<unsigned long long> launches_issued{0};
}

ZG_API int zg_hip_launch_count(zg_hip_ctx* ctx, uint64_t* launches) {
    ZG_REQUIRE(ctx != nullptr && launches != nullptr, "launch_count: null argument");
    *launches = launches_issued.load(std::memory_order_relaxed);  // nothing is sent out: what waits in the context has not been launched and is not counted
    return ZG_HIP_OK;
}

ZG_API int zg_hip_cache_stats(zg_hip_ctx* ctx, size_t* bytes_in_use, size_t* bytes_mapped, uint64_t* n_device_allocs) {
    ZG_ENTER(ctx, kWaitAll);  // host counters only: what waits keeps waiting
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

namespace zg {
// A scalar read (loss.get(0), src/ndtensor.zig:524-528; an op's status word): a copy kernel into the context's pinned
// slot, the wait for the stream, and a host copy.  The driver's own path for a few bytes into pageable memory costs
// 25 us more per call (the batch-64 train step from C: 99 -> 75-85 us).  At most kSmallD2H bytes.
int small_d2h(zg_hip_ctx* ctx, void* dst_host, const void* src, size_t bytes) {
    hipLaunchKernelGGL(copy_kernel<uint8_t>, dim3(1), dim3(kBlock), 0, ctx->stream, (uint8_t*)ctx->d2h_slot,
                       (const uint8_t*)src, bytes);
    ZG_LAUNCH_CHECK();
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    memcpy(dst_host, ctx->d2h_slot, bytes);
    return ZG_HIP_OK;
}
}  // namespace zg

ZG_API int zg_hip_memcpy_d2h(zg_hip_ctx* ctx, void* dst_host, const void* src, size_t bytes) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "memcpy_d2h");
    if (bytes == 0) return ZG_HIP_OK;
    ZG_REQUIRE(dst_host && src, "memcpy_d2h: null pointer");
    if (bytes <= kSmallD2H) return small_d2h(ctx, dst_host, src, bytes);
    ZG_HIP_TRY(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDefault, ctx->stream));
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return ZG_HIP_OK;
}

ZG_API int zg_hip_memcpy_d2d(zg_hip_ctx* ctx, void* dst, const void* src, size_t bytes) {
    ZG_ENTER(ctx, kWaitAll);
    if (bytes == 0 || !dst || !src) {
        if (int rc = flush_pending(ctx)) return rc;
        if (bytes == 0) return ZG_HIP_OK;
        ZG_REQUIRE(dst && src, "memcpy_d2d: null pointer");
    }
    // fills dropped below are owed back if the copy is then refused
    zg_pending_fill dropped[kMaxPendingFills];
    int n_dropped = 0;
    {
        // waiting fills that meet neither range stay; one that lies inside a destination the copy overwrites without
        // reading it has no reader left
        const char *s0 = (const char*)src, *d0 = (const char*)dst;
        if (s0 + bytes <= d0 || d0 + bytes <= s0) n_dropped = take_fills_inside(ctx, dst, bytes, dropped);
        // a waiting float fill that covers the destination and more (a gradient zeroed, then its leading rows
        // overwritten) and is clear of the source leaves together with the copy, in one launch
        int host_fill = -1;
        if (bytes % sizeof(float) == 0 && ((uintptr_t)dst | (uintptr_t)src) % sizeof(float) == 0)
            for (int i = 0; i < ctx->n_pending_fills && host_fill < 0; i++) {
                const char* x0 = (const char*)ctx->pending_fills[i].x;
                const char* x1 = x0 + ctx->pending_fills[i].n * sizeof(float);
                if (x0 <= d0 && d0 + bytes <= x1 && (s0 + bytes <= x0 || x1 <= s0) &&
                    ctx->pending_fills[i].n <= ((size_t)1 << 20))  // a long fill keeps its own kernel's wide stores
                    host_fill = i;
            }
        zg_pending_fill f{};
        if (host_fill >= 0) {
            f = ctx->pending_fills[host_fill];
            for (int j = host_fill + 1; j < ctx->n_pending_fills; j++) ctx->pending_fills[j - 1] = ctx->pending_fills[j];
            ctx->n_pending_fills--;
        }
        const void* ptrs[2] = {src, dst};
        const size_t lens[2] = {bytes, bytes};
        int rc = flush_pending_but_fills(ctx, ptrs, lens, 2);
        if (host_fill >= 0) {
            if (rc) {  // refused: the fills are still owed
                (void)zg_hip_mem_fill(ctx, f.x, f.n, f.value);
                requeue_fills(ctx, dropped, n_dropped);
                return rc;
            }
            hipLaunchKernelGGL(fill_and_copy_kernel, dim3(grid_for(ctx, f.n, kBlock)), dim3(kBlock), 0, ctx->stream, f.x, f.n,
                               f.value, (size_t)((const float*)dst - f.x), (const float*)src, bytes / sizeof(float));
            ZG_LAUNCH_CHECK();
            return ZG_HIP_OK;
        }
        if (rc) {
            requeue_fills(ctx, dropped, n_dropped);
            return rc;
        }
    }
    if (ctx->capturing) {
        // recorded as a kernel node like everything else in the graph
        const bool v16 = aligned16(dst) && aligned16(src) && bytes % 16 == 0;
        const size_t units = v16 ? bytes / 16 : bytes;
        if (v16)
            hipLaunchKernelGGL(copy_kernel<uint4>, dim3(grid_for(ctx, units, kBlock, false)), dim3(kBlock), 0, ctx->stream,
                               (uint4*)dst, (const uint4*)src, units);
        else
            hipLaunchKernelGGL(copy_kernel<uint8_t>, dim3(grid_for(ctx, units, kBlock)), dim3(kBlock), 0, ctx->stream,
                               (uint8_t*)dst, (const uint8_t*)src, units);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    // From 128 MiB on, between two device buffers on 16-byte boundaries, the library's own kernel: the driver's copy runs
    // at 64 % of 8 TB/s beyond the Infinity Cache (1 GiB: 422 us), a thread per 16 bytes at 74 %.
    if (bytes >= ((size_t)128 << 20) && aligned16(dst) && aligned16(src) && bytes % 16 == 0) {
        hipPointerAttribute_t pa_d, pa_s;
        const bool dev = hipPointerGetAttributes(&pa_d, dst) == hipSuccess && pa_d.type == hipMemoryTypeDevice &&
                         hipPointerGetAttributes(&pa_s, src) == hipSuccess && pa_s.type == hipMemoryTypeDevice;
        if (!dev) (void)hipGetLastError();  // a pointer the driver does not know leaves an error behind
        if (dev) {
            hipLaunchKernelGGL(copy_kernel<uint4>, dim3(grid_for(ctx, bytes / 16, kBlock, false)), dim3(kBlock), 0, ctx->stream,
                               (uint4*)dst, (const uint4*)src, bytes / 16);
            ZG_LAUNCH_CHECK();
            return ZG_HIP_OK;
        }
    }
    launches_issued.fetch_add(1, std::memory_order_relaxed);  // the driver's copy kernel
    if (hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, ctx->stream)) {
        requeue_fills(ctx, dropped, n_dropped);
        ZG_HIP_TRY(e);
    }
    return ZG_HIP_OK;
}

// Up to kMaxPendingFills float fills in one launch: workgroup b fills one slice of kFillSlice floats of the fill
// that owns it (wg_first is the running count of slices).  Slices of a 16-byte aligned array are written in
// 16-byte pieces, four per thread.
constexpr size_t kFillSlice = 4096;
struct MultiFillArgs {
    float* x[kMaxPendingFills];
    size_t n[kMaxPendingFills];
    float value[kMaxPendingFills];
    unsigned wg_first[kMaxPendingFills + 1];
    int count;
};
__global__ __launch_bounds__(kBlock) void multi_fill_kernel(MultiFillArgs a) {
    int e = 0;
    while (e + 1 < a.count && blockIdx.x >= a.wg_first[e + 1]) e++;
    const size_t s0 = (size_t)(blockIdx.x - a.wg_first[e]) * kFillSlice;
    float* x = a.x[e] + s0;
    const size_t n = a.n[e] - s0 < kFillSlice ? a.n[e] - s0 : kFillSlice;
    const float v = a.value[e];
    size_t done = 0;
    if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
        const size_t n4 = n >> 2;
        const float4 v4 = make_float4(v, v, v, v);
        for (size_t i = threadIdx.x; i < n4; i += kBlock) reinterpret_cast<float4*>(x)[i] = v4;
        done = n4 << 2;
    }
    for (size_t i = done + threadIdx.x; i < n; i += kBlock) x[i] = v;
}

namespace zg {
int flush_fills(zg_hip_ctx* ctx) {
    const int count = ctx->n_pending_fills;
    if (count == 0) return ZG_HIP_OK;
    ctx->n_pending_fills = 0;  // whatever happens below, the same fills are not sent twice
    MultiFillArgs a;
    size_t wgs = 0;
    for (int i = 0; i < count; i++) {
        a.x[i] = ctx->pending_fills[i].x;
        a.n[i] = ctx->pending_fills[i].n;
        a.value[i] = ctx->pending_fills[i].value;
        a.wg_first[i] = (unsigned)wgs;
        wgs += ceil_div_sz(a.n[i], kFillSlice);
    }
    a.wg_first[count] = (unsigned)wgs;
    a.count = count;
    hipLaunchKernelGGL(multi_fill_kernel, dim3((unsigned)wgs), dim3(kBlock), 0, ctx->stream, a);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}
int flush_kinds(zg_hip_ctx* ctx, unsigned kinds) {
    // Work of different kinds that waits at the same time touches disjoint memory (each kind's calls send out whatever
    // meets their operands before they queue), so the kinds may leave in any order; this one is fixed.
    if ((kinds & kWaitMaps) && ctx->maps.count)
        if (int rc = flush_maps(ctx)) return rc;
    if ((kinds & kWaitScatter) && ctx->scatter_wait.active)
        if (int rc = flush_scatter(ctx)) return rc;
    if ((kinds & kWaitGradDeg) && ctx->graddeg_wait.active)
        if (int rc = flush_graddeg(ctx)) return rc;
    if ((kinds & kWaitProducts) && gemm_group_waiting(ctx))
        if (int rc = flush_deferred_gemm(ctx)) return rc;
    if ((kinds & kWaitFills) && ctx->n_pending_fills)
        if (int rc = flush_fills(ctx)) return rc;
    if ((kinds & kWaitSteps) && ctx->steps.count)
        if (int rc = flush_steps(ctx)) return rc;
    return ZG_HIP_OK;
}

bool kind_touches(const zg_hip_ctx* ctx, unsigned kind, const ByteSpan* spans, int count) {
    for (int j = 0; j < count; j++) {
        const char* lo = (const char*)spans[j].p;
        if (!lo || spans[j].bytes == 0) continue;
        const char* hi = lo + spans[j].bytes;
        bool hit = false;
        switch (kind) {
            case kWaitFills:
                for (int i = 0; i < ctx->n_pending_fills && !hit; i++) {
                    const char* x0 = (const char*)ctx->pending_fills[i].x;
                    hit = x0 < hi && lo < x0 + ctx->pending_fills[i].n * sizeof(float);
                }
                break;
            case kWaitProducts: hit = gemm_group_waiting(ctx) && gemm_group_touches(ctx, lo, hi); break;
            case kWaitSteps: hit = steps_touch(ctx, lo, hi); break;
            case kWaitScatter: hit = scatter_wait_touches(ctx, lo, hi); break;
            case kWaitGradDeg: hit = graddeg_wait_touches(ctx, lo, hi); break;
            case kWaitMaps: hit = maps_touch(ctx, lo, hi); break;
            default: break;
        }
        if (hit) return true;
    }
    return false;
}

int flush_touching(zg_hip_ctx* ctx, unsigned kinds, const ByteSpan* spans, int count) {
    unsigned hit = 0;
    for (unsigned kind = 1; kind <= kWaitMaps; kind <<= 1)
        if ((kinds & kind) && (waiting_kinds(ctx) & kind) && kind_touches(ctx, kind, spans, count)) hit |= kind;
    return hit ? flush_kinds(ctx, hit) : ZG_HIP_OK;
}

bool fills_touch(zg_hip_ctx* ctx, const void* const* ptrs, const size_t* bytes, int count) {
    ByteSpan spans[8];
    const int n = count < 8 ? count : 8;
    for (int j = 0; j < n; j++) spans[j] = ByteSpan{ptrs[j], bytes[j]};
    return kind_touches(ctx, kWaitFills, spans, n);
}
bool take_fill_exact(zg_hip_ctx* ctx, const float* x, size_t n, float* value) {
    for (int i = 0; i < ctx->n_pending_fills; i++) {
        const zg_pending_fill& p = ctx->pending_fills[i];
        if (p.x == x && p.n == n) {
            *value = p.value;
            for (int j = i + 1; j < ctx->n_pending_fills; j++) ctx->pending_fills[j - 1] = ctx->pending_fills[j];
            ctx->n_pending_fills--;
            return true;
        }
    }
    return false;
}
int take_fills_inside(zg_hip_ctx* ctx, const void* lo_, size_t bytes, zg_pending_fill* out) {
    const char *lo = (const char*)lo_, *hi = lo + bytes;
    int kept = 0, taken = 0;
    for (int i = 0; i < ctx->n_pending_fills; i++) {
        const char* x0 = (const char*)ctx->pending_fills[i].x;
        const char* x1 = x0 + ctx->pending_fills[i].n * sizeof(float);
        if (!(lo <= x0 && x1 <= hi)) ctx->pending_fills[kept++] = ctx->pending_fills[i];
        else if (out) out[taken++] = ctx->pending_fills[i];
    }
    ctx->n_pending_fills = kept;
    return taken;
}
void drop_fills_inside(zg_hip_ctx* ctx, const void* lo, size_t bytes) {
    (void)take_fills_inside(ctx, lo, bytes, nullptr);
}
void requeue_fills(zg_hip_ctx* ctx, const zg_pending_fill* fills, int count) {
    for (int i = 0; i < count; i++) (void)zg_hip_mem_fill(ctx, fills[i].x, fills[i].n, fills[i].value);
}

int flush_pending_but_fills(zg_hip_ctx* ctx, const void* const* ptrs, const size_t* bytes, int count) {
    if (int rc = flush_kinds(ctx, kWaitAll & ~kWaitFills)) return rc;
    ByteSpan spans[8];
    const int n = count < 8 ? count : 8;
    for (int j = 0; j < n; j++) spans[j] = ByteSpan{ptrs[j], bytes[j]};
    return flush_touching(ctx, kWaitFills, spans, n);
}

bool absorb_zero_fill(zg_hip_ctx* ctx, const float* x, size_t n) {
    for (int i = 0; i < ctx->n_pending_fills; i++) {
        const zg_pending_fill& p = ctx->pending_fills[i];
        uint32_t bits;
        memcpy(&bits, &p.value, sizeof(bits));
        if (p.x == x && p.n == n && bits == 0u) {  // +0.0 only: x + (-0.0) and x differ for x = +0.0
            for (int j = i + 1; j < ctx->n_pending_fills; j++) ctx->pending_fills[j - 1] = ctx->pending_fills[j];
            ctx->n_pending_fills--;
            return true;
        }
    }
    return false;
}
}  // namespace zg

ZG_API int zg_hip_mem_fill(zg_hip_ctx* ctx, float* x, size_t n, float value) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    // a waiting product goes first: the fill may be of one of its operands; a bias gradient that waits alone stays
    // unless the fill meets what it reads or writes (the zero fill of the layer's input gradient comes next)
    if (ctx->deferred.active) {
        if (int rc = flush_kinds(ctx, kWaitProducts)) return rc;
    } else if (x && n) {
        const ByteSpan span{x, n * sizeof(float)};
        if (int rc = flush_touching(ctx, kWaitProducts, &span, 1)) return rc;
    }
    if (ctx->steps.count) {
        // zero_grad() after step() (examples/mnist/src/model.zig:57-62): a zero fill of exactly the gradient of a waiting
        // step is taken over by the step, whose kernel stores the zeros once it has read the gradient; any other fill
        // sends the steps out first (it may be of something they read), and zeros taken over so far leave with it
        zg_pending_steps& q = ctx->steps;
        uint32_t bits;
        memcpy(&bits, &value, sizeof(bits));
        if (bits == 0u && x && n)
            for (int i = 0; i < q.count; i++)
                if (q.g[i] == x && q.n[i] == n && !q.zero[i]) {
                    q.zero[i] = true;
                    return ZG_HIP_OK;
                }
        if (int rc = flush_steps(ctx, true)) return rc;
    }
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "mem_fill: null pointer");
    // The fill waits for the next call that is not a fill.  Two waiting fills never overlap (workgroups of one launch
    // would race, and the later fill must win), and their slices must fit one grid.
    size_t wgs = ceil_div_sz(n, kFillSlice);
    bool send_first = ctx->n_pending_fills == kMaxPendingFills;
    for (int i = 0; i < ctx->n_pending_fills && !send_first; i++) {
        const zg_pending_fill& p = ctx->pending_fills[i];
        if (x < p.x + p.n && p.x < x + n) send_first = true;
        wgs += ceil_div_sz(p.n, kFillSlice);
    }
    if (wgs > 0x7fffffffull) send_first = true;
    if (send_first)
        if (int rc = flush_fills(ctx)) return rc;
    ZG_REQUIRE(ceil_div_sz(n, kFillSlice) <= 0x7fffffffull, "mem_fill: more than 2^43 elements");
    ctx->pending_fills[ctx->n_pending_fills++] = zg_pending_fill{x, n, value};
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
    hipLaunchKernelGGL(fill_kernel<uint64_t>, dim3(grid_for(ctx, n, kBlock, false)), dim3(kBlock), 0, ctx->stream, x, n,
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
