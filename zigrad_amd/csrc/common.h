// Shared declarations of the gfx950 backend: context, error reporting, launch helpers.
#pragma once
#include <hip/hip_runtime.h>

// Every kernel launch of the library is counted (zg_hip_launch_count): the launches an op sequence costs are what the
// work that waits inside the context is there to cut, and tests hold them to what was measured.
#include <atomic>
namespace zg {
extern std::atomic<unsigned long long> launches_issued;  // process-wide: contexts on different threads share it
}
#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kernelName, numBlocks, numThreads, memPerBlock, streamId, ...)              \
    do {                                                                                               \
        zg::launches_issued.fetch_add(1, std::memory_order_relaxed);                                                                       \
        (kernelName)<<<(numBlocks), (numThreads), (memPerBlock), (streamId)>>>(__VA_ARGS__);           \
    } while (0)

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/zg_hip.h"

#define ZG_API extern "C" __attribute__((visibility("default")))

namespace zg {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kBlock = 256;        // default workgroup: 4 waves, one per SIMD
constexpr size_t kPoolAlign = 256; // min split size of the block pools, bytes

void set_error(const char* fmt, ...);

struct BlockPool;  // runtime.hip
struct GemmPlanCache;  // gemm.hip
struct PlanCache;  // index.hip
struct CachedPlan;

// One use of a cached segment plan by an op call: the entry and the caller's index arrays it was matched against.
struct PlanUse {
    CachedPlan* entry;
    const uint64_t* keys;
    const uint64_t* payload;
};

}  // namespace zg

struct zg_hip_event {
    hipEvent_t ev;
};

// A float fill that has been asked for and not launched yet (runtime.hip).
struct zg_pending_fill {
    float* x;
    size_t n;
    float value;
};
constexpr int kMaxPendingFills = 16;

// A single (unbatched) product C = alpha op(A) op(B) that has been asked for and not launched yet (gemm.hip).
struct zg_deferred_gemm {
    bool active = false;
    int kind = 0;         // 1: a layer's forward product (A as stored, B transposed); 2: an input-gradient product
    bool zeroed = false;  // the product took over a waiting zero fill of C (it was asked for as C += ...)
    const float* A = nullptr;
    const float* B = nullptr;
    float* C = nullptr;
    size_t m = 0, n = 0, k = 0, lda = 0, ldb = 0, ldc = 0;
    int trans_a = 0, trans_b = 0;
    float alpha = 1.f;
    const float* bias = nullptr;  // attached by a following row-broadcast add onto C
    const float* gate = nullptr;  // attached by a following relu_inplace_bwd on C
    int relu = 0;                 // attached by a following in-place relu_fwd on C
    const char* name = "matmul";
};

// The bias gradient of a small Linear layer (gb += column sums of gy, one launch of the column kernel) that has been
// asked for and not launched yet: the layer's two products follow it and can share its launch (gemm.hip).
struct zg_waiting_bias {
    bool active = false;
    const float* gy = nullptr;  // [R, inner]
    float* gb = nullptr;        // [inner]
    size_t R = 0, inner = 0;
    bool fresh = false;         // gb's zero fill was taken over: the sums are written (a sum of floats that starts from
                                // +0.0 is never -0.0, so s and s + 0.0 are the same bits)
};

// The aggregation of a graph-convolution layer (scatter_gcn_deg_scaled) whose plan is ready and whose apply kernel has
// not been launched yet: the layer's bias add and ReLU follow it and run as the kernel's tail (index.hip).
struct zg_waiting_scatter {
    bool active = false;
    float* dst = nullptr;
    const float* h = nullptr;
    const float* deg = nullptr;
    const uint32_t* row_ptr = nullptr;
    const uint32_t* peer = nullptr;
    const uint32_t* long_list = nullptr;  // the ordering's buckets of many entries, which a second kernel adds up
    size_t n_entries = 0;
    long n_long = -1;
    size_t n_nodes = 0, stride = 0;
    bool fresh = false;           // written, not added to (the output's zero fill was taken over)
    const float* bias = nullptr;  // attached by a following row-broadcast add onto dst
    int relu = 0;                 // attached by a following in-place relu_fwd on dst
};

// The degree gradient of scatter_gcn_deg_scaled_bwd (two launches: the edge terms, then their sums per node), asked
// for and not launched yet: the reference's graph-convolution layer computes it into a buffer that it gives back
// unread (the degrees are data of the graph, src/ndtensor.zig:1009), and a job whose output block is freed while
// it waits is dropped (index.hip).
struct zg_waiting_graddeg {
    bool active = false;
    bool by_incidence = false;
    const float* grad_output = nullptr;
    const float* h = nullptr;
    const float* deg = nullptr;
    const uint64_t* src_idx = nullptr;
    const uint64_t* tgt_idx = nullptr;
    size_t n_edge = 0, n_nodes = 0, stride = 0;
    float* grad_deg = nullptr;
    bool fresh = false;
    // by_incidence: terms in bucket order
    const uint32_t* slot_of = nullptr;
    const uint32_t* inc_row_ptr = nullptr;
    const uint32_t* inc_long_list = nullptr;  // the nodes of more than 256 terms, which a second kernel adds up
    // otherwise: two term arrays and the two orderings
    float* term_src = nullptr;
    float* term_tgt = nullptr;
    const uint32_t* rp_src = nullptr;
    const uint32_t* perm_src = nullptr;
    const uint32_t* rp_tgt = nullptr;
    const uint32_t* perm_tgt = nullptr;
    // room for the terms of every node laid out in the order they are added (null: the node's two lists are merged as
    // they are read), the row pointers of that layout and the list of nodes with many terms
    float* merged = nullptr;
    uint32_t* rp_merged = nullptr;
    uint32_t* long_merged = nullptr;
};

// Small elementwise ops of one length that have been asked for and not launched yet (elementwise.hip): the reference's
// autograd issues runs of them (a target r + gamma * max * (1 - done), a degree normalisation rsqrt(deg + count)), and
// a run leaves as one launch in which thread i carries element i through every op in call order.
constexpr int kMaxWaitingMaps = 8;
constexpr size_t kWaitingMapMaxLen = 65536;
struct zg_map_op {
    int code;           // which functor (elementwise.hip)
    int nin;            // array operands read: a, then b, then c
    int scalar;         // 0: every operand has one element per output; 1: b is one float; 2: a is one float
    int subst;          // bit 0 / 1 / 2: operand a / b / c is the output itself, over which a fill was still waiting when
    float subst_value;  // the op was asked for: the op takes the fill's value instead of loading, and the fill is dropped
    float* out;
    const float* a;
    const float* b;
    const float* c;
    float p0, p1;
};
struct zg_waiting_maps {
    int count = 0;
    size_t n = 0;
    zg_map_op op[kMaxWaitingMaps];
};

// Optimizer steps of small tensors that have been asked for and not launched yet (optim.hip).
constexpr int kMaxPendingSteps = 16;
struct zg_pending_steps {
    int count = 0;
    int kind = 0;  // 0 SGD, 1 Adam with lr_t by value, 2 Adam with lr_t read from memory when the kernel runs
    float* p[kMaxPendingSteps];
    float* g[kMaxPendingSteps];
    float* m[kMaxPendingSteps];
    float* v[kMaxPendingSteps];
    size_t n[kMaxPendingSteps];
    float lr_t[kMaxPendingSteps];            // kind 1
    const float* lr_t_mem[kMaxPendingSteps]; // kind 2
    bool zero[kMaxPendingSteps];             // a zero fill of exactly this gradient arrived while the step waited
    float lr = 0.f, b1 = 0.f, b2 = 0.f, eps = 0.f, max_norm = 0.f, delta = 0.f;
    int clip = 0;
};

struct zg_hip_ctx {
    int device = 0;
    int n_cu = 256;
    size_t total_mem = 0;
    hipStream_t stream = nullptr;

    // Internal workspace for multi-stage reductions and sort plans. Grow-only; growth synchronises the stream.
    void* ws = nullptr;
    size_t ws_bytes = 0;

    // small device slots for scalars: [0] staged host scalar (axpy alpha), [1] clip factor
    float* scalar_slot = nullptr;
    // fixed buffer for the per-workgroup partials of flat reductions (64 KiB)
    void* partials = nullptr;
    // pinned host memory that small device-to-host copies go through (runtime.hip)
    void* d2h_slot = nullptr;

    // address, on this context's device, of the fixed scratch array of the allocation-free entry point (loss.hip)
    void* noalloc_scratch = nullptr;
    size_t noalloc_scratch_bytes = 0;

    // caching allocator state (runtime.hip)
    zg::BlockPool* small_pool = nullptr;
    zg::BlockPool* large_pool = nullptr;
    size_t small_pool_bytes = 0;
    size_t large_pool_bytes = 0;
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    uint64_t n_device_allocs = 0;

    // input staging (runtime.hip): second stream for host-to-device copies, one event per direction
    hipStream_t copy_stream = nullptr;
    hipEvent_t ev_compute = nullptr, ev_copy = nullptr;

    // execution-graph capture (runtime.hip): while `capturing`, the address range of every cache block handed out
    // or returned is noted; the free part of those ranges stays with the graph when the recording ends, so a
    // replay never meets another owner at those addresses
    bool capturing = false;
    std::vector<std::pair<char*, size_t>> capture_touched;
    int live_graphs = 0;
    std::vector<void*> retired_ws;  // outgrown workspaces that an instantiated graph may still name

    // segment plans of index arrays in pinned host memory, kept between calls and matched by content (index.hip);
    // plan_uses: the cached plans the ops of the recording in progress launched their kernels on
    zg::PlanCache* plan_cache = nullptr;
    std::vector<zg::PlanUse> plan_uses;

    // Float fills wait here until the next call that is not a fill (or an allocation) and then go out as one launch:
    // callers zero their gradients tensor by tensor (examples/mnist/src/model.zig:57-62: one fill per parameter), and a
    // launch per tensor costs more than the fills themselves.  Every entry point starts with ZG_CTX, which sends
    // the waiting fills first, so no call can see memory that a fill has not reached yet.
    zg_pending_fill pending_fills[kMaxPendingFills];
    int n_pending_fills = 0;
    // hold_work false (zg_hip_set_holding): nothing stays waiting past the call that queued it, for callers that mix
    // their own HIP calls with the library's.  late_error: what launching held work at the end of such a call
    // returned; the next call on the context reports it.
    bool hold_work = true;
    int late_error = 0;

    // A layer's forward product waits one call for the bias add and the ReLU that the reference's Linear layer issues
    // right after it (examples/mnist/src/model.zig:104-110, :38-46), and an input-gradient product waits for the
    // relu_inplace_bwd that masks it (src/nn/nn.zig:44-50), letting one independent product (the weight gradient,
    // src/ndtensor.zig:1126-1128) pass: what follows is then done in the product's epilogue, the same IEEE operations
    // in the same order, instead of in one more pass over the output each.  Any other call launches the product as it
    // is, first thing (ZG_CTX), so no call ever sees memory the product has not reached; fills and a waiting product
    // never coexist (a fill launches the product first, a product launches the fills first).
    zg_deferred_gemm deferred;
    // The backward pass of a small Linear layer, gathered call by call: the bias gradient (asked for first), the
    // input-gradient product (`deferred`, kind 2, waiting for its mask) and the weight-gradient product that follows
    // it leave in one launch when the mask arrives.
    zg_deferred_gemm deferred_w;
    zg_waiting_bias bias_wait;
    zg_waiting_scatter scatter_wait;
    zg_waiting_graddeg graddeg_wait;
    zg_waiting_maps maps;
    // Cache blocks that were given back while a waiting input-gradient product still names them as operands (the
    // reference frees a node's gradient as soon as its backward has run, src/ndtensor.zig eager teardown): they return
    // to the pool right after the product is launched.
    struct {
        void* ptr;
        uint64_t block;
    } deferred_frees[4];
    int n_deferred_frees = 0;

    // Optimizer steps of tensors of up to 2^20 elements wait here while the calls that follow are more optimizer steps
    // with the same settings (Optimizer.step() walks its parameter list, src/nn/optim.zig:100-122, :177-234) and then
    // leave in the two launches of the parameter-list kernels instead of one to three launches each; same values.
    zg_pending_steps steps;

    // launch plans of the staged GEMM kernels, by shape (gemm.hip)
    zg::GemmPlanCache* gemm_plans = nullptr;

    // regions handed out by pool_map/alloc, for ownership checks at free time
    std::map<void*, size_t> raw_allocs;
    std::map<void*, size_t> host_allocs;
    // Pinned host blocks that were given back and are kept for the next zg_hip_host_alloc of their size class
    // (runtime.hip): a binding serves every `usize` tensor from pinned memory, one or more per train step, and the
    // driver's pinned allocation and release cost far more than a step's kernels.  `done` marks the point on the
    // stream after which no queued kernel reads the block; the next owner waits for it before it gets the block.
    struct HostBlock {
        void* ptr;
        size_t cap;
        hipEvent_t done;
    };
    std::map<void*, size_t> host_caps;  // capacity (size class) of every live pinned allocation
    std::vector<HostBlock> host_free_blocks;
    size_t host_cached_bytes = 0;
};

namespace zg {

// Returns a workspace of at least `bytes` bytes (256-byte aligned), or nullptr with the error set.
void* workspace(zg_hip_ctx* ctx, size_t bytes);

// Cached segment plans (index.hip).  destroy: at deinit.  retain: a saved graph takes (+1) or drops (-1) its plans,
// which are never evicted while a graph names them.  validate: before a replay, every index array the recording
// matched must still hold what it held then, or the replay would scatter by a stale plan.
// Blocking copy of a few bytes (at most 4096) from device memory to pageable host memory (runtime.hip).
int small_d2h(zg_hip_ctx* ctx, void* dst_host, const void* src, size_t bytes);
// Launches the fills that are waiting in the context (one kernel for all of them).
int flush_fills(zg_hip_ctx* ctx);
// Launches the waiting product with whatever was attached to it, and the waiting bias gradient and weight-gradient
// product of the same layer (gemm.hip).  gemm_group_waiting: whether any of the three waits.
int flush_deferred_gemm(zg_hip_ctx* ctx);
inline bool gemm_group_waiting(const zg_hip_ctx* ctx) {
    return ctx->deferred.active || ctx->deferred_w.active || ctx->bias_wait.active;
}
// Whether [lo, hi) meets an operand of the waiting products or of the waiting bias gradient (gemm.hip), of the waiting
// optimizer steps (optim.hip), of the waiting aggregation or degree gradient (index.hip), of the waiting elementwise
// ops (elementwise.hip): what kind_touches asks, kind by kind.
bool gemm_group_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi);
bool steps_touch(const zg_hip_ctx* ctx, const char* lo, const char* hi);
bool scatter_wait_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi);
bool graddeg_wait_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi);
bool maps_touch(const zg_hip_ctx* ctx, const char* lo, const char* hi);
// The single-chunk column sum y += column sums of x[R, inner] (reduce.hip), the launch the waiting bias gradient owes.
int launch_bias_col_sum(zg_hip_ctx* ctx, const float* x, float* y, size_t R, size_t inner, bool fresh);
// Launches the waiting graph-convolution aggregation with what was attached to it (index.hip); the two hooks are for
// zg_hip_add and zg_hip_relu_fwd, like deferred_take_add / deferred_take_relu below.
int flush_scatter(zg_hip_ctx* ctx);
// Launches the waiting degree gradient (index.hip).
int flush_graddeg(zg_hip_ctx* ctx);
// Launches the waiting elementwise ops as one kernel (elementwise.hip).
int flush_maps(zg_hip_ctx* ctx);
// Queues out[i] = c added to +0.0 (row_ptr[i + 1] - row_ptr[i]) times, i < n, with the waiting elementwise ops: what
// scatter_add of a constant source into a destination of zeros comes to once the offsets are sorted into buckets
// (index.hip).  False: not queued (*rc says whether something failed), the caller launches its own kernel.
bool maps_push_count(zg_hip_ctx* ctx, float* out, const uint32_t* row_ptr, size_t n, float c, int* rc);
// Whether a waiting fill meets one of the byte ranges; take_fill_exact: a waiting fill of exactly x[0 .. n) is dropped
// and its value handed over (the caller overwrites all of the range and uses the value where it would have read it);
// drop_fills_inside: waiting fills that lie wholly inside a range the caller overwrites without reading it.
bool fills_touch(zg_hip_ctx* ctx, const void* const* ptrs, const size_t* bytes, int count);
bool take_fill_exact(zg_hip_ctx* ctx, const float* x, size_t n, float* value);
void drop_fills_inside(zg_hip_ctx* ctx, const void* lo, size_t bytes);
// The same, handing the dropped fills to the caller (`out` holds kMaxPendingFills): a call that then fails owes them
// back (requeue_fills), because the memory was not overwritten after all.
int take_fills_inside(zg_hip_ctx* ctx, const void* lo, size_t bytes, zg_pending_fill* out);
void requeue_fills(zg_hip_ctx* ctx, const zg_pending_fill* fills, int count);
bool scatter_take_add(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, const float* z, size_t zl);
bool scatter_take_relu(zg_hip_ctx* ctx, const float* x, const float* y, size_t n, int* rc);
// Launches the optimizer steps that are waiting (optim.hip).  Gradients whose zero fill was taken over are zeroed by
// the update kernel when every waiting step has one; otherwise their fills are launched after the steps, or, with
// requeue_fills, put back among the waiting fills for the caller (zg_hip_mem_fill) to send with its own.
int flush_steps(zg_hip_ctx* ctx, bool requeue_fills = false);
// Returns to the pools the blocks whose free waited for the product (runtime.hip); called once it is launched.
void run_deferred_frees(zg_hip_ctx* ctx);
// ------------------------------------------------------------------------------------------------
// The one mechanism behind every kind of waiting work.  A kind is a bit; for each kind the context can say whether
// work of that kind waits (waiting_kinds), launch it (flush_kinds, always in the order maps, aggregation, degree
// gradient, products, fills, steps: kinds that wait at the same time touch disjoint memory, so any fixed order does),
// and tell whether it would read or write a byte range (kind_touches).  An entry point starts with
// ZG_ENTER(ctx, keep): everything that waits is launched except the kinds in `keep`, which the entry point looks at
// itself (to join them, to take them over, or to launch them only if they meet its operands: flush_touching).
// ------------------------------------------------------------------------------------------------
enum : unsigned {
    kWaitFills = 1u,     // float fills (runtime.hip)
    kWaitProducts = 2u,  // a layer's forward or input-gradient product, the weight-gradient product and the bias
                         // gradient that wait with it (gemm.hip)
    kWaitSteps = 4u,     // optimizer steps (optim.hip)
    kWaitScatter = 8u,   // a graph-convolution aggregation (index.hip)
    kWaitGradDeg = 16u,  // a degree gradient (index.hip)
    kWaitMaps = 32u,     // small elementwise ops (elementwise.hip)
    kWaitAll = 63u,
};
struct ByteSpan {
    const void* p;
    size_t bytes;
};
inline unsigned waiting_kinds(const zg_hip_ctx* ctx) {
    return (ctx->n_pending_fills ? kWaitFills : 0u) |
           ((ctx->deferred.active || ctx->deferred_w.active || ctx->bias_wait.active) ? kWaitProducts : 0u) |
           (ctx->steps.count ? kWaitSteps : 0u) | (ctx->scatter_wait.active ? kWaitScatter : 0u) |
           (ctx->graddeg_wait.active ? kWaitGradDeg : 0u) | (ctx->maps.count ? kWaitMaps : 0u);
}
// Launches what waits of the given kinds (runtime.hip).
int flush_kinds(zg_hip_ctx* ctx, unsigned kinds);
// Whether waiting work of one kind reads or writes any byte of the spans (null spans are skipped).
bool kind_touches(const zg_hip_ctx* ctx, unsigned kind, const ByteSpan* spans, int count);
// Of the given kinds, launches those whose waiting work meets the spans; the others keep waiting.
int flush_touching(zg_hip_ctx* ctx, unsigned kinds, const ByteSpan* spans, int count);
// Everything that waits: what a call that knows nothing about waiting work starts with.
inline int flush_pending(zg_hip_ctx* ctx) { return flush_kinds(ctx, kWaitAll); }
// Everything but the fills, and the fills too when one of them meets one of the `count` byte ranges the caller is about
// to read or write.
int flush_pending_but_fills(zg_hip_ctx* ctx, const void* const* ptrs, const size_t* bytes, int count);
// A call that may be absorbed by the waiting product: true when it was (then *rc is the call's result and the caller
// returns it), false when the call has to run as usual.
bool deferred_take_add(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, const float* z, size_t zl);
bool deferred_take_relu(zg_hip_ctx* ctx, const float* x, const float* y, size_t n, int* rc);
bool deferred_take_relu_mask(zg_hip_ctx* ctx, const float* x, const float* x_g, size_t n, int* rc);
// An op that adds into x[0 .. n) asks whether a fill of exactly that range with +0.0 is still waiting.  If so the fill
// is dropped and true comes back: the op then writes its result instead of adding it to zeros it would have to read
// (ensure_grad(0) followed by an accumulating backward op, src/ndtensor.zig:221-228), the same values without the
// fill's launch and without the read.
bool absorb_zero_fill(zg_hip_ctx* ctx, const float* x, size_t n);

inline bool anything_waits(const zg_hip_ctx* ctx) { return waiting_kinds(ctx) != 0u; }
// Lives for the length of an entry point (the ZG_CTX* macros declare one): with holding switched off, whatever the
// call queued is launched before the call returns.
struct HoldGuard {
    zg_hip_ctx* ctx;
    ~HoldGuard() {
        if (ctx && !ctx->hold_work && anything_waits(ctx))
            if (int rc = flush_pending(ctx)) ctx->late_error = rc;
    }
};

void plan_cache_destroy(zg_hip_ctx* ctx);
void gemm_plans_destroy(zg_hip_ctx* ctx);
void plan_uses_retain(const std::vector<PlanUse>& uses, int delta);
int plan_uses_validate(zg_hip_ctx* ctx, const std::vector<PlanUse>& uses);

// Looks up the device address of the fixed scratch array (loss.hip); the context's device must be current.
int noalloc_setup(zg_hip_ctx* ctx);

inline int ceil_div(size_t a, size_t b) {
    return (int)((a + b - 1) / b);
}
// d(mean smooth-L1)/d(pred) of one element (src/nn/loss.zig:259-305): (pred - target) / (beta * n) where
// |pred - target| < beta, sign(pred - target) / n elsewhere
__device__ __forceinline__ float smooth_l1_grad(float pred, float target, float beta, float n) {
    const float d = __fsub_rn(pred, target);
    if (fabsf(d) < beta) return __fdiv_rn(d, __fmul_rn(beta, n));
    const float sg = (d > 0.f) ? 1.f : ((d < 0.f) ? -1.f : 0.f);
    return __fdiv_rn(sg, n);
}

inline size_t ceil_div_sz(size_t a, size_t b) {
    return (a + b - 1) / b;
}
inline bool aligned16(const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace zg

#define ZG_REQUIRE(cond, ...)             \
    do {                                  \
        if (!(cond)) {                    \
            zg::set_error(__VA_ARGS__);   \
            return ZG_HIP_EINVAL;         \
        }                                 \
    } while (0)

#define ZG_HIP_TRY(expr)                                                                         \
    do {                                                                                         \
        hipError_t _e = (expr);                                                                  \
        if (_e != hipSuccess) {                                                                  \
            zg::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return (_e == hipErrorOutOfMemory) ? ZG_HIP_EOOM : ZG_HIP_ERUNTIME;                  \
        }                                                                                        \
    } while (0)

// After a kernel launch: report launch-configuration errors without synchronising.
#define ZG_LAUNCH_CHECK()                                                                        \
    do {                                                                                         \
        hipError_t _e = hipGetLastError();                                                       \
        if (_e != hipSuccess) {                                                                  \
            zg::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(_e), __FILE__, __LINE__); \
            return ZG_HIP_ERUNTIME;                                                              \
        }                                                                                        \
    } while (0)

// What ZG_ENTER starts with: a context, the guard for contexts that hold nothing, and the error that launching held
// work at the end of an earlier call left behind.
#define ZG_CTX_ENTER(ctx)                                    \
    ZG_REQUIRE((ctx) != nullptr, "null context");            \
    zg::HoldGuard _zg_hold_guard{(ctx)};                     \
    (void)_zg_hold_guard;                                    \
    if ((ctx)->late_error) {                                 \
        const int _rc_late = (ctx)->late_error;              \
        (ctx)->late_error = 0;                               \
        return _rc_late;                                     \
    }
// First statement of every entry point.  `keep`: the kinds of waiting work (kWait* bits) the entry point deals with
// itself; everything else that waits is launched before the call's own work is queued, so no call can observe memory
// that waiting work has not reached.  ZG_CTX is the common case: the entry point knows nothing of waiting work.
#define ZG_ENTER(ctx, keep)                                                                    \
    ZG_CTX_ENTER(ctx)                                                                          \
    if (const unsigned _zg_w = zg::waiting_kinds(ctx) & ~(unsigned)(keep)) {                   \
        if (int _rc_w = zg::flush_kinds(ctx, _zg_w)) return _rc_w;                             \
    }
#define ZG_CTX(ctx) ZG_ENTER(ctx, 0u)

// Entry points that synchronise, allocate from the driver or touch host memory cannot be recorded into a graph.
#define ZG_NOT_CAPTURING(ctx, who)                                                                       \
    do {                                                                                                 \
        if ((ctx)->capturing) {                                                                          \
            zg::set_error("%s: not allowed while an execution graph is being captured", who);            \
            return ZG_HIP_ECAPTURE;                                                                      \
        }                                                                                                \
    } while (0)
