// Fused optimizer updates: src/nn/optim.zig:100-122 (SGD.update) and :177-234 (Adam.update), one op
// per parameter tensor.  The per-tensor gradient clip never synchronises with the host: a reduction
// leaves the clip factor in a device slot and the update kernel reads it.
//
// HBM traffic per element: SGD reads p,g and writes p (12 B; +4 B when the clip changes g);
// Adam reads p,g,m,v and writes p,m,v (28 B; +4 B when the clip changes g).
#include "reduce_device.h"

namespace zg {

// zero_g: the gradient is left zero instead of clipped (zero_grad() right after step(): one pass less over it)
template <bool CLIP>
__global__ __launch_bounds__(kBlock) void sgd_kernel(float* p, float* g, size_t n, float nlr, const float* factor,
                                                      bool zero_g) {
    const float f = CLIP ? factor[0] : 1.0f;
    const bool scale = CLIP && (f != 1.0f);
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g)) & 15u) == 0;
    size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    if (vec) {
        float4* p4 = reinterpret_cast<float4*>(p);
        float4* g4 = reinterpret_cast<float4*>(g);
        const size_t n4 = n >> 2;
        for (size_t i = tid; i < n4; i += nt) {
            float4 pv = p4[i], gv = g4[i];
            if (scale) {
                gv.x = __fmul_rn(gv.x, f);
                gv.y = __fmul_rn(gv.y, f);
                gv.z = __fmul_rn(gv.z, f);
                gv.w = __fmul_rn(gv.w, f);
                if (!zero_g) g4[i] = gv;
            }
            if (zero_g) g4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            pv.x = __fadd_rn(pv.x, __fmul_rn(nlr, gv.x));
            pv.y = __fadd_rn(pv.y, __fmul_rn(nlr, gv.y));
            pv.z = __fadd_rn(pv.z, __fmul_rn(nlr, gv.z));
            pv.w = __fadd_rn(pv.w, __fmul_rn(nlr, gv.w));
            p4[i] = pv;
        }
        tid += n4 << 2;
    }
    for (size_t i = tid; i < n; i += nt) {
        float gv = g[i];
        if (scale) {
            gv = __fmul_rn(gv, f);
            if (!zero_g) g[i] = gv;
        }
        if (zero_g) g[i] = 0.f;
        p[i] = __fadd_rn(p[i], __fmul_rn(nlr, gv));
    }
}

__device__ __forceinline__ void adam_elem(float& p, float& g, float& m, float& v, bool scale, float f, float lr_t,
                                          float b1, float b2, float omb1, float omb2, float eps) {
    if (scale) g = __fmul_rn(g, f);
    // src/nn/optim.zig:226-229, evaluated left to right in fp32
    m = __fadd_rn(__fmul_rn(b1, m), __fmul_rn(omb1, g));
    v = __fadd_rn(__fmul_rn(b2, v), __fmul_rn(__fmul_rn(omb2, g), g));
    p = __fsub_rn(p, __fdiv_rn(__fmul_rn(lr_t, m), __fadd_rn(sqrtf(v), eps)));
}

template <bool CLIP>
__global__ __launch_bounds__(kBlock) void adam_kernel(float* p, float* g, float* m, float* v, size_t n,
                                                       float lr_t_value, const float* lr_t_ptr, float b1, float b2,
                                                       float omb1, float omb2, float eps, const float* factor,
                                                       bool zero_g) {
    const float lr_t = lr_t_ptr ? lr_t_ptr[0] : lr_t_value;
    const float f = CLIP ? factor[0] : 1.0f;
    const bool scale = CLIP && (f != 1.0f);
    const bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                       reinterpret_cast<uintptr_t>(v)) & 15u) == 0;
    size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    if (vec) {
        float4* p4 = reinterpret_cast<float4*>(p);
        float4* g4 = reinterpret_cast<float4*>(g);
        float4* m4 = reinterpret_cast<float4*>(m);
        float4* v4 = reinterpret_cast<float4*>(v);
        const size_t n4 = n >> 2;
        for (size_t i = tid; i < n4; i += nt) {
            float4 pv = p4[i], gv = g4[i], mv = m4[i], vv = v4[i];
            adam_elem(pv.x, gv.x, mv.x, vv.x, scale, f, lr_t, b1, b2, omb1, omb2, eps);
            adam_elem(pv.y, gv.y, mv.y, vv.y, scale, f, lr_t, b1, b2, omb1, omb2, eps);
            adam_elem(pv.z, gv.z, mv.z, vv.z, scale, f, lr_t, b1, b2, omb1, omb2, eps);
            adam_elem(pv.w, gv.w, mv.w, vv.w, scale, f, lr_t, b1, b2, omb1, omb2, eps);
            if (zero_g) g4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            else if (scale) g4[i] = gv;
            m4[i] = mv;
            v4[i] = vv;
            p4[i] = pv;
        }
        tid += n4 << 2;
    }
    for (size_t i = tid; i < n; i += nt) {
        float pv = p[i], gv = g[i], mv = m[i], vv = v[i];
        adam_elem(pv, gv, mv, vv, scale, f, lr_t, b1, b2, omb1, omb2, eps);
        if (zero_g) g[i] = 0.f;
        else if (scale) g[i] = gv;
        m[i] = mv;
        v[i] = vv;
        p[i] = pv;
    }
}

// The update loop of the one-workgroup kernels: eight independent elements in flight per thread (the loop is latency
// bound: one element per trip cost a memory round trip each), same arithmetic per element as sgd_kernel / adam_kernel.
constexpr int kInFlight = 8;  // elements per thread and trip
template <bool ADAM>
__device__ __forceinline__ void update_in_workgroup(float* p, float* g, float* m, float* v, size_t n, bool scale, float f,
                                                    float lr_t, float b1, float b2, float omb1, float omb2, float eps,
                                                    bool zero_grads) {
    const size_t nt = blockDim.x;
    for (size_t base = threadIdx.x; base < n; base += kInFlight * nt) {
        float gv[kInFlight], pv[kInFlight], mv[kInFlight], vv[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const size_t i = base + (size_t)u * nt;
            const bool ok = i < n;
            gv[u] = ok ? g[i] : 0.f;
            pv[u] = ok ? p[i] : 0.f;
            mv[u] = (ADAM && ok) ? m[i] : 0.f;
            vv[u] = (ADAM && ok) ? v[i] : 1.f;
        }
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const size_t i = base + (size_t)u * nt;
            if (i >= n) continue;
            if (ADAM) {
                adam_elem(pv[u], gv[u], mv[u], vv[u], scale, f, lr_t, b1, b2, omb1, omb2, eps);
                m[i] = mv[u];
                v[i] = vv[u];
                p[i] = pv[u];
            } else {
                if (scale) gv[u] = __fmul_rn(gv[u], f);
                p[i] = __fadd_rn(pv[u], __fmul_rn(lr_t, gv[u]));
            }
            if (zero_grads) g[i] = 0.f;
            else if (scale) g[i] = gv[u];
        }
    }
}

// Small tensors with the gradient clip on: one workgroup computes the norm exactly as flat_single_kernel does (same
// per-thread accumulation and the same combine tree), publishes the clip factor, and goes on to the update.
// One launch instead of two; the arithmetic per element is that of sgd_kernel / adam_kernel, so the values are
// the same.  `factor_out` keeps the slot the two-kernel path fills.
constexpr size_t kClippedSingleMax = 4096;  // Adam: beyond this the update alone keeps one compute unit busy for microseconds
constexpr size_t kClippedSgdSingleMax = 32768;  // SGD: 65536 elements take 13 us this way, 9 us as a norm and an update launch
template <bool ADAM>
__global__ __launch_bounds__(kFlatSingle) void clipped_update_small_kernel(float* p, float* g, float* m, float* v,
                                                                           size_t n, float step_scale,
                                                                           const float* lr_t_ptr, float b1, float b2,
                                                                           float omb1, float omb2, float eps,
                                                                           float max_norm, float delta,
                                                                           float* factor_out) {
    __shared__ float smem[kFlatSingle / kWave];
    __shared__ float factor_s;
    float acc = flat_accumulate<TermSq, 1>(g, nullptr, n, 0.f, threadIdx.x, blockDim.x);
    acc = block_reduce<SumAcc>(acc, smem);
    if (threadIdx.x == 0) {
        FinClipFactor{&factor_s, max_norm, delta}(acc);
        factor_out[0] = factor_s;
    }
    __syncthreads();
    const float f = factor_s;
    const bool scale = f != 1.0f;
    const float lr_t = (ADAM && lr_t_ptr) ? lr_t_ptr[0] : step_scale;  // SGD: step_scale = -lr
    update_in_workgroup<ADAM>(p, g, m, v, n, scale, f, lr_t, b1, b2, omb1, omb2, eps, false);
}

// The same update for up to kMultiMax small tensors in two launches (one without the clip).  norm_multi_kernel:
// workgroup b forms tensor b's clip factor as clipped_update_small_kernel does (same accumulation tree).
// update_multi_kernel: the tensors are cut into slices of kMultiSlice elements, one workgroup each, so that a tensor
// of tens of thousands of elements is spread over many compute units (the update is arithmetic-bound on one); each
// workgroup looks up its tensor's factor, reads its lr_t from memory when asked to, and with `zero_grads` leaves the
// gradient zero instead of clipped (optim.step() followed by model.zero_grad(),
// examples/mnist/src/main-simple.zig:70-71).  The arithmetic per element is that of sgd_kernel / adam_kernel.
constexpr int kMultiMax = 16;
constexpr int kMultiThreads = 256;
constexpr int kMultiSlice = kMultiThreads * kInFlight;  // one trip of update_in_workgroup
struct MultiArgs {
    float* p[kMultiMax];
    float* g[kMultiMax];
    float* m[kMultiMax];
    float* v[kMultiMax];
    size_t n[kMultiMax];
    float lr_t[kMultiMax];       // Adam: lr_t per tensor; SGD: -lr
    int wg_first[kMultiMax + 1]; // update_multi_kernel: tensor b owns workgroups wg_first[b] .. wg_first[b + 1] - 1
    const float* lr_t_mem[kMultiMax];  // Adam under replay: *lr_t_mem[b] is read when the kernel runs (null: use lr_t[b])
    float* factors;              // clip factor per tensor, written by norm_multi_kernel
    float* partials[kMultiMax];  // tensors beyond kFlatSingleMax: the first-stage sums of norm_partials_multi_kernel
    int n_partials[kMultiMax];   //   and how many (0: the tensor's norm is formed by one workgroup)
    int part_first[kMultiMax + 1];  // norm_partials_multi_kernel: tensor b owns workgroups part_first[b] .. part_first[b + 1] - 1
    float b1, b2, omb1, omb2, eps, max_norm, delta;
    int clip, zero_grads, count;
};

// First stage of the squared norms of the tensors beyond kFlatSingleMax, all in one launch: each workgroup runs the
// block of flat_partial_kernel it would run in the tensor's own launch.
__global__ __launch_bounds__(kFlatBlock) void norm_partials_multi_kernel(MultiArgs a) {
    __shared__ float smem[kFlatBlock / kWave];
    int b = 0;
    while (b + 1 < a.count && (int)blockIdx.x >= a.part_first[b + 1]) b++;
    flat_partial_block<TermSq, 1>(a.g[b], nullptr, a.n[b], 0.f, a.partials[b], (size_t)((int)blockIdx.x - a.part_first[b]),
                                  (size_t)a.n_partials[b], smem);
}

__global__ __launch_bounds__(kFlatSingle) void norm_multi_kernel(MultiArgs a) {
    __shared__ float smem[kFlatSingle / kWave];
    const int b = blockIdx.x;
    float acc = 0.f;
    if (a.n_partials[b]) {
        // the second stage as flat_final_kernel runs it: kFlatBlock threads gather, the others hold zeros, which
        // leave every sum of the combine tree as it is
        if (threadIdx.x < kFlatBlock)
            for (int i = threadIdx.x; i < a.n_partials[b]; i += kFlatBlock) acc = SumAcc::combine(acc, a.partials[b][i]);
    } else {
        acc = flat_accumulate<TermSq, 1>(a.g[b], nullptr, a.n[b], 0.f, threadIdx.x, blockDim.x);
    }
    acc = block_reduce<SumAcc>(acc, smem);
    if (threadIdx.x == 0) FinClipFactor{a.factors + b, a.max_norm, a.delta}(acc);
}

template <bool ADAM>
__global__ __launch_bounds__(kMultiThreads) void update_multi_kernel(MultiArgs a) {
    int b = 0;
    while (b + 1 < a.count && (int)blockIdx.x >= a.wg_first[b + 1]) b++;
    const size_t off = (size_t)((int)blockIdx.x - a.wg_first[b]) * kMultiSlice;
    const size_t left = a.n[b] - off;
    const size_t n = left < (size_t)kMultiSlice ? left : (size_t)kMultiSlice;
    const float f = a.clip ? a.factors[b] : 1.0f;
    const bool scale = f != 1.0f;
    const float lr_t = (ADAM && a.lr_t_mem[b]) ? a.lr_t_mem[b][0] : a.lr_t[b];
    update_in_workgroup<ADAM>(a.p[b] + off, a.g[b] + off, ADAM ? a.m[b] + off : nullptr, ADAM ? a.v[b] + off : nullptr, n,
                              scale, f, lr_t, a.b1, a.b2, a.omb1, a.omb2, a.eps, a.zero_grads != 0);
}

static int update_grid(zg_hip_ctx* ctx, size_t n) {
    size_t blocks = ceil_div_sz(n, (size_t)kBlock * 4);
    // one trip per thread, consecutive workgroups on consecutive 4 KiB of every stream: a grid capped at 16 workgroups per
    // compute unit, every thread striding through the whole array, ran Adam on 268 M elements at 56 % of 8 TB/s against
    // 69 % (16.7 M elements: 68.7 -> 67.3 us)
    (void)ctx;
    size_t cap = 0x7fffffffull;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace zg

using namespace zg;

static int sgd_launch(zg_hip_ctx* ctx, float* param, float* grad, size_t n, float lr, int clip, float max_norm,
                      float delta) {
    float* factor = ctx->scalar_slot + 1;
    if (clip && n <= kClippedSgdSingleMax) {
        hipLaunchKernelGGL((clipped_update_small_kernel<false>), dim3(1), dim3(kFlatSingle), 0, ctx->stream, param, grad,
                           (float*)nullptr, (float*)nullptr, n, -lr, (const float*)nullptr, 0.f, 0.f, 0.f, 0.f, 0.f,
                           max_norm, delta, factor);
    } else if (clip) {
        int rc = flat_reduce<TermSq, 1>(ctx, grad, nullptr, n, 0.f, FinClipFactor{factor, max_norm, delta});
        if (rc) return rc;
        hipLaunchKernelGGL((sgd_kernel<true>), dim3(update_grid(ctx, n)), dim3(kBlock), 0, ctx->stream, param, grad, n,
                           -lr, factor, false);
    } else {
        hipLaunchKernelGGL((sgd_kernel<false>), dim3(update_grid(ctx, n)), dim3(kBlock), 0, ctx->stream, param, grad,
                           n, -lr, factor, false);
    }
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// src/nn/optim.zig:190-191, fp32 throughout
static float adam_lr_t(float lr, float beta1, float beta2, uint64_t t) {
    const float tf = (float)t;
    return lr * sqrtf(1.0f - powf(beta2, tf)) / (1.0f - powf(beta1, tf));
}

static int adam_launch(zg_hip_ctx* ctx, float* param, float* grad, float* m, float* v, size_t n, float lr_t,
                       const float* lr_t_ptr, float beta1, float beta2, float epsilon, int clip, float max_norm,
                       float delta) {
    const float omb1 = 1.0f - beta1, omb2 = 1.0f - beta2;
    float* factor = ctx->scalar_slot + 1;
    if (clip && n <= kClippedSingleMax) {
        hipLaunchKernelGGL((clipped_update_small_kernel<true>), dim3(1), dim3(kFlatSingle), 0, ctx->stream, param, grad,
                           m, v, n, lr_t, lr_t_ptr, beta1, beta2, omb1, omb2, epsilon, max_norm, delta, factor);
    } else if (clip) {
        int rc = flat_reduce<TermSq, 1>(ctx, grad, nullptr, n, 0.f, FinClipFactor{factor, max_norm, delta});
        if (rc) return rc;
        hipLaunchKernelGGL((adam_kernel<true>), dim3(update_grid(ctx, n)), dim3(kBlock), 0, ctx->stream, param, grad, m,
                           v, n, lr_t, lr_t_ptr, beta1, beta2, omb1, omb2, epsilon, factor, false);
    } else {
        hipLaunchKernelGGL((adam_kernel<false>), dim3(update_grid(ctx, n)), dim3(kBlock), 0, ctx->stream, param, grad,
                           m, v, n, lr_t, lr_t_ptr, beta1, beta2, omb1, omb2, epsilon, factor, false);
    }
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

constexpr size_t kMultiBigMax = (size_t)1 << 20;
static int step_multi(zg_hip_ctx* ctx, const char* name, bool adam, size_t n_tensors, float* const* params,
                      float* const* grads, float* const* ms, float* const* vs, const size_t* lens, const float* lr_t,
                      int lr_t_in_memory, float lr, float beta1, float beta2, float epsilon, int clip, float max_norm,
                      float delta, int zero_grads);

namespace zg {
// The waiting steps: one of them alone takes the per-tensor launches it would have taken, several take the
// parameter-list kernels (the same arithmetic per element and the same norm trees: the values do not depend on which).
static int launch_steps(zg_hip_ctx* ctx, const zg_pending_steps& q, int zero_grads) {
    if (q.count == 1) {
        if (q.kind == 0) return sgd_launch(ctx, q.p[0], q.g[0], q.n[0], q.lr, q.clip, q.max_norm, q.delta);
        return adam_launch(ctx, q.p[0], q.g[0], q.m[0], q.v[0], q.n[0], q.lr_t[0], q.kind == 2 ? q.lr_t_mem[0] : nullptr, q.b1,
                           q.b2, q.eps, q.clip, q.max_norm, q.delta);
    }
    if (q.kind == 2) {
        // lr_t read from memory: the list kernels take one base pointer and index it, so the tensors go one by one
        // unless their lr_t slots are consecutive floats
        bool consecutive = true;
        for (int i = 1; i < q.count; i++) consecutive = consecutive && q.lr_t_mem[i] == q.lr_t_mem[0] + i;
        if (!consecutive) {
            for (int i = 0; i < q.count; i++)
                if (int rc = adam_launch(ctx, q.p[i], q.g[i], q.m[i], q.v[i], q.n[i], 0.f, q.lr_t_mem[i], q.b1, q.b2, q.eps,
                                         q.clip, q.max_norm, q.delta))
                    return rc;
            return ZG_HIP_OK;
        }
        return step_multi(ctx, "adam_step_at", true, (size_t)q.count, q.p, q.g, q.m, q.v, q.n, q.lr_t_mem[0], 1, 0.f, q.b1, q.b2,
                          q.eps, q.clip, q.max_norm, q.delta, zero_grads);
    }
    return step_multi(ctx, q.kind ? "adam_step" : "sgd_step", q.kind != 0, (size_t)q.count, q.p, q.g, q.m, q.v, q.n, q.lr_t, 0,
                      q.lr, q.b1, q.b2, q.eps, q.clip, q.max_norm, q.delta, zero_grads);
}

bool steps_touch(const zg_hip_ctx* ctx, const char* lo, const char* hi) {
    const zg_pending_steps& q = ctx->steps;
    for (int i = 0; i < q.count; i++) {
        const float* arrays[4] = {q.p[i], q.g[i], q.m[i], q.v[i]};
        for (const float* a : arrays)
            if (a && (const char*)a < hi && lo < (const char*)(a + q.n[i])) return true;
        if (q.kind == 2 && q.lr_t_mem[i] && (const char*)q.lr_t_mem[i] < hi && lo < (const char*)(q.lr_t_mem[i] + 1)) return true;
    }
    return false;
}

int flush_steps(zg_hip_ctx* ctx, bool requeue_fills) {
    const zg_pending_steps q = ctx->steps;
    ctx->steps.count = 0;
    if (q.count == 0) return ZG_HIP_OK;
    int n_zero = 0;
    for (int i = 0; i < q.count; i++) n_zero += q.zero[i] ? 1 : 0;
    // zero_grad() after step(): when every waiting step's gradient is to be zeroed and the list kernels run, the update
    // kernel stores the zeros as it reads the gradients (zg_hip_*_step_multi with zero_grads)
    bool in_kernel = n_zero == q.count && q.count > 1;
    if (in_kernel && q.kind == 2)
        for (int i = 1; i < q.count; i++) in_kernel = in_kernel && q.lr_t_mem[i] == q.lr_t_mem[0] + i;
    const int rc = launch_steps(ctx, q, in_kernel ? 1 : 0);
    if (n_zero && !(in_kernel && rc == ZG_HIP_OK)) {  // the zeros are owed as fills, after the steps
        if (ctx->n_pending_fills + n_zero > kMaxPendingFills)
            if (int rcf = flush_fills(ctx)) return rc ? rc : rcf;
        for (int i = 0; i < q.count; i++)
            if (q.zero[i]) ctx->pending_fills[ctx->n_pending_fills++] = zg_pending_fill{q.g[i], q.n[i], 0.f};
        if (!requeue_fills)
            if (int rcf = flush_fills(ctx)) return rc ? rc : rcf;
    }
    return rc;
}
}  // namespace zg

// One optimizer step of one tensor.  It joins the waiting steps when it has their settings and touches none of their
// tensors (otherwise they are sent first).
static int step_entry(zg_hip_ctx* ctx, int kind, float* param, float* grad, float* m, float* v, size_t n, float lr,
                      float lr_t, const float* lr_t_mem, float b1, float b2, float eps, int clip, float max_norm,
                      float delta) {
    if (gemm_group_waiting(ctx) || ctx->n_pending_fills) {  // the gradients come from them
        if (gemm_group_waiting(ctx))
            if (int rc = flush_deferred_gemm(ctx)) return rc;
        if (int rc = flush_fills(ctx)) return rc;
    }
    zg_pending_steps& q = ctx->steps;
    // a step that touches memory a waiting step touches (the same tensor again, or buffers that overlap in any way)
    // must not share its launch: the waiting steps go first
    bool named = false;
    {
        const float* mine[4] = {param, grad, kind ? m : nullptr, kind ? v : nullptr};
        for (int i = 0; i < q.count && !named; i++) {
            const float* theirs[4] = {q.p[i], q.g[i], q.kind ? q.m[i] : nullptr, q.kind ? q.v[i] : nullptr};
            for (const float* a : mine)
                for (const float* b : theirs)
                    named = named || (a && b && a < b + q.n[i] && b < a + n);
        }
    }
    const bool same = q.count == 0 || (q.kind == kind && q.clip == clip && q.max_norm == max_norm && q.delta == delta &&
                                       (kind ? (q.b1 == b1 && q.b2 == b2 && q.eps == eps) : q.lr == lr));
    if (named || !same || q.count == kMaxPendingSteps)
        if (int rc = flush_steps(ctx)) return rc;
    if (q.count == 0) {
        q.kind = kind;
        q.lr = lr;
        q.b1 = b1;
        q.b2 = b2;
        q.eps = eps;
        q.clip = clip;
        q.max_norm = max_norm;
        q.delta = delta;
    }
    const int i = q.count++;
    q.p[i] = param;
    q.g[i] = grad;
    q.m[i] = m;
    q.v[i] = v;
    q.n[i] = n;
    q.lr_t[i] = lr_t;
    q.lr_t_mem[i] = lr_t_mem;
    q.zero[i] = false;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_sgd_step(zg_hip_ctx* ctx, float* param, float* grad, size_t n, float lr, int clip, float max_norm,
                           float delta) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(param && grad, "sgd_step: null pointer");
    return step_entry(ctx, 0, param, grad, nullptr, nullptr, n, lr, 0.f, nullptr, 0.f, 0.f, 0.f, clip, max_norm, delta);
}

ZG_API int zg_hip_adam_step(zg_hip_ctx* ctx, float* param, float* grad, float* m, float* v, size_t n, uint64_t t,
                            float lr, float beta1, float beta2, float epsilon, int clip, float max_norm, float delta) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(param && grad && m && v, "adam_step: null pointer");
    ZG_REQUIRE(t >= 1, "adam_step: t must be >= 1");
    return step_entry(ctx, 1, param, grad, m, v, n, 0.f, adam_lr_t(lr, beta1, beta2, t), nullptr, beta1, beta2, epsilon, clip,
                      max_norm, delta);
}

ZG_API int zg_hip_adam_lr_t(float lr, float beta1, float beta2, uint64_t t, float* lr_t) {
    ZG_REQUIRE(lr_t != nullptr && t >= 1, "adam_lr_t: null output or t < 1");
    *lr_t = adam_lr_t(lr, beta1, beta2, t);
    return ZG_HIP_OK;
}

ZG_API int zg_hip_adam_step_at(zg_hip_ctx* ctx, float* param, float* grad, float* m, float* v, size_t n,
                               const float* lr_t, float beta1, float beta2, float epsilon, int clip, float max_norm,
                               float delta) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(param && grad && m && v && lr_t, "adam_step_at: null pointer");
    return step_entry(ctx, 2, param, grad, m, v, n, 0.f, 0.f, lr_t, beta1, beta2, epsilon, clip, max_norm, delta);
}

// Parameter lists (the tensors are independent, so the launches need not follow the list order; a tensor listed
// twice is the exception and is handled below): the clip factors of all tensors of a batch come from two launches (the
// first stage of the two-stage norm of every tensor beyond kFlatSingleMax, with the blocks and the combine tree of the
// per-tensor path, then one workgroup per tensor), tensors of up to kMultiBigMax elements share the update launch, and
// larger ones take the per-tensor update kernels with their 16-byte grid-stride walks.
static int step_multi(zg_hip_ctx* ctx, const char* name, bool adam, size_t n_tensors, float* const* params,
                      float* const* grads, float* const* ms, float* const* vs, const size_t* lens, const float* lr_t,
                      int lr_t_in_memory, float lr, float beta1, float beta2, float epsilon, int clip, float max_norm,
                      float delta, int zero_grads) {
    ZG_REQUIRE(n_tensors == 0 || (params && grads && lens), "%s: null list", name);
    ZG_REQUIRE(!adam || n_tensors == 0 || (ms && vs && lr_t), "%s: null list", name);
    MultiArgs a;
    int filled = 0;
    size_t partials_used = 0;  // floats of the context's partials buffer handed to this batch
    const size_t partials_room = ((size_t)64 << 10) / sizeof(float);
    // One batch: the first stage of the norms of its larger tensors (one launch), every tensor's clip factor (one
    // launch), the update of the tensors of up to kMultiBigMax elements in slices (one launch), and the update of
    // each larger tensor by the per-tensor kernel, which reads its factor from the batch's slot.
    auto flush = [&]() -> int {
        if (!filled) return ZG_HIP_OK;
        a.count = filled;
        if (clip) {
            if (a.part_first[filled] > 0) {
                hipLaunchKernelGGL(norm_partials_multi_kernel, dim3((unsigned)a.part_first[filled]), dim3(kFlatBlock), 0,
                                   ctx->stream, a);
                ZG_LAUNCH_CHECK();
            }
            hipLaunchKernelGGL(norm_multi_kernel, dim3(filled), dim3(kFlatSingle), 0, ctx->stream, a);
            ZG_LAUNCH_CHECK();
        }
        const unsigned grid = (unsigned)a.wg_first[filled];
        if (grid) {
            if (adam) hipLaunchKernelGGL((update_multi_kernel<true>), dim3(grid), dim3(kMultiThreads), 0, ctx->stream, a);
            else hipLaunchKernelGGL((update_multi_kernel<false>), dim3(grid), dim3(kMultiThreads), 0, ctx->stream, a);
            ZG_LAUNCH_CHECK();
        }
        for (int b = 0; b < filled; b++) {
            const size_t n = a.n[b];
            if (n <= kMultiBigMax) continue;
            const float* factor = a.factors + b;
            const dim3 g(update_grid(ctx, n)), t(kBlock);
            if (adam) {
                if (clip)
                    hipLaunchKernelGGL((adam_kernel<true>), g, t, 0, ctx->stream, a.p[b], a.g[b], a.m[b], a.v[b], n, a.lr_t[b],
                                       a.lr_t_mem[b], a.b1, a.b2, a.omb1, a.omb2, a.eps, factor, zero_grads != 0);
                else
                    hipLaunchKernelGGL((adam_kernel<false>), g, t, 0, ctx->stream, a.p[b], a.g[b], a.m[b], a.v[b], n, a.lr_t[b],
                                       a.lr_t_mem[b], a.b1, a.b2, a.omb1, a.omb2, a.eps, factor, zero_grads != 0);
            } else {
                if (clip)
                    hipLaunchKernelGGL((sgd_kernel<true>), g, t, 0, ctx->stream, a.p[b], a.g[b], n, a.lr_t[b], factor,
                                       zero_grads != 0);
                else
                    hipLaunchKernelGGL((sgd_kernel<false>), g, t, 0, ctx->stream, a.p[b], a.g[b], n, a.lr_t[b], factor,
                                       zero_grads != 0);
            }
            ZG_LAUNCH_CHECK();
        }
        filled = 0;
        partials_used = 0;
        return ZG_HIP_OK;
    };
    a.b1 = beta1;
    a.b2 = beta2;
    a.omb1 = 1.0f - beta1;
    a.omb2 = 1.0f - beta2;
    a.eps = epsilon;
    a.max_norm = max_norm;
    a.delta = delta;
    a.clip = clip;
    a.zero_grads = zero_grads;
    a.factors = ctx->scalar_slot + 16;  // kMultiMax floats of the context's 64
    a.wg_first[0] = 0;
    a.part_first[0] = 0;
    for (size_t i = 0; i < n_tensors; i++) {
        const size_t n = lens[i];
        if (n == 0) continue;
        ZG_REQUIRE(params[i] && grads[i] && (!adam || (ms[i] && vs[i])), "%s: null pointer in tensor %zu", name, i);
        // a tensor that is listed twice is updated twice, in list order: the second update waits for the first
        bool listed = false;
        for (int b = 0; b < filled; b++) listed = listed || a.p[b] == params[i] || a.g[b] == grads[i];
        const size_t parts = (clip && n > kFlatSingleMax) ? flat_partial_blocks(ctx, n) : 0;
        if (listed || partials_used + parts > partials_room)
            if (int rc = flush()) return rc;
        a.p[filled] = params[i];
        a.g[filled] = grads[i];
        a.m[filled] = adam ? ms[i] : nullptr;
        a.v[filled] = adam ? vs[i] : nullptr;
        a.n[filled] = n;
        a.lr_t[filled] = adam ? (lr_t_in_memory ? 0.f : lr_t[i]) : -lr;
        a.lr_t_mem[filled] = (adam && lr_t_in_memory) ? lr_t + i : nullptr;
        a.partials[filled] = parts ? (float*)ctx->partials + partials_used : nullptr;
        a.n_partials[filled] = (int)parts;
        a.part_first[filled + 1] = a.part_first[filled] + (int)parts;
        partials_used += parts;
        // tensors beyond kMultiBigMax keep the per-tensor update kernels (16-byte grid-stride walks): no slices
        a.wg_first[filled + 1] = a.wg_first[filled] + (n <= kMultiBigMax ? (int)ceil_div_sz(n, kMultiSlice) : 0);
        if (++filled == kMultiMax)
            if (int rc = flush()) return rc;
    }
    return flush();
}

ZG_API int zg_hip_sgd_step_multi(zg_hip_ctx* ctx, size_t n_tensors, float* const* params, float* const* grads,
                                 const size_t* lens, float lr, int clip, float max_norm, float delta, int zero_grads) {
    ZG_CTX(ctx);
    return step_multi(ctx, "sgd_step_multi", false, n_tensors, params, grads, nullptr, nullptr, lens, nullptr, 0, lr, 0.f,
                      0.f, 0.f, clip, max_norm, delta, zero_grads);
}

ZG_API int zg_hip_adam_step_multi(zg_hip_ctx* ctx, size_t n_tensors, float* const* params, float* const* grads,
                                  float* const* ms, float* const* vs, const size_t* lens, const float* lr_t,
                                  int lr_t_in_memory, float beta1, float beta2, float epsilon, int clip, float max_norm,
                                  float delta, int zero_grads) {
    ZG_CTX(ctx);
    return step_multi(ctx, "adam_step_multi", true, n_tensors, params, grads, ms, vs, lens, lr_t, lr_t_in_memory, 0.f,
                      beta1, beta2, epsilon, clip, max_norm, delta, zero_grads);
}
