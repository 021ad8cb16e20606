// Elementwise binary (broadcasting) and unary forward/backward ops.
//
// All of these are HBM-bound streams.  The kernels move 128 bits per lane per access, keep four
// independent accesses in flight per thread and never re-read an operand; the broadcasting form
// holds the short operand in registers while it walks down the rows of the long one.
// Arithmetic is kept as separate fp32 multiplies and adds (no contraction) so each element rounds
// exactly like the host loop it replaces.
#include "reduce_device.h"

namespace zg {

// ------------------------------------------------------------------------------------------------
// generic map kernel: out[i] = Op::f(a[i], b[i], c[i], p0, p1)
// ------------------------------------------------------------------------------------------------
constexpr int kUnroll = 4;

template <class Op, int NIN>
__global__ __launch_bounds__(kBlock) void map_vec4_kernel(float* out, const float* a, const float* b,
                                                           const float* c, size_t n, float p0, float p1) {
    const size_t n4 = n >> 2;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* b4 = reinterpret_cast<const float4*>(b);
    const float4* c4 = reinterpret_cast<const float4*>(c);
    float4* o4 = reinterpret_cast<float4*>(out);
    size_t base = (size_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * (kBlock * kUnroll);
    // Three or more streams run at 71-76 % of HBM bandwidth through the caches and at 83-88 % with the non-temporal
    // hint on what is touched once (measured on [8192,4096]: mul 70.6 -> 60.5 us, relu_bwd 88.5 -> 76.3 us).  An operand
    // that is also the output keeps plain accesses (its line is written right after it is read), and an in-place op of
    // two streams is fastest with plain accesses throughout (56.8 us against 58.6).
    const bool aliased = out == a || (NIN > 1 && out == b) || (NIN > 2 && out == c);
    const bool nt = NIN > 1 && !(NIN == 2 && aliased);  // (one input, one output: 39.3 us plain, 42.0 us with the hint)
    for (; base < n4; base += stride) {
        float4 va[kUnroll], vb[kUnroll], vc[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            size_t i = base + (size_t)u * kBlock;
            if (i < n4) {
                va[u] = (nt && a != out) ? nt_load(a4 + i) : a4[i];
                if (NIN > 1) vb[u] = (nt && b != out) ? nt_load(b4 + i) : b4[i];
                if (NIN > 2) vc[u] = (nt && c != out) ? nt_load(c4 + i) : c4[i];
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            size_t i = base + (size_t)u * kBlock;
            if (i < n4) {
                float4 r;
                r.x = Op::f(va[u].x, NIN > 1 ? vb[u].x : 0.f, NIN > 2 ? vc[u].x : 0.f, p0, p1);
                r.y = Op::f(va[u].y, NIN > 1 ? vb[u].y : 0.f, NIN > 2 ? vc[u].y : 0.f, p0, p1);
                r.z = Op::f(va[u].z, NIN > 1 ? vb[u].z : 0.f, NIN > 2 ? vc[u].z : 0.f, p0, p1);
                r.w = Op::f(va[u].w, NIN > 1 ? vb[u].w : 0.f, NIN > 2 ? vc[u].w : 0.f, p0, p1);
                if (nt && !aliased) nt_store(r, o4 + i);
                else o4[i] = r;
            }
        }
    }
    // tail (n % 4 elements), handled by the first threads of block 0
    const size_t tail0 = n4 << 2;
    if (blockIdx.x == 0) {
        size_t i = tail0 + threadIdx.x;
        if (i < n) out[i] = Op::f(a[i], NIN > 1 ? b[i] : 0.f, NIN > 2 ? c[i] : 0.f, p0, p1);
    }
}

template <class Op, int NIN>
__global__ __launch_bounds__(kBlock) void map_scalar_kernel(float* out, const float* a, const float* b,
                                                             const float* c, size_t n, float p0, float p1) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (; i < n; i += stride) out[i] = Op::f(a[i], NIN > 1 ? b[i] : 0.f, NIN > 2 ? c[i] : 0.f, p0, p1);
}

static int map_grid(zg_hip_ctx* ctx, size_t items, int per_block) {
    size_t blocks = ceil_div_sz(items, (size_t)per_block);
    // one trip per thread at any size (a capped grid whose threads stride through the array is 2 to 5 % slower beyond
    // 33 M elements)
    (void)ctx;
    size_t cap = 0x7fffffffull;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

// Waiting elementwise ops (see zg_waiting_maps): chain_code<Op>() is the op's number in the one-launch kernel, -1 for
// an op that always takes its own launch; chain_push queues an op, sending the waiting ones out first when it cannot
// join them; false: the caller launches the op itself (after flush_maps).
template <class Op> constexpr int chain_code() { return -1; }
static bool chain_push(zg_hip_ctx* ctx, int code, int nin, int scalar, float* out, const float* a, const float* b,
                       const float* c, size_t n, float p0, float p1, int* rc);
// An elementwise op that takes its own launch: the waiting elementwise ops go out first, and the waiting fills too when
// one of them meets an operand (lengths in floats; null operands are skipped).
static int settle_before_launch(zg_hip_ctx* ctx, const float* out, size_t n_out, const float* a, size_t n_a,
                                const float* b, size_t n_b, const float* c, size_t n_c) {
    if (int rc = flush_kinds(ctx, kWaitMaps)) return rc;
    const ByteSpan spans[4] = {{out, n_out * sizeof(float)}, {a, n_a * sizeof(float)}, {b, n_b * sizeof(float)},
                               {c, n_c * sizeof(float)}};
    return flush_touching(ctx, kWaitFills, spans, 4);
}

template <class Op, int NIN>
static int launch_map(zg_hip_ctx* ctx, float* out, const float* a, const float* b, const float* c, size_t n,
                      float p0 = 0.f, float p1 = 0.f) {
    if (n == 0) return ZG_HIP_OK;
    {
        int rc = ZG_HIP_OK;
        if (chain_code<Op>() >= 0 && chain_push(ctx, chain_code<Op>(), NIN, 0, out, a, b, c, n, p0, p1, &rc)) return rc;
        if (rc) return rc;
        if ((rc = settle_before_launch(ctx, out, n, a, n, NIN > 1 ? b : nullptr, n, NIN > 2 ? c : nullptr, n))) return rc;
    }
    bool vec = aligned16(out) && aligned16(a) && (NIN < 2 || aligned16(b)) && (NIN < 3 || aligned16(c)) && n >= 4;
    if (vec) {
        int grid = map_grid(ctx, n >> 2, kBlock * kUnroll);
        hipLaunchKernelGGL((map_vec4_kernel<Op, NIN>), dim3(grid), dim3(kBlock), 0, ctx->stream, out, a, b, c, n, p0,
                           p1);
    } else {
        int grid = map_grid(ctx, n, kBlock);
        hipLaunchKernelGGL((map_scalar_kernel<Op, NIN>), dim3(grid), dim3(kBlock), 0, ctx->stream, out, a, b, c, n, p0,
                           p1);
    }
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// binary ops with the reference's broadcasting regimes
// ------------------------------------------------------------------------------------------------
struct AddOp { static __device__ __forceinline__ float f(float a, float b) { return __fadd_rn(a, b); } };
struct SubOp { static __device__ __forceinline__ float f(float a, float b) { return __fsub_rn(a, b); } };
struct MulOp { static __device__ __forceinline__ float f(float a, float b) { return __fmul_rn(a, b); } };
struct DivOp { static __device__ __forceinline__ float f(float a, float b) { return __fdiv_rn(a, b); } };

// adapters to the map kernel
template <class B> struct Bin2 { static __device__ __forceinline__ float f(float a, float b, float, float, float) { return B::f(a, b); } };
// scalar operand broadcast from device memory: p is read once per thread
template <class B, bool SCALAR_LHS>
__global__ __launch_bounds__(kBlock) void bin_scalar_kernel(float* out, const float* vec, const float* scalar,
                                                             size_t n) {
    const float s = scalar[0];
    const bool v4ok = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(vec)) & 15u) == 0;
    if (v4ok) {
        const size_t n4 = n >> 2;
        const float4* v4 = reinterpret_cast<const float4*>(vec);
        float4* o4 = reinterpret_cast<float4*>(out);
        size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
        const size_t stride = (size_t)gridDim.x * kBlock;
        for (; i < n4; i += stride) {
            float4 v = v4[i], r;
            r.x = SCALAR_LHS ? B::f(s, v.x) : B::f(v.x, s);
            r.y = SCALAR_LHS ? B::f(s, v.y) : B::f(v.y, s);
            r.z = SCALAR_LHS ? B::f(s, v.z) : B::f(v.z, s);
            r.w = SCALAR_LHS ? B::f(s, v.w) : B::f(v.w, s);
            o4[i] = r;
        }
        if (blockIdx.x == 0) {
            size_t t = (n4 << 2) + threadIdx.x;
            if (t < n) out[t] = SCALAR_LHS ? B::f(s, vec[t]) : B::f(vec[t], s);
        }
    } else {
        size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
        const size_t stride = (size_t)gridDim.x * kBlock;
        for (; i < n; i += stride) out[i] = SCALAR_LHS ? B::f(s, vec[i]) : B::f(vec[i], s);
    }
}

// Row broadcast: `lng` is [rows, period], `sht` is [period]; period % 4 == 0, all 16-byte aligned.
// Thread (tx, ty): tx walks float4 columns, ty walks rows; the short operand stays in registers.
constexpr int kRbX = 64, kRbY = 4, kRbRows = 4;
template <class B, bool SHORT_LHS>
__global__ __launch_bounds__(kRbX * kRbY) void bin_rowbcast_kernel(float* out, const float* lng, const float* sht,
                                                                    size_t rows, size_t p4) {
    const size_t col = (size_t)blockIdx.x * kRbX + threadIdx.x;
    if (col >= p4) return;
    const float4 s = reinterpret_cast<const float4*>(sht)[col];
    const float4* l4 = reinterpret_cast<const float4*>(lng);
    float4* o4 = reinterpret_cast<float4*>(out);
    const size_t row_step = (size_t)gridDim.y * kRbY;
    // each thread handles kRbRows rows per trip: rows r, r+row_step, ...
    size_t r = (size_t)blockIdx.y * kRbY + threadIdx.y;
    for (; r < rows; r += row_step * kRbRows) {
        float4 v[kRbRows];
#pragma unroll
        for (int u = 0; u < kRbRows; u++) {
            size_t rr = r + (size_t)u * row_step;
            if (rr < rows) v[u] = l4[rr * p4 + col];
        }
#pragma unroll
        for (int u = 0; u < kRbRows; u++) {
            size_t rr = r + (size_t)u * row_step;
            if (rr < rows) {
                float4 q;
                q.x = SHORT_LHS ? B::f(s.x, v[u].x) : B::f(v[u].x, s.x);
                q.y = SHORT_LHS ? B::f(s.y, v[u].y) : B::f(v[u].y, s.y);
                q.z = SHORT_LHS ? B::f(s.z, v[u].z) : B::f(v[u].z, s.z);
                q.w = SHORT_LHS ? B::f(s.w, v[u].w) : B::f(v[u].w, s.w);
                o4[rr * p4 + col] = q;
            }
        }
    }
}

// Fallback for any period/alignment: z[i] = x[i % xl] o y[i % yl] (one of the two is the identity map)
template <class B>
__global__ __launch_bounds__(kBlock) void bin_modulo_kernel(float* out, const float* x, size_t xl, const float* y,
                                                             size_t yl, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (; i < n; i += stride) {
        size_t xi = (xl == n) ? i : i % xl;
        size_t yi = (yl == n) ? i : i % yl;
        out[i] = B::f(x[xi], y[yi]);
    }
}

// The same for a long operand and a result on 16-byte boundaries, whatever the period: the long operand is walked as one
// flat array of 16-byte pieces, four per thread in flight; a workgroup divides once (where its chunk starts in the short
// operand), a piece finds its place from there and its four values step through the short operand, wrapping at its
// end.  ([8192, 32001] + [32001]: 701 us with a 64-bit remainder per value, 37 % of 8 TB/s.)
constexpr int kPeriodU = 4;
template <class B, bool SHORT_LHS>
struct BinPeriod {
    __device__ __forceinline__ float operator()(float l, float s) const { return SHORT_LHS ? B::f(s, l) : B::f(l, s); }
};
struct AxpbyPeriod {  // the broadcast op: alpha * short + beta * long
    float alpha, beta;
    __device__ __forceinline__ float operator()(float l, float s) const {
        return __fadd_rn(__fmul_rn(alpha, s), __fmul_rn(beta, l));
    }
};
template <class F>
__global__ __launch_bounds__(kBlock) void bin_period_kernel(F f, float* out, const float* lng, const float* sht, size_t n,
                                                             size_t p) {
    constexpr size_t kChunk = (size_t)kBlock * kPeriodU;
    const float4* l4 = reinterpret_cast<const float4*>(lng);
    float4* o4 = reinterpret_cast<float4*>(out);
    const size_t n4 = n >> 2;
    for (size_t c0 = (size_t)blockIdx.x * kChunk; c0 < n4; c0 += (size_t)gridDim.x * kChunk) {
        const size_t e0 = c0 << 2, cq = e0 / p, cs = e0 - cq * p;
        float4 v[kPeriodU];
        float sv[kPeriodU][4];
#pragma unroll
        for (int u = 0; u < kPeriodU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            if (j < n4) {
                v[u] = nt_load(l4 + j);
                size_t q, s;
                flat_divmod(0, cs, 4 * (threadIdx.x + (size_t)u * kBlock), p, q, s);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    sv[u][k] = sht[s];
                    if (++s == p) s = 0;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kPeriodU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            if (j < n4) {
                float4 o;
                o.x = f(v[u].x, sv[u][0]);
                o.y = f(v[u].y, sv[u][1]);
                o.z = f(v[u].z, sv[u][2]);
                o.w = f(v[u].w, sv[u][3]);
                nt_store(o, o4 + j);
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t i = (n4 << 2) + threadIdx.x;
        out[i] = f(lng[i], sht[i % p]);
    }
}

__global__ void broadcast_modulo_kernel(float* y, const float* x, size_t xl, size_t yl, float alpha, float beta) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < yl; i += stride) y[i] = __fadd_rn(__fmul_rn(alpha, x[i % xl]), __fmul_rn(beta, y[i]));
}

template <class B>
static int binary_op(zg_hip_ctx* ctx, const char* name, const float* x, size_t xl, const float* y, size_t yl, float* z,
                     size_t zl) {
    ZG_ENTER(ctx, kWaitMaps | kWaitFills);
    // An empty result from empty or one-element operands is what the host's loops make of it: nothing
    // (src/device/host_device.zig:975-1019: equal lengths, or a scalar against an empty slice).  An empty operand
    // against a longer one never ends there and is refused here.
    if (zl == 0 && xl <= 1 && yl <= 1 && xl + yl < 2) return ZG_HIP_OK;
    ZG_REQUIRE(xl > 0 && yl > 0 && zl > 0, "%s: empty operand", name);
    ZG_REQUIRE(x && y && z, "%s: null pointer", name);
    const size_t mx = xl > yl ? xl : yl, mn = xl < yl ? xl : yl;
    // src/device/opspec.zig:1-11: the longer length is a multiple of the shorter and z has the longer length
    ZG_REQUIRE(mx % mn == 0, "%s: lengths %zu and %zu do not broadcast", name, xl, yl);
    ZG_REQUIRE(zl == mx, "%s: z.len %zu != max(x.len, y.len) %zu", name, zl, mx);

    if (xl == yl) return launch_map<Bin2<B>, 2>(ctx, z, x, y, nullptr, zl);
    if (mn == 1) {
        {
            int rc = ZG_HIP_OK;
            if (chain_push(ctx, chain_code<Bin2<B>>(), 2, xl == 1 ? 2 : 1, z, x, y, nullptr, zl, 0.f, 0.f, &rc)) return rc;
            if (rc) return rc;
        }
        if (int rc = settle_before_launch(ctx, z, zl, x, xl, y, yl, nullptr, 0)) return rc;
        int grid = map_grid(ctx, (zl + 3) / 4, kBlock);
        if (xl == 1)
            hipLaunchKernelGGL((bin_scalar_kernel<B, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, z, y, x, zl);
        else
            hipLaunchKernelGGL((bin_scalar_kernel<B, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, z, x, y, zl);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (int rc = settle_before_launch(ctx, z, zl, x, xl, y, yl, nullptr, 0)) return rc;
    const bool short_lhs = xl < yl;
    const float* lng = short_lhs ? y : x;
    const float* sht = short_lhs ? x : y;
    // rows of whole 16-byte pieces: a workgroup per group of rows keeps its pieces of the short operand in registers.  Not
    // for rows of fewer than 64 values (a workgroup then has a few lanes at work: [1048576, 4 ... 32] took 66 us
    // whatever the row length, 6 to 47 us as a flat walk) nor from 256 MiB up, where the flat walk is 4 to 14 % faster
    if (mn % 4 == 0 && mn >= 64 && zl < ((size_t)1 << 26) && aligned16(lng) && aligned16(sht) && aligned16(z)) {
        size_t p4 = mn / 4, rows = mx / mn;
        unsigned gx = (unsigned)ceil_div_sz(p4, kRbX);
        // a workgroup per group of rows, up to the grid's limit (65536 rows of 4096: 466 -> 370 us against 16 workgroups
        // per compute unit whose threads loop over the rest)
        size_t gy = ceil_div_sz(rows, (size_t)kRbY * kRbRows);
        if (gy < 1) gy = 1;
        if (gy > 65535) gy = 65535;
        dim3 grid(gx, (unsigned)gy), block(kRbX, kRbY);
        if (short_lhs)
            hipLaunchKernelGGL((bin_rowbcast_kernel<B, true>), grid, block, 0, ctx->stream, z, lng, sht, rows, p4);
        else
            hipLaunchKernelGGL((bin_rowbcast_kernel<B, false>), grid, block, 0, ctx->stream, z, lng, sht, rows, p4);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (aligned16(lng) && aligned16(z) && zl >= 4) {
        int grid = map_grid(ctx, zl >> 2, kBlock * kPeriodU);
        if (short_lhs)
            hipLaunchKernelGGL((bin_period_kernel<BinPeriod<B, true>>), dim3(grid), dim3(kBlock), 0, ctx->stream,
                               BinPeriod<B, true>{}, z, lng, sht, zl, mn);
        else
            hipLaunchKernelGGL((bin_period_kernel<BinPeriod<B, false>>), dim3(grid), dim3(kBlock), 0, ctx->stream,
                               BinPeriod<B, false>{}, z, lng, sht, zl, mn);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    int grid = map_grid(ctx, zl, kBlock);
    hipLaunchKernelGGL((bin_modulo_kernel<B>), dim3(grid), dim3(kBlock), 0, ctx->stream, z, x, xl, y, yl, zl);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// unary forward/backward functors.  Argument order of f() is the order the launcher passes arrays.
// ------------------------------------------------------------------------------------------------
#define ZG_OP(NAME, BODY)                                                                        \
    struct NAME {                                                                                \
        static __device__ __forceinline__ float f(float a, float b, float c, float p0, float p1) { \
            (void)a; (void)b; (void)c; (void)p0; (void)p1;                                       \
            BODY                                                                                 \
        }                                                                                        \
    };

// forward ops: a = x
ZG_OP(PowFwd, return powf(a, p0);)
ZG_OP(SqrtFwd, return sqrtf(a);)
ZG_OP(RsqrtFwd, return __fdiv_rn(1.0f, sqrtf(fmaxf(a, p0)));)
ZG_OP(ExpFwd, return expf(a);)
ZG_OP(ReluFwd, return a > 0.f ? a : 0.f;)
ZG_OP(TanhFwd, return tanhf(a);)
ZG_OP(SigmFwd, return __fdiv_rn(1.0f, __fadd_rn(1.0f, expf(-a)));)
ZG_OP(ClampFwd, return fminf(p1, fmaxf(p0, a));)
// backward ops: a = x (or y), b = x_g (accumulated into), c = y_g
ZG_OP(PowBwd, if (a < p1) return __fadd_rn(b, 0.0f);
      return __fadd_rn(b, __fmul_rn(__fmul_rn(p0, powf(a, __fsub_rn(p0, 1.0f))), c));)
ZG_OP(SqrtBwd, if (a < p0) return __fadd_rn(b, 0.0f);
      return __fadd_rn(b, __fmul_rn(__fdiv_rn(0.5f, sqrtf(a)), c));)
ZG_OP(RsqrtBwd, if (a < p0) return __fadd_rn(b, 0.0f);
      float s = sqrtf(a); float inv = __fdiv_rn(1.0f, __fmul_rn(a, s));
      return __fadd_rn(b, __fmul_rn(__fmul_rn(-0.5f, inv), c));)
// exp_bwd: a = y, b = x_g, c = y_g
ZG_OP(ExpBwd, return __fadd_rn(b, __fmul_rn(a, c));)
ZG_OP(ReluBwd, return __fadd_rn(b, (a > 0.f) ? c : 0.f);)
// relu_inplace_bwd: a = x, b = x_g
ZG_OP(ReluInplaceBwd, return (a <= 0.f) ? 0.f : b;)
// tanh_bwd: a = y, b = x_g, c = y_g
ZG_OP(TanhBwd, return __fadd_rn(b, __fmul_rn(__fsub_rn(1.0f, __fmul_rn(a, a)), c));)
ZG_OP(TanhInplaceBwd, return __fmul_rn(b, __fsub_rn(1.0f, __fmul_rn(a, a)));)
ZG_OP(SigmBwd, return __fadd_rn(b, __fmul_rn(__fmul_rn(a, __fsub_rn(1.0f, a)), c));)
ZG_OP(SigmInplaceBwd, return __fmul_rn(b, __fmul_rn(a, __fsub_rn(1.0f, a)));)
ZG_OP(ClampBwd, return (p0 < a && a < p1) ? __fadd_rn(b, c) : b;)
// scale: a = x
ZG_OP(ScaleOp, return __fmul_rn(a, p0);)
// broadcast / scaled copy: a = x, b = y -> alpha*x + beta*y
ZG_OP(ScaledCopy, return __fadd_rn(__fmul_rn(p0, a), __fmul_rn(p1, b));)
ZG_OP(ScaledCopyNoRead, return __fmul_rn(p0, a);)
// binary ops with one operand passed by value: a = the array's element, p0 = the scalar; R: x o s, L: s o x
ZG_OP(AddScalarR, return __fadd_rn(a, p0);)
ZG_OP(AddScalarL, return __fadd_rn(p0, a);)
ZG_OP(SubScalarR, return __fsub_rn(a, p0);)
ZG_OP(SubScalarL, return __fsub_rn(p0, a);)
ZG_OP(MulScalarR, return __fmul_rn(a, p0);)
ZG_OP(MulScalarL, return __fmul_rn(p0, a);)
ZG_OP(DivScalarR, return __fdiv_rn(a, p0);)
ZG_OP(DivScalarL, return __fdiv_rn(p0, a);)
// smooth-l1 / mse backward: a = pred, b = target, c = grad; p0 = beta or scale, p1 = n
ZG_OP(SmoothL1Bwd, return __fadd_rn(c, smooth_l1_grad(a, b, p0, p1));)
ZG_OP(MseBwd, return __fadd_rn(c, __fmul_rn(p0, __fsub_rn(a, b)));)

// ------------------------------------------------------------------------------------------------
// waiting elementwise ops: one launch for a run of small ops of one length
// ------------------------------------------------------------------------------------------------
#define ZG_CHAIN_OPS(X)                                                                                              \
    X(0, Bin2<AddOp>) X(1, Bin2<SubOp>) X(2, Bin2<MulOp>) X(3, Bin2<DivOp>) X(4, PowFwd) X(5, SqrtFwd) X(6, RsqrtFwd) \
    X(7, ExpFwd) X(8, ReluFwd) X(9, TanhFwd) X(10, SigmFwd) X(11, ClampFwd) X(12, PowBwd) X(13, SqrtBwd)             \
    X(14, RsqrtBwd) X(15, ExpBwd) X(16, ReluBwd) X(17, ReluInplaceBwd) X(18, TanhBwd) X(19, TanhInplaceBwd)          \
    X(20, SigmBwd) X(21, SigmInplaceBwd) X(22, ClampBwd) X(23, ScaleOp) X(24, SmoothL1Bwd) X(25, MseBwd)          \
    X(27, AddScalarR) X(28, AddScalarL) X(29, SubScalarR) X(30, SubScalarL) X(31, MulScalarR) X(32, MulScalarL)      \
    X(33, DivScalarR) X(34, DivScalarL)
#define ZG_CHAIN_CODE(N, OP) template <> constexpr int chain_code<OP>() { return N; }
ZG_CHAIN_OPS(ZG_CHAIN_CODE)
#undef ZG_CHAIN_CODE

constexpr int kChainCountCode = 26;  // out[i] = p0 added (a[i + 1] - a[i]) times, a an array of uint32 bucket bounds
struct MapChainArgs {
    zg_map_op op[kMaxWaitingMaps];
    int count;
    size_t n;
};
// Thread i carries element i through the ops in call order: each op loads its operands from memory and stores its
// result, so an op that reads what an earlier one wrote (always at the same index: the queue admits nothing else) gets
// it from its own store.  The arithmetic is each op's functor, as in its own kernel.
__global__ __launch_bounds__(kBlock) void map_chain_kernel(MapChainArgs g) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= g.n) return;
    for (int k = 0; k < g.count; k++) {
        const zg_map_op& o = g.op[k];
        if (o.code == kChainCountCode) {
            const uint32_t* bounds = reinterpret_cast<const uint32_t*>(o.a);
            const uint32_t cnt = bounds[i + 1] - bounds[i];
            float r = 0.f;
            for (uint32_t e = 0; e < cnt; e++) r = __fadd_rn(r, o.p0);
            o.out[i] = r;
            continue;
        }
        const float a = (o.subst & 1) ? o.subst_value : o.a[o.scalar == 2 ? 0 : i];
        const float b = o.nin > 1 ? ((o.subst & 2) ? o.subst_value : o.b[o.scalar == 1 ? 0 : i]) : 0.f;
        const float c = o.nin > 2 ? ((o.subst & 4) ? o.subst_value : o.c[i]) : 0.f;
        float r = 0.f;
        switch (o.code) {
#define ZG_CHAIN_CASE(N, OP) case N: r = OP::f(a, b, c, o.p0, o.p1); break;
            ZG_CHAIN_OPS(ZG_CHAIN_CASE)
#undef ZG_CHAIN_CASE
        }
        o.out[i] = r;
    }
}

int flush_maps(zg_hip_ctx* ctx) {
    zg_waiting_maps& q = ctx->maps;
    if (q.count == 0) return ZG_HIP_OK;
    MapChainArgs g;
    for (int k = 0; k < q.count; k++) g.op[k] = q.op[k];
    g.count = q.count;
    g.n = q.n;
    q.count = 0;
    hipLaunchKernelGGL(map_chain_kernel, dim3((unsigned)ceil_div_sz(g.n, kBlock)), dim3(kBlock), 0, ctx->stream, g);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// Two accesses of which one writes may share a launch when they cannot meet, or when they are the same n elements (then
// thread i alone touches element i of both, in call order).  A one-float operand is read by every thread, so nothing in
// the run may write it.
struct MapRange {
    const char* lo;
    const char* hi;
    bool per_element;
};
static bool map_ranges_conflict(const MapRange& w, const MapRange& o) {
    if (!(w.lo < o.hi && o.lo < w.hi)) return false;
    return !(w.per_element && o.per_element && w.lo == o.lo && w.hi == o.hi);
}
static int map_op_ranges(const zg_map_op& o, size_t n, MapRange* r) {  // r[0] is the output
    int m = 0;
    auto put = [&](const float* p, bool scalar) {
        r[m++] = MapRange{(const char*)p, (const char*)(p + (scalar ? 1 : n)), !scalar};
    };
    put(o.out, false);
    if (o.code == kChainCountCode) {  // n + 1 bucket bounds, read by neighbouring threads: nothing in the run may write them
        r[m++] = MapRange{(const char*)o.a, (const char*)o.a + (n + 1) * sizeof(uint32_t), false};
        return m;
    }
    put(o.a, o.scalar == 2);
    if (o.nin > 1) put(o.b, o.scalar == 1);
    if (o.nin > 2) put(o.c, false);
    return m;
}

bool maps_touch(const zg_hip_ctx* ctx, const char* lo, const char* hi) {
    const zg_waiting_maps& q = ctx->maps;
    for (int k = 0; k < q.count; k++) {
        MapRange r[4];
        const int m = map_op_ranges(q.op[k], q.n, r);
        for (int j = 0; j < m; j++)
            if (r[j].lo < hi && lo < r[j].hi) return true;
    }
    return false;
}

static bool chain_push(zg_hip_ctx* ctx, int code, int nin, int scalar, float* out, const float* a, const float* b,
                       const float* c, size_t n, float p0, float p1, int* rc) {
    *rc = ZG_HIP_OK;
    if (code < 0 || n == 0 || n > kWaitingMapMaxLen) return false;
    zg_map_op o{code, nin, scalar, 0, 0.f, out, a, b, c, p0, p1};
    MapRange mine[4];
    int n_mine = map_op_ranges(o, n, mine);
    // the op's own operands: in place is fine, a shifted overlap is not (its own kernel would race too: let it)
    for (int j = 1; j < n_mine; j++)
        if (map_ranges_conflict(mine[0], mine[j])) return false;
    // From here on the op is queued.  A fill of exactly its output that is still waiting has no other reader: the op
    // overwrites all of it, and where the output is also an operand (x_g += ..., in place) it takes the fill's value
    // instead of loading it (ensure_grad(0) followed by an accumulating backward, src/ndtensor.zig:221-228).  Other
    // fills that meet an operand go out first; the rest keep waiting.
    if (ctx->n_pending_fills) {
        float value = 0.f;
        if (take_fill_exact(ctx, out, n, &value)) {
            o.subst_value = value;
            if (scalar != 2 && a == out) o.subst |= 1;
            if (nin > 1 && scalar != 1 && b == out) o.subst |= 2;
            if (nin > 2 && c == out) o.subst |= 4;
        }
        const void* ptrs[4];
        size_t bytes[4];
        for (int j = 0; j < n_mine; j++) {
            ptrs[j] = mine[j].lo;
            bytes[j] = (size_t)(mine[j].hi - mine[j].lo);
        }
        if (fills_touch(ctx, ptrs, bytes, n_mine))
            if ((*rc = flush_fills(ctx))) return false;
    }
    zg_waiting_maps& q = ctx->maps;
    bool joins = q.count > 0 && q.count < kMaxWaitingMaps && q.n == n;
    for (int k = 0; k < q.count && joins; k++) {
        MapRange theirs[4];
        const int n_theirs = map_op_ranges(q.op[k], q.n, theirs);
        for (int j = 0; j < n_mine && joins; j++) joins = !map_ranges_conflict(theirs[0], mine[j]);   // they write
        for (int j = 1; j < n_theirs && joins; j++) joins = !map_ranges_conflict(mine[0], theirs[j]);  // I write
    }
    if (q.count > 0 && !joins)
        if ((*rc = flush_maps(ctx))) return false;
    if (q.count == 0) q.n = n;
    q.op[q.count++] = o;
    return true;
}

bool maps_push_count(zg_hip_ctx* ctx, float* out, const uint32_t* row_ptr, size_t n, float c, int* rc) {
    return chain_push(ctx, kChainCountCode, 1, 0, out, reinterpret_cast<const float*>(row_ptr), nullptr, nullptr, n, c, 0.f,
                      rc);
}

}  // namespace zg

using namespace zg;

#define ZG_CHECK_N(name, n, ...)                                         \
    ZG_ENTER(ctx, kWaitMaps | kWaitFills);                                               \
    if ((n) == 0) return ZG_HIP_OK;                                      \
    {                                                                    \
        const void* _ptrs[] = {__VA_ARGS__};                             \
        for (const void* _p : _ptrs) ZG_REQUIRE(_p != nullptr, "%s: null pointer", name); \
    }

ZG_API int zg_hip_add(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* z, size_t zl) {
    // a bias row added onto the output of a product that is still waiting becomes part of that product's launch
    if (ctx && ctx->deferred.active && deferred_take_add(ctx, x, xl, y, yl, z, zl)) return ZG_HIP_OK;
    if (ctx && ctx->scatter_wait.active && scatter_take_add(ctx, x, xl, y, yl, z, zl)) return ZG_HIP_OK;
    return binary_op<AddOp>(ctx, "add", x, xl, y, yl, z, zl);
}
ZG_API int zg_hip_sub(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* z, size_t zl) {
    return binary_op<SubOp>(ctx, "sub", x, xl, y, yl, z, zl);
}
ZG_API int zg_hip_mul(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* z, size_t zl) {
    return binary_op<MulOp>(ctx, "mul", x, xl, y, yl, z, zl);
}
ZG_API int zg_hip_div(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* z, size_t zl) {
    return binary_op<DivOp>(ctx, "div", x, xl, y, yl, z, zl);
}

// The scalar operand of add_scalar & co (src/ndarray.zig:251: `.y = &.{s}`, a value on the caller's stack) by value: it
// travels as a kernel argument, so nothing is copied to the device, a small op joins the waiting elementwise ops, and
// the call can be recorded into an execution graph.  Same IEEE operation as the two-array form on a one-float operand.
template <class OpR, class OpL>
static int scalar_op(zg_hip_ctx* ctx, const char* name, const float* x, size_t n, float s, int scalar_is_lhs, float* z) {
    ZG_CHECK_N(name, n, x, z);
    if (scalar_is_lhs) return launch_map<OpL, 1>(ctx, z, x, nullptr, nullptr, n, s);
    return launch_map<OpR, 1>(ctx, z, x, nullptr, nullptr, n, s);
}
ZG_API int zg_hip_add_scalar(zg_hip_ctx* ctx, const float* x, size_t n, float s, int scalar_is_lhs, float* z) {
    return scalar_op<AddScalarR, AddScalarL>(ctx, "add_scalar", x, n, s, scalar_is_lhs, z);
}
ZG_API int zg_hip_sub_scalar(zg_hip_ctx* ctx, const float* x, size_t n, float s, int scalar_is_lhs, float* z) {
    return scalar_op<SubScalarR, SubScalarL>(ctx, "sub_scalar", x, n, s, scalar_is_lhs, z);
}
ZG_API int zg_hip_mul_scalar(zg_hip_ctx* ctx, const float* x, size_t n, float s, int scalar_is_lhs, float* z) {
    return scalar_op<MulScalarR, MulScalarL>(ctx, "mul_scalar", x, n, s, scalar_is_lhs, z);
}
ZG_API int zg_hip_div_scalar(zg_hip_ctx* ctx, const float* x, size_t n, float s, int scalar_is_lhs, float* z) {
    return scalar_op<DivScalarR, DivScalarL>(ctx, "div_scalar", x, n, s, scalar_is_lhs, z);
}

ZG_API int zg_hip_pow_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n, float e) {
    ZG_CHECK_N("pow_fwd", n, x, y);
    return launch_map<PowFwd, 1>(ctx, y, x, nullptr, nullptr, n, e);
}
ZG_API int zg_hip_pow_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, const float* y_g, size_t n, float e, float eps) {
    ZG_CHECK_N("pow_bwd", n, x, x_g, y_g);
    return launch_map<PowBwd, 3>(ctx, x_g, x, x_g, y_g, n, e, eps);
}
ZG_API int zg_hip_sqrt_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n) {
    ZG_CHECK_N("sqrt_fwd", n, x, y);
    return launch_map<SqrtFwd, 1>(ctx, y, x, nullptr, nullptr, n);
}
ZG_API int zg_hip_sqrt_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, const float* y_g, size_t n, float eps) {
    ZG_CHECK_N("sqrt_bwd", n, x, x_g, y_g);
    return launch_map<SqrtBwd, 3>(ctx, x_g, x, x_g, y_g, n, eps);
}
ZG_API int zg_hip_rsqrt_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n, float eps) {
    ZG_CHECK_N("rsqrt_fwd", n, x, y);
    return launch_map<RsqrtFwd, 1>(ctx, y, x, nullptr, nullptr, n, eps);
}
ZG_API int zg_hip_rsqrt_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, const float* y_g, size_t n, float eps) {
    ZG_CHECK_N("rsqrt_bwd", n, x, x_g, y_g);
    return launch_map<RsqrtBwd, 3>(ctx, x_g, x, x_g, y_g, n, eps);
}
ZG_API int zg_hip_exp_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n) {
    ZG_CHECK_N("exp_fwd", n, x, y);
    return launch_map<ExpFwd, 1>(ctx, y, x, nullptr, nullptr, n);
}
ZG_API int zg_hip_exp_bwd(zg_hip_ctx* ctx, float* x_g, const float* y, const float* y_g, size_t n) {
    ZG_CHECK_N("exp_bwd", n, x_g, y, y_g);
    return launch_map<ExpBwd, 3>(ctx, x_g, y, x_g, y_g, n);
}
ZG_API int zg_hip_relu_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n) {
    // in place on the output of a product that is still waiting: done in that product's epilogue
    int taken_rc = 0;
    if (ctx && ctx->deferred.active && deferred_take_relu(ctx, x, y, n, &taken_rc)) return taken_rc;
    if (ctx && ctx->scatter_wait.active && scatter_take_relu(ctx, x, y, n, &taken_rc)) return taken_rc;
    ZG_CHECK_N("relu_fwd", n, x, y);
    return launch_map<ReluFwd, 1>(ctx, y, x, nullptr, nullptr, n);
}
ZG_API int zg_hip_relu_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, const float* y_g, size_t n) {
    ZG_CHECK_N("relu_bwd", n, x, x_g, y_g);
    return launch_map<ReluBwd, 3>(ctx, x_g, x, x_g, y_g, n);
}
ZG_API int zg_hip_relu_inplace_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, size_t n) {
    // the mask of an input gradient whose product is still waiting: applied in that product's epilogue
    int taken_rc = 0;
    if (ctx && ctx->deferred.active && deferred_take_relu_mask(ctx, x, x_g, n, &taken_rc)) return taken_rc;
    ZG_CHECK_N("relu_inplace_bwd", n, x, x_g);
    return launch_map<ReluInplaceBwd, 2>(ctx, x_g, x, x_g, nullptr, n);
}
ZG_API int zg_hip_tanh_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n) {
    ZG_CHECK_N("tanh_fwd", n, x, y);
    return launch_map<TanhFwd, 1>(ctx, y, x, nullptr, nullptr, n);
}
ZG_API int zg_hip_tanh_bwd(zg_hip_ctx* ctx, float* x_g, const float* y, const float* y_g, size_t n) {
    ZG_CHECK_N("tanh_bwd", n, x_g, y, y_g);
    return launch_map<TanhBwd, 3>(ctx, x_g, y, x_g, y_g, n);
}
ZG_API int zg_hip_tanh_inplace_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, size_t n) {
    ZG_CHECK_N("tanh_inplace_bwd", n, x, x_g);
    return launch_map<TanhInplaceBwd, 2>(ctx, x_g, x, x_g, nullptr, n);
}
ZG_API int zg_hip_sigm_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n) {
    ZG_CHECK_N("sigm_fwd", n, x, y);
    return launch_map<SigmFwd, 1>(ctx, y, x, nullptr, nullptr, n);
}
ZG_API int zg_hip_sigm_bwd(zg_hip_ctx* ctx, float* x_g, const float* y, const float* y_g, size_t n) {
    ZG_CHECK_N("sigm_bwd", n, x_g, y, y_g);
    return launch_map<SigmBwd, 3>(ctx, x_g, y, x_g, y_g, n);
}
ZG_API int zg_hip_sigm_inplace_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, size_t n) {
    ZG_CHECK_N("sigm_inplace_bwd", n, x, x_g);
    return launch_map<SigmInplaceBwd, 2>(ctx, x_g, x, x_g, nullptr, n);
}
ZG_API int zg_hip_clamp_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t n, float lo, float hi) {
    ZG_CHECK_N("clamp_fwd", n, x, y);
    return launch_map<ClampFwd, 1>(ctx, y, x, nullptr, nullptr, n, lo, hi);
}
ZG_API int zg_hip_clamp_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, const float* y_g, size_t n, float lo,
                            float hi) {
    ZG_CHECK_N("clamp_bwd", n, x, x_g, y_g);
    return launch_map<ClampBwd, 3>(ctx, x_g, x, x_g, y_g, n, lo, hi);
}
ZG_API int zg_hip_scale(zg_hip_ctx* ctx, float* x, size_t n, float alpha) {
    ZG_CHECK_N("scale", n, x);
    return launch_map<ScaleOp, 1>(ctx, x, x, nullptr, nullptr, n, alpha);
}

// src/device/host_device.zig:782-795 (see the oracle for the double application when lengths are equal)
ZG_API int zg_hip_broadcast(zg_hip_ctx* ctx, const float* x, size_t xl, float* y, size_t yl, float alpha, float beta) {
    ZG_CTX(ctx);
    ZG_REQUIRE(xl > 0 && yl > 0 && x && y, "broadcast: empty or null operand");
    ZG_REQUIRE(yl % xl == 0, "broadcast: y.len %zu is not a multiple of x.len %zu", yl, xl);
    if (xl == yl) {
        int rc = launch_map<ScaledCopy, 2>(ctx, y, x, y, nullptr, yl, alpha, beta);
        if (rc) return rc;
        return launch_map<ScaledCopy, 2>(ctx, y, x, y, nullptr, yl, alpha, beta);
    }
    if (aligned16(y) && yl >= 4) {  // the flat walk in 16-byte pieces of the binary ops (33554432 values from 16: 60 -> 48 us)
        int grid = map_grid(ctx, yl >> 2, kBlock * kPeriodU);
        hipLaunchKernelGGL((bin_period_kernel<AxpbyPeriod>), dim3(grid), dim3(kBlock), 0, ctx->stream,
                           AxpbyPeriod{alpha, beta}, y, y, x, yl, xl);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    int grid = map_grid(ctx, yl, kBlock);
    hipLaunchKernelGGL(broadcast_modulo_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, y, x, xl, yl, alpha, beta);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_smooth_l1_bwd(zg_hip_ctx* ctx, const float* pred, const float* target, float* grad, size_t n,
                                float beta) {
    ZG_CHECK_N("smooth_l1_bwd", n, pred, target, grad);
    return launch_map<SmoothL1Bwd, 3>(ctx, grad, pred, target, grad, n, beta, (float)n);
}

ZG_API int zg_hip_mse_bwd(zg_hip_ctx* ctx, const float* pred, const float* target, float* grad, size_t n) {
    ZG_CHECK_N("mse_bwd", n, pred, target, grad);
    return launch_map<MseBwd, 3>(ctx, grad, pred, target, grad, n, 2.0f / (float)n);
}
