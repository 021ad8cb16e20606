// Wavefront / workgroup reduction building blocks shared by the reduction, loss and optimizer kernels.
#pragma once
#include "common.h"

namespace zg {

// 16-byte loads and stores with the non-temporal hint, for data a kernel touches exactly once
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 nt_load(const float4* p) {
    const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store(float4 v, float4* p) {
    const f32x4_t o = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(o, reinterpret_cast<f32x4_t*>(p));
}

// Quotient and remainder by p of (cq * p + cs + add), for cs < p and add < 8192, without a 64-bit division: a flat walk
// over a matrix divides once per chunk and places each of its pieces with this.
__device__ __forceinline__ void flat_divmod(size_t cq, size_t cs, size_t add, size_t p, size_t& q, size_t& s) {
    size_t off = cs + add;
    if (p >= 8192) {
        q = cq;
        if (off >= p) {
            off -= p;
            q++;
        }
        s = off;
    } else {
        const uint32_t qq = (uint32_t)off / (uint32_t)p;
        q = cq + qq;
        s = off - (size_t)qq * p;
    }
}


// ---- accumulator policies -------------------------------------------------------------------
// combine(a, b) must give the same result for (a, b) and (b, a): the butterfly shuffles below apply
// it with the operands in either order on the two lanes of a pair.

struct SumAcc {
    using Acc = float;
    static __device__ __forceinline__ Acc init() { return 0.f; }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) { return __fadd_rn(a, b); }
    static __device__ __forceinline__ Acc shfl_xor(Acc a, int m) { return __shfl_xor(a, m, kWave); }
};

// strict '>' running max from -inf (src/device/host_device.zig:862-873); NaNs never win
struct MaxAcc {
    using Acc = float;
    static __device__ __forceinline__ Acc init() { return -INFINITY; }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) { return (b > a) ? b : a; }
    static __device__ __forceinline__ Acc shfl_xor(Acc a, int m) { return __shfl_xor(a, m, kWave); }
};

// value + position; larger value wins, equal values keep the smaller position (first occurrence)
struct ArgAccT {
    float v;
    uint32_t i;
};
struct ArgmaxAcc {
    using Acc = ArgAccT;
    static __device__ __forceinline__ Acc init() { return Acc{-INFINITY, 0xffffffffu}; }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) {
        bool take_b = (b.v > a.v) || (b.v == a.v && b.i < a.i);
        return take_b ? b : a;
    }
    static __device__ __forceinline__ Acc shfl_xor(Acc a, int m) {
        Acc r;
        r.v = __shfl_xor(a.v, m, kWave);
        r.i = (uint32_t)__shfl_xor((int)a.i, m, kWave);
        return r;
    }
};

// |value| + position + signed value: the element cblas_isamax picks (first index of the largest |x|)
// The element of largest magnitude, first on ties (cblas_isamax).  Magnitudes are compared as the bit patterns of |x|,
// which order like the values for everything finite and infinite and put every NaN above them (all NaNs count alike):
// an array that holds a NaN yields its first NaN, as the BLAS the reference is built with documents (mkl_rt), instead
// of an element that only looks like the maximum.
struct AbsArgAccT {
    uint32_t a;  // bits of |x|, any NaN as 0x7f800001
    uint32_t i;
    float v;
};
struct AbsArgmaxAcc {
    using Acc = AbsArgAccT;
    static __device__ __forceinline__ Acc init() { return Acc{0u, 0xffffffffu, 0.f}; }
    static __device__ __forceinline__ Acc combine(Acc x, Acc y) {
        bool take_y = (y.a > x.a) || (y.a == x.a && y.i < x.i);
        return take_y ? y : x;
    }
    static __device__ __forceinline__ Acc shfl_xor(Acc x, int m) {
        Acc r;
        r.a = (uint32_t)__shfl_xor((int)x.a, m, kWave);
        r.i = (uint32_t)__shfl_xor((int)x.i, m, kWave);
        r.v = __shfl_xor(x.v, m, kWave);
        return r;
    }
};

// two running sums (used by the online softmax: see loss.hip) are handled there.

// ---- wave and block reductions ---------------------------------------------------------------
template <class P, int WIDTH = kWave>
__device__ __forceinline__ typename P::Acc group_reduce(typename P::Acc v) {
#pragma unroll
    for (int m = WIDTH / 2; m >= 1; m >>= 1) v = P::combine(v, P::shfl_xor(v, m));
    return v;
}

// Result valid in every thread of wave 0 (in particular thread 0). `smem` holds >= blockDim.x/64 entries.
// All threads of the block must call it.
template <class P>
__device__ __forceinline__ typename P::Acc block_reduce(typename P::Acc v, typename P::Acc* smem) {
    v = group_reduce<P>(v);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int nw = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();  // smem may still be read from a previous call
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    if (wave == 0) {
        v = (lane < nw) ? smem[lane] : P::init();
        v = group_reduce<P>(v);
    }
    return v;
}

// ------------------------------------------------------------------------------------------------
// flat reductions
// ------------------------------------------------------------------------------------------------
struct TermId {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float, size_t, float) { return a; }
};
struct TermAbs {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float, size_t, float) { return fabsf(a); }
};
struct TermSq {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float, size_t, float) { return __fmul_rn(a, a); }
};
struct TermDot {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float b, size_t, float) { return __fmul_rn(a, b); }
};
// src/nn/loss.zig:266-274
struct TermSmoothL1 {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float b, size_t, float beta) {
        float d = __fsub_rn(a, b), ad = fabsf(d);
        if (ad < beta) return __fdiv_rn(__fmul_rn(0.5f, __fmul_rn(d, d)), beta);
        return __fsub_rn(ad, __fmul_rn(0.5f, beta));
    }
};
// src/nn/loss.zig:99-102
struct TermSqDiff {
    using P = SumAcc;
    static __device__ __forceinline__ float term(float a, float b, size_t, float) {
        float d = __fsub_rn(a, b);
        return __fmul_rn(d, d);
    }
};
struct TermAbsArg {
    using P = AbsArgmaxAcc;
    static __device__ __forceinline__ AbsArgAccT term(float a, float, size_t i, float) {
        const uint32_t bits = __float_as_uint(a) & 0x7fffffffu;
        return AbsArgAccT{bits > 0x7f800000u ? 0x7f800001u : bits, (uint32_t)i, a};
    }
};

struct FinStore {
    float* y;
    __device__ void operator()(float s) const { y[0] = s; }
};
struct FinAxpby {  // src/device/reduce.zig:45
    float* y;
    float alpha, beta;
    __device__ void operator()(float s) const {
        float r = __fmul_rn(alpha, s);
        y[0] = (beta == 0.f) ? r : __fadd_rn(r, __fmul_rn(beta, y[0]));
    }
};
struct FinSqrt {
    float* y;
    __device__ void operator()(float s) const { y[0] = sqrtf(s); }
};
struct FinDivN {
    float* y;
    float n;
    __device__ void operator()(float s) const { y[0] = __fdiv_rn(s, n); }
};
// src/device/host_device.zig:339-346: the factor clip_nrm2 multiplies by, 1 when no clipping happens
struct FinClipFactor {
    float* factor;
    float max_norm, delta;
    __device__ void operator()(float s) const {
        float norm = sqrtf(s);
        factor[0] = (norm > max_norm) ? __fdiv_rn(max_norm, __fadd_rn(norm, delta)) : 1.0f;
    }
};
struct FinAbsArg {
    float* y;
    __device__ void operator()(AbsArgAccT a) const { y[0] = a.v; }
};

constexpr int kFlatBlock = 256;
constexpr int kFlatSingle = 1024;       // block size of the single-workgroup path
constexpr size_t kFlatSingleMax = 131072;  // up to this many elements one workgroup does everything (one launch of 4-5 us
                                           // against two of 7: measured at 65537 to 131072 elements)
constexpr int kMaxPartials = 2048;

template <class T, int NIN>
__device__ __forceinline__ typename T::P::Acc flat_accumulate(const float* a, const float* b, size_t n, float p0,
                                                               size_t tid, size_t nthreads) {
    using P = typename T::P;
    typename P::Acc acc = P::init();
    const bool vec = ((reinterpret_cast<uintptr_t>(a) | (NIN > 1 ? reinterpret_cast<uintptr_t>(b) : 0)) & 15u) == 0;
    if (vec) {
        const size_t n4 = n >> 2;
        const float4* a4 = reinterpret_cast<const float4*>(a);
        const float4* b4 = reinterpret_cast<const float4*>(b);
        size_t i = tid;
        // eight independent loads in flight per trip while that many are left, then two (a workgroup that walks the
        // 100352 gradients of a 784 x 128 layer alone, just written by another kernel: 7.2 us in twelve trips of two,
        // 6.3 us with three trips of eight, against 2.6 us for a CU to take in 400 KB at all); the terms join the sum in
        // the order of i either way
        for (; i + 7 * nthreads < n4; i += 8 * nthreads) {
            float4 u[8], w[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                u[k] = a4[i + k * nthreads];
                w[k] = make_float4(0, 0, 0, 0);
                if (NIN > 1) w[k] = b4[i + k * nthreads];
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const size_t j = i + k * nthreads;
                acc = P::combine(acc, T::term(u[k].x, w[k].x, 4 * j + 0, p0));
                acc = P::combine(acc, T::term(u[k].y, w[k].y, 4 * j + 1, p0));
                acc = P::combine(acc, T::term(u[k].z, w[k].z, 4 * j + 2, p0));
                acc = P::combine(acc, T::term(u[k].w, w[k].w, 4 * j + 3, p0));
            }
        }
        for (; i + nthreads < n4; i += 2 * nthreads) {
            float4 u0 = a4[i], u1 = a4[i + nthreads];
            float4 w0 = make_float4(0, 0, 0, 0), w1 = w0;
            if (NIN > 1) {
                w0 = b4[i];
                w1 = b4[i + nthreads];
            }
            acc = P::combine(acc, T::term(u0.x, w0.x, 4 * i + 0, p0));
            acc = P::combine(acc, T::term(u0.y, w0.y, 4 * i + 1, p0));
            acc = P::combine(acc, T::term(u0.z, w0.z, 4 * i + 2, p0));
            acc = P::combine(acc, T::term(u0.w, w0.w, 4 * i + 3, p0));
            const size_t j = i + nthreads;
            acc = P::combine(acc, T::term(u1.x, w1.x, 4 * j + 0, p0));
            acc = P::combine(acc, T::term(u1.y, w1.y, 4 * j + 1, p0));
            acc = P::combine(acc, T::term(u1.z, w1.z, 4 * j + 2, p0));
            acc = P::combine(acc, T::term(u1.w, w1.w, 4 * j + 3, p0));
        }
        for (; i < n4; i += nthreads) {
            float4 u0 = a4[i];
            float4 w0 = make_float4(0, 0, 0, 0);
            if (NIN > 1) w0 = b4[i];
            acc = P::combine(acc, T::term(u0.x, w0.x, 4 * i + 0, p0));
            acc = P::combine(acc, T::term(u0.y, w0.y, 4 * i + 1, p0));
            acc = P::combine(acc, T::term(u0.z, w0.z, 4 * i + 2, p0));
            acc = P::combine(acc, T::term(u0.w, w0.w, 4 * i + 3, p0));
        }
        for (size_t t = (n4 << 2) + tid; t < n; t += nthreads)
            acc = P::combine(acc, T::term(a[t], NIN > 1 ? b[t] : 0.f, t, p0));
    } else {
        for (size_t i = tid; i < n; i += nthreads) acc = P::combine(acc, T::term(a[i], NIN > 1 ? b[i] : 0.f, i, p0));
    }
    return acc;
}

// one workgroup reduces everything and finalises
template <class T, int NIN, class Fin>
__global__ __launch_bounds__(kFlatSingle) void flat_single_kernel(const float* a, const float* b, size_t n, float p0,
                                                                  Fin fin) {
    using P = typename T::P;
    __shared__ typename P::Acc smem[kFlatSingle / kWave];
    typename P::Acc acc = flat_accumulate<T, NIN>(a, b, n, p0, threadIdx.x, blockDim.x);
    acc = block_reduce<P>(acc, smem);
    if (threadIdx.x == 0) fin(acc);
}

// The first stage of the two-launch form.  A workgroup walks the input in chunks of kFlatChunk consecutive 16-byte
// pieces (16 KiB per stream), four pieces per thread in flight: consecutive workgroups on consecutive chunks keep
// DRAM pages open, which a grid-stride walk of the whole array does not (67 MB of squares: 18 -> 11 us).
constexpr int kFlatU = 4;
constexpr size_t kFlatChunk = (size_t)kFlatBlock * kFlatU;
// Workgroup `block` of `nblocks` of that stage (a device function so that a launch over several arrays can run the
// same blocks, see optim.hip).
template <class T, int NIN>
__device__ __forceinline__ void flat_partial_block(const float* a, const float* b, size_t n, float p0,
                                                   typename T::P::Acc* partials, size_t block, size_t nblocks,
                                                   typename T::P::Acc* smem) {
    using P = typename T::P;
    typename P::Acc acc = P::init();
    const bool vec = ((reinterpret_cast<uintptr_t>(a) | (NIN > 1 ? reinterpret_cast<uintptr_t>(b) : 0)) & 15u) == 0;
    if (vec) {
        const size_t n4 = n >> 2;
        const float4* a4 = reinterpret_cast<const float4*>(a);
        const float4* b4 = reinterpret_cast<const float4*>(b);
        for (size_t c0 = block * kFlatChunk; c0 < n4; c0 += nblocks * kFlatChunk) {
            float4 u[kFlatU], w[kFlatU];
#pragma unroll
            for (int k = 0; k < kFlatU; k++) {
                const size_t i = c0 + threadIdx.x + (size_t)k * kFlatBlock;
                u[k] = make_float4(0, 0, 0, 0);
                w[k] = u[k];
                if (i < n4) {
                    u[k] = a4[i];
                    if (NIN > 1) w[k] = b4[i];
                }
            }
#pragma unroll
            for (int k = 0; k < kFlatU; k++) {
                const size_t i = c0 + threadIdx.x + (size_t)k * kFlatBlock;
                if (i < n4) {
                    acc = P::combine(acc, T::term(u[k].x, w[k].x, 4 * i + 0, p0));
                    acc = P::combine(acc, T::term(u[k].y, w[k].y, 4 * i + 1, p0));
                    acc = P::combine(acc, T::term(u[k].z, w[k].z, 4 * i + 2, p0));
                    acc = P::combine(acc, T::term(u[k].w, w[k].w, 4 * i + 3, p0));
                }
            }
        }
        const size_t tid = block * kFlatBlock + threadIdx.x, nthreads = nblocks * kFlatBlock;
        for (size_t t = (n4 << 2) + tid; t < n; t += nthreads)
            acc = P::combine(acc, T::term(a[t], NIN > 1 ? b[t] : 0.f, t, p0));
    } else {
        acc = flat_accumulate<T, NIN>(a, b, n, p0, block * kFlatBlock + threadIdx.x, nblocks * kFlatBlock);
    }
    acc = block_reduce<P>(acc, smem);
    if (threadIdx.x == 0) partials[block] = acc;
}

template <class T, int NIN>
__global__ __launch_bounds__(kFlatBlock) void flat_partial_kernel(const float* a, const float* b, size_t n, float p0,
                                                                   typename T::P::Acc* partials) {
    __shared__ typename T::P::Acc smem[kFlatBlock / kWave];
    flat_partial_block<T, NIN>(a, b, n, p0, partials, blockIdx.x, gridDim.x, smem);
}

template <class P, class Fin>
__global__ __launch_bounds__(kFlatBlock) void flat_final_kernel(const typename P::Acc* partials, int n_partials,
                                                                 Fin fin) {
    __shared__ typename P::Acc smem[kFlatBlock / kWave];
    typename P::Acc acc = P::init();
    for (int i = threadIdx.x; i < n_partials; i += kFlatBlock) acc = P::combine(acc, partials[i]);
    acc = block_reduce<P>(acc, smem);
    if (threadIdx.x == 0) fin(acc);
}

// Workgroups of the first stage for n elements: one chunk per workgroup until the partials buffer is full.
static inline size_t flat_partial_blocks(const zg_hip_ctx* ctx, size_t n) {
    size_t blocks = ceil_div_sz(n, kFlatChunk * 4);
    size_t cap = (size_t)ctx->n_cu * 8;
    if (cap > (size_t)kMaxPartials) cap = kMaxPartials;
    return blocks > cap ? cap : blocks;
}

// `partials` holds the per-workgroup results of the two-launch form: room for kMaxPartials accumulators.
template <class T, int NIN, class Fin>
static int flat_reduce_into(zg_hip_ctx* ctx, const float* a, const float* b, size_t n, float p0, Fin fin,
                            void* partials_mem) {
    using P = typename T::P;
    // two operands, or the magnitude-and-position accumulator of max_fwd: one workgroup takes 8.8 and 11.1 us for 131072
    // elements, the two launches 7
    const size_t single_max = (NIN > 1 || sizeof(typename P::Acc) > sizeof(float)) ? kFlatSingleMax / 2 : kFlatSingleMax;
    if (n <= single_max) {
        hipLaunchKernelGGL((flat_single_kernel<T, NIN, Fin>), dim3(1), dim3(kFlatSingle), 0, ctx->stream, a, b, n, p0,
                           fin);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    const size_t blocks = flat_partial_blocks(ctx, n);
    static_assert(kMaxPartials * sizeof(typename P::Acc) <= (64 << 10), "partials buffer too small");
    auto* partials = (typename P::Acc*)partials_mem;
    hipLaunchKernelGGL((flat_partial_kernel<T, NIN>), dim3((unsigned)blocks), dim3(kFlatBlock), 0, ctx->stream, a, b, n,
                       p0, partials);
    ZG_LAUNCH_CHECK();
    hipLaunchKernelGGL((flat_final_kernel<P, Fin>), dim3(1), dim3(kFlatBlock), 0, ctx->stream, partials, (int)blocks,
                       fin);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

template <class T, int NIN, class Fin>
static int flat_reduce(zg_hip_ctx* ctx, const float* a, const float* b, size_t n, float p0, Fin fin) {
    return flat_reduce_into<T, NIN, Fin>(ctx, a, b, n, p0, fin, ctx->partials);
}

// x *= factor[0], skipped entirely when the factor is exactly 1
static __global__ __launch_bounds__(kBlock) void scale_by_device_factor_kernel(float* x, size_t n, const float* factor) {
    const float f = factor[0];
    if (f == 1.0f) return;
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    if (vec) {
        float4* x4 = reinterpret_cast<float4*>(x);
        const size_t n4 = n >> 2;
        for (size_t i = tid; i < n4; i += nt) {
            float4 v = x4[i];
            v.x = __fmul_rn(v.x, f);
            v.y = __fmul_rn(v.y, f);
            v.z = __fmul_rn(v.z, f);
            v.w = __fmul_rn(v.w, f);
            x4[i] = v;
        }
        for (size_t t = (n4 << 2) + tid; t < n; t += nt) x[t] = __fmul_rn(x[t], f);
    } else {
        for (size_t i = tid; i < n; i += nt) x[i] = __fmul_rn(x[i], f);
    }
}


// ------------------------------------------------------------------------------------------------
// sums along the first or a middle axis of [outer, R, inner] (used by reduce.hip and by the fused Linear backward)
// ------------------------------------------------------------------------------------------------
struct AxisSum {
    using P = SumAcc;
    using Out = float;
    static __device__ __forceinline__ float term(float v, uint32_t) { return v; }
    static __device__ __forceinline__ void store(Out* y, size_t o, float s, float alpha, float beta) {
        float r = __fmul_rn(alpha, s);
        y[o] = (beta == 0.f) ? r : __fadd_rn(r, __fmul_rn(beta, y[o]));
    }
};

// inner > 1: column-style.  Workgroup = cx column-threads x ry row-threads (cx*ry = 256), each thread owns V
// adjacent columns and walks rows ty, ty+ry, ... of its row chunk.  grid = (column groups, row chunks, outer).
// With one row chunk the result is stored directly; otherwise per-chunk partials go to `partials`
// laid out [outer, chunks, inner] and col_final_kernel combines them in chunk order.
// The block coordinates are arguments (bx: column group, by: row chunk of n_chunks, bz: outer slice) and `smem` is
// kBlock * V accumulators of the caller's LDS, so that another kernel can run this block beside other work.
template <class A, int V>
__device__ __forceinline__ void col_reduce_block(const float* x, typename A::Out* y, typename A::P::Acc* partials,
                                                 size_t R, size_t inner, int log2_cx, size_t rows_per_chunk,
                                                 float alpha, float beta, unsigned bx, unsigned by, unsigned bz,
                                                 unsigned n_chunks, typename A::P::Acc* smem) {
    using P = typename A::P;
    using Acc = typename P::Acc;
    const int cx = 1 << log2_cx, ry = kBlock >> log2_cx;
    const int tx = threadIdx.x & (cx - 1), ty = threadIdx.x >> log2_cx;
    const size_t colv = (size_t)bx * cx + tx;  // in units of V columns
    const size_t col0 = colv * V;
    const size_t outer = bz;
    const size_t r_begin = (size_t)by * rows_per_chunk;
    size_t r_end = r_begin + rows_per_chunk;
    if (r_end > R) r_end = R;
    Acc acc[V];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = P::init();
    const bool active = col0 < inner;
    if (active) {
        const float* xb = x + outer * R * inner + col0;
        size_t r = r_begin + ty;
        if constexpr (V == 4) {
            // eight rows in flight while there are eight left, then four, then one by one: always combined in row order
            for (; r + 7 * (size_t)ry < r_end; r += 8 * (size_t)ry) {
                float4 vs[8];
#pragma unroll
                for (int u = 0; u < 8; u++) vs[u] = *reinterpret_cast<const float4*>(xb + (r + (size_t)u * ry) * inner);
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    uint32_t rr = (uint32_t)(r + (size_t)u * ry);
                    acc[0] = P::combine(acc[0], A::term(vs[u].x, rr));
                    acc[1 % V] = P::combine(acc[1 % V], A::term(vs[u].y, rr));
                    acc[2 % V] = P::combine(acc[2 % V], A::term(vs[u].z, rr));
                    acc[3 % V] = P::combine(acc[3 % V], A::term(vs[u].w, rr));
                }
            }
            for (; r + 3 * (size_t)ry < r_end; r += 4 * (size_t)ry) {
                float4 v0 = *reinterpret_cast<const float4*>(xb + r * inner);
                float4 v1 = *reinterpret_cast<const float4*>(xb + (r + ry) * inner);
                float4 v2 = *reinterpret_cast<const float4*>(xb + (r + 2 * (size_t)ry) * inner);
                float4 v3 = *reinterpret_cast<const float4*>(xb + (r + 3 * (size_t)ry) * inner);
                const float4 vs[4] = {v0, v1, v2, v3};
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    uint32_t rr = (uint32_t)(r + (size_t)u * ry);
                    acc[0] = P::combine(acc[0], A::term(vs[u].x, rr));
                    acc[1 % V] = P::combine(acc[1 % V], A::term(vs[u].y, rr));
                    acc[2 % V] = P::combine(acc[2 % V], A::term(vs[u].z, rr));
                    acc[3 % V] = P::combine(acc[3 % V], A::term(vs[u].w, rr));
                }
            }
            for (; r < r_end; r += ry) {
                float4 v0 = *reinterpret_cast<const float4*>(xb + r * inner);
                uint32_t rr = (uint32_t)r;
                acc[0] = P::combine(acc[0], A::term(v0.x, rr));
                acc[1 % V] = P::combine(acc[1 % V], A::term(v0.y, rr));
                acc[2 % V] = P::combine(acc[2 % V], A::term(v0.z, rr));
                acc[3 % V] = P::combine(acc[3 % V], A::term(v0.w, rr));
            }
        } else {
            // sixteen rows in flight while there are sixteen left (a single workgroup walking thousands of short rows
            // waits for memory once per trip), then four, then one by one: always combined in row order
            for (; r + 15 * (size_t)ry < r_end; r += 16 * (size_t)ry) {
                float vs[16];
#pragma unroll
                for (int u = 0; u < 16; u++) vs[u] = xb[(r + (size_t)u * ry) * inner];
#pragma unroll
                for (int u = 0; u < 16; u++) acc[0] = P::combine(acc[0], A::term(vs[u], (uint32_t)(r + (size_t)u * ry)));
            }
            for (; r + 3 * (size_t)ry < r_end; r += 4 * (size_t)ry) {
                float v0 = xb[r * inner], v1 = xb[(r + ry) * inner], v2 = xb[(r + 2 * (size_t)ry) * inner],
                      v3 = xb[(r + 3 * (size_t)ry) * inner];
                acc[0] = P::combine(acc[0], A::term(v0, (uint32_t)r));
                acc[0] = P::combine(acc[0], A::term(v1, (uint32_t)(r + ry)));
                acc[0] = P::combine(acc[0], A::term(v2, (uint32_t)(r + 2 * (size_t)ry)));
                acc[0] = P::combine(acc[0], A::term(v3, (uint32_t)(r + 3 * (size_t)ry)));
            }
            for (; r < r_end; r += ry) acc[0] = P::combine(acc[0], A::term(xb[r * inner], (uint32_t)r));
        }
    }
    // combine the ry row-threads of each column in ty order
#pragma unroll
    for (int v = 0; v < V; v++) smem[threadIdx.x * V + v] = acc[v];
    __syncthreads();
    if (ty == 0 && active) {
        for (int t = 1; t < ry; t++) {
#pragma unroll
            for (int v = 0; v < V; v++) acc[v] = P::combine(acc[v], smem[((t << log2_cx) + tx) * V + v]);
        }
#pragma unroll
        for (int v = 0; v < V; v++) {
            size_t c = col0 + v;
            if (c < inner) {
                if (n_chunks == 1)
                    A::store(y, outer * inner + c, acc[v], alpha, beta);
                else
                    partials[(outer * n_chunks + by) * inner + c] = acc[v];
            }
        }
    }
}


// Launch geometry of col_reduce_block for rows of `inner` elements starting at x: V columns per thread, 2^log2_cx
// column-threads per workgroup, gx column groups.
struct ColReduceShape {
    int V, log2_cx;
    size_t gx;
};
// `wide`: all 256 threads side by side (4 KiB of a row per workgroup and trip with V = 4, neighbouring workgroups on the
// neighbouring 4 KiB), each walking the rows of its chunk one after the other: for matrices of many long rows, where
// the narrow shape's four pieces of 1 KiB from four different rows per trip leave the bandwidth to the luck of how the
// rows fall on the memory channels (column sums of [8192,4096]: 19 to 32 us depending on the allocation).
static inline ColReduceShape col_reduce_shape(const float* x, size_t inner, bool wide = false) {
    ColReduceShape s;
    s.V = ((inner % 4 == 0) && aligned16(x)) ? 4 : 1;
    const size_t colv = inner / s.V;
    s.log2_cx = 0;
    // narrow: at most 64 column threads (1 KiB of a row per workgroup with V = 4): more workgroups, fewer partials
    const int max_log2 = (wide && s.V == 4) ? 8 : 6;
    while ((1u << s.log2_cx) < colv && s.log2_cx < max_log2) s.log2_cx++;
    s.gx = ceil_div_sz(colv, (size_t)1 << s.log2_cx);
    return s;
}
constexpr size_t kColSingleChunkMax = 65536;  // up to this many elements the rows are not split into chunks

}  // namespace zg
