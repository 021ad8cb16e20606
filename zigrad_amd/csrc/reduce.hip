// Reductions: flat (sum|x|, sum, nrm2, dot, isamax-style max, clip), along an axis (sum / max /
// argmax over the last, the first or a middle axis), and unbroadcast.
//
// All of them are HBM-bound single passes.  Flat and column reductions with many rows are two
// launches (per-block partials, then one block that combines the partials in a fixed order); there is
// no cross-workgroup communication inside a kernel and no floating-point atomics, so results do not
// depend on scheduling.
#include "reduce_device.h"

namespace zg {

// max_bwd: x_g[i] += y_g[0] where x[i] == y[0]   (src/device/host_device.zig:582-588)
__global__ __launch_bounds__(kBlock) void max_bwd_kernel(const float* x, float* x_g, size_t n, const float* y,
                                                          const float* y_g) {
    const float val = y[0], grd = y_g[0];
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    for (; i < n; i += nt)
        if (val == x[i]) x_g[i] = __fadd_rn(x_g[i], grd);
}

// y += alpha[0] * x with alpha in device memory (src/device/host_device.zig:269-275)
__global__ __launch_bounds__(kBlock) void axpy_kernel(const float* x, float* y, size_t n, const float* alpha_ptr,
                                                       float alpha_value) {
    const float al = alpha_ptr ? alpha_ptr[0] : alpha_value;
    const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    if (vec) {
        const float4* x4 = reinterpret_cast<const float4*>(x);
        float4* y4 = reinterpret_cast<float4*>(y);
        const size_t n4 = n >> 2;
        for (size_t i = tid; i < n4; i += nt) {
            float4 u = x4[i], v = y4[i];
            v.x = __fadd_rn(v.x, __fmul_rn(al, u.x));
            v.y = __fadd_rn(v.y, __fmul_rn(al, u.y));
            v.z = __fadd_rn(v.z, __fmul_rn(al, u.z));
            v.w = __fadd_rn(v.w, __fmul_rn(al, u.w));
            y4[i] = v;
        }
        for (size_t t = (n4 << 2) + tid; t < n; t += nt) y[t] = __fadd_rn(y[t], __fmul_rn(al, x[t]));
    } else {
        for (size_t i = tid; i < n; i += nt) y[i] = __fadd_rn(y[i], __fmul_rn(al, x[i]));
    }
}

static int stream_grid(zg_hip_ctx* ctx, size_t n, size_t per_thread) {
    size_t blocks = ceil_div_sz(n, (size_t)kBlock * per_thread);
    (void)ctx;  // one trip per thread at any size (axpy on 268 M elements: 58 -> 71 % of 8 TB/s without the cap)
    size_t cap = 0x7fffffffull;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

// ------------------------------------------------------------------------------------------------
// reductions along an axis.  x is viewed as [outer, R, inner]; R is reduced.
// ------------------------------------------------------------------------------------------------
struct AxisMax {
    using P = MaxAcc;
    using Out = float;
    static __device__ __forceinline__ float term(float v, uint32_t) { return v; }
    static __device__ __forceinline__ void store(Out* y, size_t o, float s, float, float) { y[o] = s; }
};
struct AxisArgmax {
    using P = ArgmaxAcc;
    using Out = uint64_t;
    static __device__ __forceinline__ ArgAccT term(float v, uint32_t r) { return ArgAccT{v, r}; }
    // an all -inf / NaN slice keeps the sentinel; the host loop would answer 0 there
    static __device__ __forceinline__ void store(Out* y, size_t o, ArgAccT s, float, float) {
        y[o] = (s.i == 0xffffffffu) ? 0 : (uint64_t)s.i;
    }
};

// inner == 1: rows of `cols` contiguous elements, TPR threads per row, 256/TPR rows per workgroup
template <class A, int TPR>
__global__ __launch_bounds__(kBlock) void row_reduce_kernel(const float* x, typename A::Out* y, size_t rows, size_t cols,
                                                             float alpha, float beta) {
    using P = typename A::P;
    constexpr int kRows = kBlock / TPR;
    const int lane = threadIdx.x % TPR;
    const size_t row = (size_t)blockIdx.x * kRows + threadIdx.x / TPR;
    typename P::Acc acc = P::init();
    if (row < rows) {
        const float* xr = x + row * cols;
        // A row starts wherever row * cols puts it: its values before the first 16-byte boundary and after the last whole
        // 16-byte piece (at most three each) are dealt to the lanes one by one, the pieces between are read 16 bytes at a time
        // (sums over the rows of [8192, 32001] value by value: 47 % of 8 TB/s against 84 % for 32000 columns).  Rows of
        // fewer than eight pieces per lane that are not whole pieces stay value by value.
        size_t h = (size_t)((0 - (reinterpret_cast<uintptr_t>(xr) >> 2)) & 3);
        if (h > cols) h = cols;
        const bool vec = (h == 0 && cols % 4 == 0) || cols >= (size_t)8 * TPR;
        if (vec) {
            const float4* x4 = reinterpret_cast<const float4*>(xr + h);
            const size_t c4 = (cols - h) >> 2;
            const uint32_t h32 = (uint32_t)h;
            for (size_t i = lane; i < h; i += TPR) acc = P::combine(acc, A::term(xr[i], (uint32_t)i));
            // whole trips of four loads per lane, then one partial trip whose loads are in flight together as well, the
            // ones past the row's end left out: the trip count is the same for every lane, so a row of 1000 columns takes
            // one memory round trip like a row of 1024 (lanes that finish one by one cost a quarter more)
            size_t j0 = 0;
            for (; j0 + 4 * TPR <= c4; j0 += 4 * TPR) {
                const size_t j = j0 + lane;
                float4 v0 = nt_load(x4 + j), v1 = nt_load(x4 + j + TPR), v2 = nt_load(x4 + j + 2 * TPR), v3 = nt_load(x4 + j + 3 * TPR);
                const float4 vs[4] = {v0, v1, v2, v3};
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    uint32_t c = h32 + (uint32_t)(4 * (j + (size_t)u * TPR));
                    acc = P::combine(acc, A::term(vs[u].x, c + 0));
                    acc = P::combine(acc, A::term(vs[u].y, c + 1));
                    acc = P::combine(acc, A::term(vs[u].z, c + 2));
                    acc = P::combine(acc, A::term(vs[u].w, c + 3));
                }
            }
            if (j0 < c4) {
                const size_t j = j0 + lane;
                const bool streamed = cols >= 512;  // rows of a few hundred bytes are read faster through the caches
                float4 vs[4];
#pragma unroll
                for (int u = 0; u < 4; u++)
                    if (j + (size_t)u * TPR < c4) vs[u] = streamed ? nt_load(x4 + j + (size_t)u * TPR) : x4[j + (size_t)u * TPR];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    if (j + (size_t)u * TPR < c4) {
                        uint32_t c = h32 + (uint32_t)(4 * (j + (size_t)u * TPR));
                        acc = P::combine(acc, A::term(vs[u].x, c + 0));
                        acc = P::combine(acc, A::term(vs[u].y, c + 1));
                        acc = P::combine(acc, A::term(vs[u].z, c + 2));
                        acc = P::combine(acc, A::term(vs[u].w, c + 3));
                    }
                }
            }
            for (size_t i = h + (c4 << 2) + (size_t)lane; i < cols; i += TPR) acc = P::combine(acc, A::term(xr[i], (uint32_t)i));
        } else {
            for (size_t j = lane; j < cols; j += TPR) acc = P::combine(acc, A::term(xr[j], (uint32_t)j));
        }
    }
    if (TPR <= kWave) {
        acc = group_reduce<P, (TPR <= kWave ? TPR : kWave)>(acc);
    } else {
        __shared__ typename P::Acc smem[kBlock / kWave];
        acc = block_reduce<P>(acc, smem);
    }
    if (lane == 0 && row < rows) A::store(y, row, acc, alpha, beta);
}

// inner == 1 with few, long rows (a handful of rows of a million columns would keep a handful of workgroups busy): the
// rows are cut into segments of `seg` columns (a multiple of 4), workgroup (s, r) reduces segment s of row r and leaves
// its result at partials[s * rows + r]; col_final_kernel then combines a row's segments in a fixed order.
template <class A>
__global__ __launch_bounds__(kBlock) void row_segments_kernel(const float* x, typename A::P::Acc* partials, size_t rows,
                                                               size_t cols, size_t seg) {
    using P = typename A::P;
    __shared__ typename P::Acc smem[kBlock / kWave];
    const size_t s = blockIdx.x, row = blockIdx.y;
    const size_t c_begin = s * seg, c_end = c_begin + seg < cols ? c_begin + seg : cols;
    const float* xr = x + row * cols;
    typename P::Acc acc = P::init();
    // the segment's values before its first 16-byte boundary and after its last whole 16-byte piece (at most three each,
    // none where rows start on 16-byte boundaries) go to the first threads, the pieces between are read 16 bytes at a time
    const float* sp = xr + c_begin;
    const size_t len = c_end - c_begin;
    size_t h = (size_t)((0 - (reinterpret_cast<uintptr_t>(sp) >> 2)) & 3);
    if (h > len) h = len;
    if (threadIdx.x < h) acc = P::combine(acc, A::term(sp[threadIdx.x], (uint32_t)(c_begin + threadIdx.x)));
    {
        const float4* x4 = reinterpret_cast<const float4*>(sp + h);
        const size_t j_end = (len - h) >> 2;
        const uint32_t c0 = (uint32_t)(c_begin + h);
        size_t j = threadIdx.x;
        for (; j + 3 * kBlock < j_end; j += 4 * kBlock) {
            const float4 vs[4] = {nt_load(x4 + j), nt_load(x4 + j + kBlock), nt_load(x4 + j + 2 * kBlock),
                                  nt_load(x4 + j + 3 * kBlock)};
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t c = c0 + (uint32_t)(4 * (j + (size_t)u * kBlock));
                acc = P::combine(acc, A::term(vs[u].x, c + 0));
                acc = P::combine(acc, A::term(vs[u].y, c + 1));
                acc = P::combine(acc, A::term(vs[u].z, c + 2));
                acc = P::combine(acc, A::term(vs[u].w, c + 3));
            }
        }
        for (; j < j_end; j += kBlock) {
            const float4 v = x4[j];
            const uint32_t c = c0 + (uint32_t)(4 * j);
            acc = P::combine(acc, A::term(v.x, c + 0));
            acc = P::combine(acc, A::term(v.y, c + 1));
            acc = P::combine(acc, A::term(v.z, c + 2));
            acc = P::combine(acc, A::term(v.w, c + 3));
        }
        const size_t tail = h + (j_end << 2) + threadIdx.x;
        if (tail < len) acc = P::combine(acc, A::term(sp[tail], (uint32_t)(c_begin + tail)));
    }
    acc = block_reduce<P>(acc, smem);
    if (threadIdx.x == 0) partials[s * rows + row] = acc;
}

// inner > 1: column-style, see col_reduce_block
template <class A, int V>
__global__ __launch_bounds__(kBlock) void col_reduce_kernel(const float* x, typename A::Out* y,
                                                             typename A::P::Acc* partials, size_t R, size_t inner,
                                                             int log2_cx, size_t rows_per_chunk, float alpha,
                                                             float beta) {
    __shared__ typename A::P::Acc smem[kBlock * V];
    col_reduce_block<A, V>(x, y, partials, R, inner, log2_cx, rows_per_chunk, alpha, beta, blockIdx.x, blockIdx.y,
                           blockIdx.z, gridDim.y, smem);
}

// Workgroup = 64 adjacent outputs x 4 waves; wave w combines chunks w, w+4, w+8, ... of its outputs with all its
// loads in flight at once (16 per thread up to 64 chunks, rounds of 32 beyond), then the four wave results are combined in
// wave order.  The order is fixed, so the result does not depend on scheduling.
template <class A>
__global__ __launch_bounds__(kBlock) void col_final_kernel(const typename A::P::Acc* partials, typename A::Out* y,
                                                            size_t n_out, size_t inner, int chunks, float alpha,
                                                            float beta) {
    using P = typename A::P;
    using Acc = typename P::Acc;
    __shared__ Acc smem[kBlock];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const size_t o = (size_t)blockIdx.x * 64 + lane;
    Acc acc = P::init();
    if (o < n_out) {
        const size_t outer = o / inner, c = o % inner;
        const Acc* pp = partials + (outer * chunks) * inner + c;
        if (chunks <= 64) {  // one round: 16 loads in flight per thread
            Acc t[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int k = w + 4 * u;
                if (k < chunks) t[u] = pp[(size_t)k * inner];
            }
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int k = w + 4 * u;
                if (k < chunks) acc = P::combine(acc, t[u]);
            }
        } else {
            for (int base = 0; base < chunks; base += 128) {  // 128 chunks per round: 32 loads in flight per thread
                Acc t[32];
#pragma unroll
                for (int u = 0; u < 32; u++) {
                    const int k = base + w + 4 * u;
                    if (k < chunks) t[u] = pp[(size_t)k * inner];
                }
#pragma unroll
                for (int u = 0; u < 32; u++) {
                    const int k = base + w + 4 * u;
                    if (k < chunks) acc = P::combine(acc, t[u]);
                }
            }
        }
    }
    smem[threadIdx.x] = acc;
    __syncthreads();
    if (w == 0 && o < n_out) {
        for (int t = 1; t < 4; t++) acc = P::combine(acc, smem[t * 64 + lane]);
        A::store(y, o, acc, alpha, beta);
    }
}

template <class A>
static int axis_reduce(zg_hip_ctx* ctx, const float* x, typename A::Out* y, size_t outer, size_t R, size_t inner,
                       float alpha, float beta) {
    using Acc = typename A::P::Acc;
    if (outer == 0 || R == 0 || inner == 0) return ZG_HIP_OK;
    if (inner == 1) {
        const size_t rows = outer, cols = R;
        // few long rows: segments of at least 4096 columns, about eight workgroups per compute unit, then a row's segments
        // are combined by the column kernel's final pass (7 x 1048576: 137 -> 9 us; 64 x 262144: 40 -> 13 us)
        // (below a million elements or so, rows of up to 65536 columns are done sooner in the one launch: 7 x 65536
        // 5.1 against 7.6 us)
        if (rows < 2 * (size_t)ctx->n_cu && (cols >= 131072 || (cols >= 16384 && rows * cols >= ((size_t)1 << 20)))) {
            const size_t want = ceil_div_sz(8 * (size_t)ctx->n_cu, rows);
            size_t seg = ceil_div_sz(ceil_div_sz(cols, want), 1024) * 1024;
            if (seg < 4096) seg = 4096;
            const size_t n_seg = ceil_div_sz(cols, seg);
            if (n_seg >= 2) {
                Acc* partials = (Acc*)workspace(ctx, n_seg * rows * sizeof(Acc));
                if (!partials) return ZG_HIP_EOOM;
                hipLaunchKernelGGL((row_segments_kernel<A>), dim3((unsigned)n_seg, (unsigned)rows), dim3(kBlock), 0, ctx->stream,
                                   x, partials, rows, cols, seg);
                ZG_LAUNCH_CHECK();
                hipLaunchKernelGGL((col_final_kernel<A>), dim3((unsigned)ceil_div_sz(rows, 64)), dim3(kBlock), 0, ctx->stream,
                                   partials, y, rows, rows, (int)n_seg, alpha, beta);
                ZG_LAUNCH_CHECK();
                return ZG_HIP_OK;
            }
        }
#define ZG_ROW(TPR)                                                                                          \
    hipLaunchKernelGGL((row_reduce_kernel<A, TPR>), dim3((unsigned)ceil_div_sz(rows, kBlock / TPR)), dim3(kBlock), 0, \
                       ctx->stream, x, y, rows, cols, alpha, beta)
        // lanes per row so that a lane has 8 to 16 values of a short row: with four lanes on a row of 4 to 12 values
        // and sixteen on one of 64 to 128 most lanes had one load or none (sums over the rows of [8388608, 4]: 70 -> 27 us,
        // [2097152, 16]: 25.6 -> 21.2 us, [524288, 64]: 25.1 -> 20.8 us, 82 to 86 % of 8 TB/s)
        if (cols < 16) ZG_ROW(1);
        else if (cols < 32) ZG_ROW(2);
        else if (cols < 64) ZG_ROW(4);
        else if (cols < 192) ZG_ROW(8);
        else if (cols <= 256) ZG_ROW(16);
        else if (cols <= 16384 || rows >= (size_t)ctx->n_cu * 8) ZG_ROW(64);
        else ZG_ROW(256);
#undef ZG_ROW
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    const bool wide = inner >= 1024 && R >= 256 && outer * R * inner > kColSingleChunkMax;
    const ColReduceShape cs = col_reduce_shape(x, inner, wide);
    const bool v4 = cs.V == 4;
    const int log2_cx = cs.log2_cx;
    const int ry = kBlock >> log2_cx;
    const size_t gx = cs.gx;
    // row chunks: enough workgroups to cover the machine several times, but at least 4 trips of ry rows each
    size_t want = (size_t)ctx->n_cu * 8;
    size_t chunks = ceil_div_sz(want, gx * outer);
    size_t max_chunks = ceil_div_sz(R, (size_t)ry * 4);
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks < 1) chunks = 1;
    // keeps the partials buffer and the serial tail of the final stage small (the wide shape has a quarter of the
    // column groups, so it takes more chunks for enough workgroups)
    size_t chunk_cap = (wide && ry == 1) ? 256 : 64;
    if (!(wide && ry == 1)) {
        // tall matrices of few columns: with 64 chunks a matrix of a single column group runs on 64 workgroups (4194304 x
        // 64: 361 us, 37 % of 8 TB/s).  128 workgroups in all from 64 MiB and 256 from 256 MiB, so chunks of 512 KiB at
        // least (4194304 x 64: 187 us, 1048576 x 64: 62 -> 43 us, 262144 x 256: 62 -> 41 us); more than that and the
        // final stage, one workgroup per 64 outputs walking every chunk, costs what the first stage gains
        const size_t total = outer * R * inner;
        const size_t groups = total >= ((size_t)1 << 26) ? 256 : total >= ((size_t)1 << 24) ? 128 : 64;
        size_t c = groups / (gx * outer);
        if (c > chunk_cap) chunk_cap = c;
    }
    if (chunks > chunk_cap) chunks = chunk_cap;
    if (outer * R * inner <= kColSingleChunkMax) chunks = 1;  // a second launch costs more than a chunk split saves
    const size_t rows_per_chunk = ceil_div_sz(R, chunks);
    chunks = ceil_div_sz(R, rows_per_chunk);
    ZG_REQUIRE(outer <= 65535, "axis reduction: %zu leading slices exceed the grid limit", outer);
    Acc* partials = nullptr;
    if (chunks > 1) {
        partials = (Acc*)workspace(ctx, outer * chunks * inner * sizeof(Acc));
        if (!partials) return ZG_HIP_EOOM;
    }
    dim3 grid((unsigned)gx, (unsigned)chunks, (unsigned)outer);
    if (v4)
        hipLaunchKernelGGL((col_reduce_kernel<A, 4>), grid, dim3(kBlock), 0, ctx->stream, x, y, partials, R, inner,
                           log2_cx, rows_per_chunk, alpha, beta);
    else
        hipLaunchKernelGGL((col_reduce_kernel<A, 1>), grid, dim3(kBlock), 0, ctx->stream, x, y, partials, R, inner,
                           log2_cx, rows_per_chunk, alpha, beta);
    ZG_LAUNCH_CHECK();
    if (chunks > 1) {
        const size_t n_out = outer * inner;
        hipLaunchKernelGGL((col_final_kernel<A>), dim3((unsigned)ceil_div_sz(n_out, 64)), dim3(kBlock), 0,
                           ctx->stream, partials, y, n_out, inner, (int)chunks, alpha, beta);
        ZG_LAUNCH_CHECK();
    }
    return ZG_HIP_OK;
}

static size_t prod(const uint64_t* s, size_t from, size_t to) {
    size_t n = 1;
    for (size_t i = from; i < to; i++) n *= (size_t)s[i];
    return n;
}

static int check_axis_args(const char* name, const void* x, const uint64_t* x_shape, size_t x_rank, const void* y,
                           size_t y_len, size_t dim) {
    ZG_REQUIRE(x && y && x_shape, "%s: null pointer", name);
    ZG_REQUIRE(x_rank >= 1 && x_rank <= 8, "%s: rank %zu not in 1..8", name, x_rank);
    ZG_REQUIRE(dim < x_rank, "%s: dim %zu out of range for rank %zu", name, dim, x_rank);
    for (size_t i = 0; i < x_rank; i++) ZG_REQUIRE(x_shape[i] > 0, "%s: zero-sized dim %zu", name, i);
    const size_t total = prod(x_shape, 0, x_rank);
    ZG_REQUIRE(x_shape[dim] < 0xffffffffull, "%s: reduced dim too large", name);
    ZG_REQUIRE(y_len == total / x_shape[dim] || y_len == 1, "%s: y.len %zu does not match the reduced shape (%zu)", name,
               y_len, total / (size_t)x_shape[dim]);
    return ZG_HIP_OK;
}

// sum_along with the case split of src/device/host_device.zig:798-847
static int sum_along_impl(zg_hip_ctx* ctx, const float* x, const uint64_t* x_shape, size_t x_rank, float* y,
                          size_t y_len, size_t dim, float alpha, float beta) {
    const size_t total = prod(x_shape, 0, x_rank);
    if (y_len == 1) return flat_reduce<TermId, 1>(ctx, x, nullptr, total, 0.f, FinAxpby{y, alpha, beta});
    const size_t outer = prod(x_shape, 0, dim), R = x_shape[dim], inner = prod(x_shape, dim + 1, x_rank);
    ZG_REQUIRE(y_len >= outer * inner, "sum_along: y.len %zu too small for %zu outputs", y_len, outer * inner);
    return axis_reduce<AxisSum>(ctx, x, y, outer, R, inner, alpha, beta);
}

int launch_bias_col_sum(zg_hip_ctx* ctx, const float* x, float* y, size_t R, size_t inner, bool fresh) {
    return axis_reduce<AxisSum>(ctx, x, y, 1, R, inner, 1.f, fresh ? 0.f : 1.f);
}

}  // namespace zg

using namespace zg;

ZG_API int zg_hip_sum(zg_hip_ctx* ctx, const float* x, size_t n, float* y) {
    ZG_CTX(ctx);
    if (n == 0 && y) return zg_hip_mem_fill(ctx, y, 1, 0.f);  // the BLAS call on no elements: 0 (src/device/host_device.zig:315-321)
    ZG_REQUIRE(x && y && n > 0, "sum: null or empty operand");
    return flat_reduce<TermAbs, 1>(ctx, x, nullptr, n, 0.f, FinStore{y});
}

ZG_API int zg_hip_nrm2(zg_hip_ctx* ctx, const float* x, size_t n, float* y) {
    ZG_CTX(ctx);
    if (n == 0 && y) return zg_hip_mem_fill(ctx, y, 1, 0.f);  // (src/device/host_device.zig:331)
    ZG_REQUIRE(x && y && n > 0, "nrm2: null or empty operand");
    return flat_reduce<TermSq, 1>(ctx, x, nullptr, n, 0.f, FinSqrt{y});
}

ZG_API int zg_hip_dot(zg_hip_ctx* ctx, const float* x, const float* y, size_t n, float* z) {
    ZG_CTX(ctx);
    if (n == 0 && z) return zg_hip_mem_fill(ctx, z, 1, 0.f);  // (src/device/host_device.zig:224)
    ZG_REQUIRE(x && y && z && n > 0, "dot: null or empty operand");
    return flat_reduce<TermDot, 2>(ctx, x, y, n, 0.f, FinStore{z});
}

ZG_API int zg_hip_max_fwd(zg_hip_ctx* ctx, const float* x, size_t n, float* y) {
    ZG_CTX(ctx);
    ZG_REQUIRE(x && y && n > 0, "max_fwd: null or empty operand");
    ZG_REQUIRE(n < 0xffffffffull, "max_fwd: more than 2^32-1 elements");
    return flat_reduce<TermAbsArg, 1>(ctx, x, nullptr, n, 0.f, FinAbsArg{y});
}

ZG_API int zg_hip_max_bwd(zg_hip_ctx* ctx, const float* x, float* x_g, size_t n, const float* y, const float* y_g) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && x_g && y && y_g, "max_bwd: null pointer");
    hipLaunchKernelGGL(max_bwd_kernel, dim3(stream_grid(ctx, n, 4)), dim3(kBlock), 0, ctx->stream, x, x_g, n, y, y_g);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// The norm never leaves the device: a reduction writes the clip factor to a device slot and the
// scaling kernel reads it (and returns immediately when the factor is 1).
ZG_API int zg_hip_clip_nrm2(zg_hip_ctx* ctx, float* x, size_t n, float max_norm, float delta) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x != nullptr, "clip_nrm2: null pointer");
    float* factor = ctx->scalar_slot + 1;
    int rc = flat_reduce<TermSq, 1>(ctx, x, nullptr, n, 0.f, FinClipFactor{factor, max_norm, delta});
    if (rc) return rc;
    hipLaunchKernelGGL(scale_by_device_factor_kernel, dim3(stream_grid(ctx, n, 8)), dim3(kBlock), 0, ctx->stream, x, n,
                       factor);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_axpy(zg_hip_ctx* ctx, const float* x, float* y, size_t n, const float* alpha, int alpha_on_device) {
    ZG_CTX(ctx);
    if (n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && y && alpha, "axpy: null pointer");
    // a host scalar travels as a kernel argument; a device scalar is read by the kernel
    hipLaunchKernelGGL(axpy_kernel, dim3(stream_grid(ctx, n, 8)), dim3(kBlock), 0, ctx->stream, x, y, n,
                       alpha_on_device ? alpha : (const float*)nullptr, alpha_on_device ? 0.f : alpha[0]);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_smooth_l1_fwd(zg_hip_ctx* ctx, const float* pred, const float* target, size_t n, float beta,
                                float* loss) {
    ZG_CTX(ctx);
    ZG_REQUIRE(pred && target && loss && n > 0, "smooth_l1_fwd: null or empty operand");
    return flat_reduce<TermSmoothL1, 2>(ctx, pred, target, n, beta, FinDivN{loss, (float)n});
}

// smooth_l1_fwd followed by the backward of the scalar loss (upstream gradient 1): grad (+)= d loss / d pred.  Up to
// kSmoothL1SmallMax elements take one launch of one workgroup, which forms the mean as flat_single_kernel does and
// the gradient elements as the separate backward op does; larger inputs take the separate launches.
constexpr size_t kSmoothL1SmallMax = 4096;
template <bool ACC>
__global__ __launch_bounds__(kFlatSingle) void smooth_l1_small_kernel(const float* pred, const float* target, float* grad,
                                                                      size_t n, float beta, float* loss) {
    __shared__ float smem[kFlatSingle / kWave];
    float acc = flat_accumulate<TermSmoothL1, 2>(pred, target, n, beta, threadIdx.x, blockDim.x);
    acc = block_reduce<SumAcc>(acc, smem);
    if (threadIdx.x == 0) FinDivN{loss, (float)n}(acc);
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float d = smooth_l1_grad(pred[i], target[i], beta, (float)n);
        grad[i] = ACC ? __fadd_rn(grad[i], d) : d;
    }
}

ZG_API int zg_hip_smooth_l1_fwd_bwd(zg_hip_ctx* ctx, const float* pred, const float* target, float* grad, size_t n,
                                    float beta, float* loss, int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(pred && target && grad && loss && n > 0, "smooth_l1_fwd_bwd: null or empty operand");
    if (n <= kSmoothL1SmallMax) {
        if (accumulate)
            hipLaunchKernelGGL(smooth_l1_small_kernel<true>, dim3(1), dim3(kFlatSingle), 0, ctx->stream, pred, target, grad, n,
                               beta, loss);
        else
            hipLaunchKernelGGL(smooth_l1_small_kernel<false>, dim3(1), dim3(kFlatSingle), 0, ctx->stream, pred, target, grad,
                               n, beta, loss);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (int rc = zg_hip_smooth_l1_fwd(ctx, pred, target, n, beta, loss)) return rc;
    if (!accumulate)
        if (int rc = zg_hip_mem_fill(ctx, grad, n, 0.f)) return rc;
    return zg_hip_smooth_l1_bwd(ctx, pred, target, grad, n, beta);
}

ZG_API int zg_hip_mse_fwd(zg_hip_ctx* ctx, const float* pred, const float* target, size_t n, float* loss) {
    ZG_CTX(ctx);
    ZG_REQUIRE(pred && target && loss && n > 0, "mse_fwd: null or empty operand");
    return flat_reduce<TermSqDiff, 2>(ctx, pred, target, n, 0.f, FinDivN{loss, (float)n});
}

ZG_API int zg_hip_sum_along(zg_hip_ctx* ctx, const float* x, const uint64_t* x_shape, size_t x_rank, float* y,
                            size_t y_len, size_t dim, float alpha, float beta) {
    ZG_CTX(ctx);
    int rc = check_axis_args("sum_along", x, x_shape, x_rank, y, y_len, dim);
    if (rc) return rc;
    return sum_along_impl(ctx, x, x_shape, x_rank, y, y_len, dim, alpha, beta);
}

ZG_API int zg_hip_max_along(zg_hip_ctx* ctx, const float* x, const uint64_t* x_shape, size_t x_rank, float* y,
                            size_t y_len, size_t dim) {
    ZG_ENTER(ctx, kWaitAll);
    int rc = check_axis_args("max_along", x, x_shape, x_rank, y, y_len, dim);
    if (rc == ZG_HIP_OK && y_len != prod(x_shape, 0, x_rank) / x_shape[dim]) {
        set_error("max_along: y.len %zu != %zu", y_len, prod(x_shape, 0, x_rank) / (size_t)x_shape[dim]);
        rc = ZG_HIP_EINVAL;
    }
    if (rc) {  // refused: what waits is launched as by any other call
        (void)flush_pending(ctx);
        return rc;
    }
    const size_t outer = prod(x_shape, 0, dim), R = x_shape[dim], inner = prod(x_shape, dim + 1, x_rank);
    zg_pending_fill dropped[kMaxPendingFills];
    int n_dropped = 0;
    {
        // every element of y is written and none is read: a fill inside y that still waits has no reader left
        // (NDArray.max_along zero-fills its output first, src/ndarray.zig:567); the other waiting fills stay unless
        // they meet x or y
        const char *x0 = (const char*)x, *x1 = x0 + outer * R * inner * sizeof(float);
        const char *y0 = (const char*)y, *y1 = y0 + y_len * sizeof(float);
        if (x0 < y1 && y0 < x1) {
            if ((rc = flush_pending(ctx))) return rc;
        } else {
            n_dropped = take_fills_inside(ctx, y, y_len * sizeof(float), dropped);
            const void* ptrs[2] = {x, y};
            const size_t bytes[2] = {(size_t)(x1 - x0), (size_t)(y1 - y0)};
            rc = flush_pending_but_fills(ctx, ptrs, bytes, 2);
        }
    }
    if (rc == ZG_HIP_OK) rc = axis_reduce<AxisMax>(ctx, x, y, outer, R, inner, 1.f, 0.f);
    if (rc) requeue_fills(ctx, dropped, n_dropped);  // refused: y was not overwritten, its fills are still owed
    return rc;
}

ZG_API int zg_hip_argmax_along(zg_hip_ctx* ctx, const float* x, const uint64_t* x_shape, size_t x_rank, uint64_t* y,
                               size_t y_len, size_t dim) {
    ZG_CTX(ctx);
    int rc = check_axis_args("argmax_along", x, x_shape, x_rank, y, y_len, dim);
    if (rc) return rc;
    const size_t outer = prod(x_shape, 0, dim), R = x_shape[dim], inner = prod(x_shape, dim + 1, x_rank);
    ZG_REQUIRE(y_len == outer * inner, "argmax_along: y.len %zu != %zu", y_len, outer * inner);
    return axis_reduce<AxisArgmax>(ctx, x, y, outer, R, inner, 1.f, 0.f);
}

// src/ndarray.zig:701-719
ZG_API size_t zg_hip_unbroadcast_scratch_len(const uint64_t* x_shape, size_t x_rank, const uint64_t* y_shape,
                                             size_t y_rank) {
    if (!x_shape || !y_shape || x_rank < y_rank) return 0;
    const size_t x_size = prod(x_shape, 0, x_rank), y_size = prod(y_shape, 0, y_rank);
    const size_t delta = x_rank - y_rank;
    size_t coef;
    if (delta > 0) {
        coef = prod(x_shape, 0, delta);
    } else {
        size_t mm = x_rank;
        for (size_t i = 0; i < x_rank; i++)
            if (x_shape[i] != y_shape[i]) {
                mm = i;
                break;
            }
        if (mm == x_rank) return 0;
        coef = x_shape[mm];
    }
    const size_t n = y_size * coef;
    return n == x_size ? 0 : n;
}

namespace zg {
__global__ __launch_bounds__(kBlock) void scaled_copy_kernel(const float* x, float* y, size_t n, float alpha, float beta) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
    for (; i < n; i += nt) {
        float r = __fmul_rn(alpha, x[i]);
        y[i] = (beta == 0.f) ? r : __fadd_rn(r, __fmul_rn(beta, y[i]));
    }
}
}  // namespace zg

// The staging of src/device/host_device.zig:709-780: one fold over the leading extra dims, then one
// sum_along per interior 1-dim, alpha/beta applied at every stage exactly as the reference does.
ZG_API int zg_hip_unbroadcast(zg_hip_ctx* ctx, const float* x, const uint64_t* x_shape_in, size_t x_rank_in, float* y,
                              const uint64_t* y_shape_in, size_t y_rank_in, float* scratch, size_t scratch_len,
                              float alpha, float beta) {
    ZG_ENTER(ctx, kWaitAll);
    // what waits goes out before this call's first launch (below); a refused call sends it out too
    struct Settle {
        zg_hip_ctx* ctx;
        bool done = false;
        ~Settle() { if (!done) (void)flush_pending(ctx); }
    } settle{ctx};
    ZG_REQUIRE(x && y && x_shape_in && y_shape_in, "unbroadcast: null pointer");
    ZG_REQUIRE(x_rank_in >= 1 && x_rank_in <= 8 && y_rank_in >= 1 && y_rank_in <= 8, "unbroadcast: rank not in 1..8");
    ZG_REQUIRE(x_rank_in >= y_rank_in, "unbroadcast: x rank %zu < y rank %zu", x_rank_in, y_rank_in);
    const size_t x_len = prod(x_shape_in, 0, x_rank_in), y_len = prod(y_shape_in, 0, y_rank_in);
    ZG_REQUIRE(x_len > 0 && y_len > 0 && x_len % y_len == 0, "unbroadcast: sizes %zu and %zu are incompatible", x_len,
               y_len);
    ZG_REQUIRE(x != y, "unbroadcast: input and output alias");
    if (x_len == y_len) {
        settle.done = true;
        if (int rc = flush_pending(ctx)) return rc;
        hipLaunchKernelGGL(scaled_copy_kernel, dim3(stream_grid(ctx, x_len, 4)), dim3(kBlock), 0, ctx->stream, x, y,
                           x_len, alpha, beta);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    uint64_t xs[8], ys[8];
    size_t xr = 0, yr = 0;
    {
        size_t s = 0;
        while (s < x_rank_in && x_shape_in[s] == 1) s++;
        for (size_t i = s; i < x_rank_in; i++) xs[xr++] = x_shape_in[i];
        size_t b = 0, e = y_rank_in;
        while (b < e && y_shape_in[b] == 1) b++;
        while (e > b && y_shape_in[e - 1] == 1) e--;
        for (size_t i = b; i < e; i++) ys[yr++] = y_shape_in[i];
    }
    size_t ones = 0;
    for (size_t i = 0; i < yr; i++) ones += (ys[i] == 1);

    // every stage is validated before the first launch
    if (xr > yr) {
        const size_t dif = xr - yr;
        const size_t col = prod(xs, dif, xr);
        if (ones == 0) ZG_REQUIRE(col <= y_len, "unbroadcast: fold writes %zu elements into y of %zu", col, y_len);
        else ZG_REQUIRE(scratch && col <= scratch_len, "unbroadcast: scratch of %zu floats needed, %zu given", col, scratch_len);
    }
    settle.done = true;
    if (xr > yr && ones == 0 && alpha == 1.f && beta == 1.f && (x + x_len <= y || y + y_len <= x)) {
        // y += column sums of x, a bias gradient (src/ndtensor.zig:780-796).  A zero fill of exactly y that still
        // waits (zero_grad() before the backward pass) is taken over: the sums are written.  The other waiting fills
        // stay unless they meet x or y; everything else that waits goes out.
        const size_t dif = xr - yr;
        const size_t row = prod(xs, 0, dif), col = prod(xs, dif, xr);
        const bool fresh = absorb_zero_fill(ctx, y, col);
        const void* ptrs[2] = {x, y};
        const size_t bytes[2] = {x_len * sizeof(float), col * sizeof(float)};
        int rc = flush_pending_but_fills(ctx, ptrs, bytes, 2);
        if (rc == ZG_HIP_OK) {
            if (row > 1 && col > 1 && row * col <= kColSingleChunkMax) {
                // one launch of the column kernel: it waits for the layer's two products, which can share its launch
                zg_waiting_bias& b = ctx->bias_wait;
                b.active = true;
                b.gy = x;
                b.gb = y;
                b.R = row;
                b.inner = col;
                b.fresh = fresh;
                return ZG_HIP_OK;
            }
            rc = axis_reduce<AxisSum>(ctx, x, y, 1, row, col, 1.f, fresh ? 0.f : 1.f);
        }
        if (rc && fresh) (void)zg_hip_mem_fill(ctx, y, col, 0.f);  // refused: the zeros are still owed
        return rc;
    }
    if (int rc = flush_pending(ctx)) return rc;
    if (xr > yr) {
        const size_t dif = xr - yr;
        const size_t row = prod(xs, 0, dif), col = prod(xs, dif, xr);
        int rc = axis_reduce<AxisSum>(ctx, x, ones == 0 ? y : scratch, 1, row, col, alpha, beta);
        if (rc) return rc;
        if (ones == 0) return ZG_HIP_OK;
        for (size_t i = dif; i < xr; i++) xs[i - dif] = xs[i];
        xr -= dif;
    }
    size_t i = 0;
    while (ones > 0 && i < xr) {
        if (i < yr && ys[i] == 1 && xs[i] != 1) {
            const float* xd = (xr == x_rank_in) ? x : scratch;
            float* yd = (ones == 1) ? y : scratch;
            const size_t yl = (ones == 1) ? y_len : scratch_len;
            const size_t need = prod(xs, 0, xr) / xs[i];
            ZG_REQUIRE(xd != nullptr && yd != nullptr, "unbroadcast: scratch required but null");
            ZG_REQUIRE(yl == 1 || yl >= need, "unbroadcast: stage output of %zu elements does not fit %zu", need, yl);
            ZG_REQUIRE(xd != yd, "unbroadcast: a stage would read and write the scratch buffer at once");
            int rc = sum_along_impl(ctx, xd, xs, xr, yd, yl, i, alpha, beta);
            if (rc) return rc;
            for (size_t j = i + 1; j < xr; j++) xs[j - 1] = xs[j];
            for (size_t j = i + 1; j < yr; j++) ys[j - 1] = ys[j];
            xr--;
            yr--;
            ones--;
            continue;
        }
        i++;
    }
    return ZG_HIP_OK;
}
