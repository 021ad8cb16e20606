// Softmax / cross-entropy kernels: the host loops of src/nn/loss.zig:130-257 as device ops.
//
// Every kernel streams each logit row once per pass with 128-bit accesses.  The integer-label forward
// needs a single pass (online max / sum-of-exponentials); the one-hot forward needs two (it must write
// the probabilities the reference keeps for backward).  Row losses are written to a buffer and summed
// by a fixed-order reduction, so the loss value does not depend on scheduling.
#include "reduce_device.h"

namespace zg {

// exp for the streaming passes of the integer-label kernels: the hardware exponential (v_exp_f32 on x*log2 e).
// Its relative error grows with |x| (about |x| * 1e-7), far below the 1e-5 bound for softmax terms, and it
// keeps these passes HBM-bound: the full-precision routine costs about as many VALU cycles as the load takes.
__device__ __forceinline__ float fexp(float x) {
    return __expf(x);
}

// running (max, sum of exp(x - max))
struct OnlineAccT {
    float m, s;
};
struct OnlineAcc {
    using Acc = OnlineAccT;
    static __device__ __forceinline__ Acc init() { return Acc{-INFINITY, 0.f}; }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) {
        float m = fmaxf(a.m, b.m);
        if (m == -INFINITY) return Acc{m, 0.f};
        float s = __fadd_rn(__fmul_rn(a.s, expf(__fsub_rn(a.m, m))), __fmul_rn(b.s, expf(__fsub_rn(b.m, m))));
        return Acc{m, s};
    }
    static __device__ __forceinline__ Acc shfl_xor(Acc a, int msk) {
        return Acc{__shfl_xor(a.m, msk, kWave), __shfl_xor(a.s, msk, kWave)};
    }
};

__device__ __forceinline__ void online_push(OnlineAccT& a, float x) {
    if (x > a.m) {
        a.s = __fmul_rn(a.s, expf(__fsub_rn(a.m, x)));  // exp(-inf) = 0 on the first element
        a.m = x;
    }
    a.s = __fadd_rn(a.s, expf(__fsub_rn(x, a.m)));
}

// Elements of a row before its first 16-byte boundary (0 to 3, fewer for a row that ends before it).
__device__ __forceinline__ size_t row_head(const float* xr, size_t cols) {
    const size_t h = (size_t)((0 - (reinterpret_cast<uintptr_t>(xr) >> 2)) & 3);
    return h < cols ? h : cols;
}

// one pass over a row: per-thread online accumulation, then a group reduction.  A row starts wherever row * cols puts
// it: the elements before its first 16-byte boundary and after its last whole 16-byte piece (at most three each) are
// pushed one by one by the first lanes, the pieces between are read 16 bytes at a time.  (A row of 32001 or 50257
// columns read value by value ran at 37 % of 8 TB/s where 32000 columns reach 83 %.)
// Rows of fewer than 8 * TPR columns that are not whole 16-byte pieces are pushed value by value by all lanes: with one
// or two pieces per lane the head and the tail cost more than the pieces save ([4194304, 7]: 151 us value by value,
// 204 us in pieces).  KEEP: plain loads, for a caller whose second pass reads the row again; else the row is read with
// the non-temporal hint.
template <int TPR>
__device__ __forceinline__ bool row_in_pieces(size_t h, size_t cols) {
    return (h == 0 && cols % 4 == 0) || cols >= (size_t)8 * TPR;
}
template <int TPR, bool KEEP = false>
__device__ __forceinline__ OnlineAccT row_online(const float* xr, size_t cols, int lane) {
    OnlineAccT acc = OnlineAcc::init();
    const size_t h = row_head(xr, cols);
    auto load = [](const float4* p) { return KEEP ? *p : nt_load(p); };
    if (!row_in_pieces<TPR>(h, cols)) {
        for (size_t j = lane; j < cols; j += TPR)
            if (xr[j] != -INFINITY) online_push(acc, xr[j]);
    } else {
        for (size_t i = lane; i < h; i += TPR)
            if (xr[i] != -INFINITY) online_push(acc, xr[i]);
        const float4* x4 = reinterpret_cast<const float4*>(xr + h);
        const size_t c4 = (cols - h) >> 2;
        // four 16-byte loads in flight per thread; past the end of the row they are replaced by -inf, which adds
        // exp(-inf) = 0, so the last partial round takes the same path as the others
        const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        for (size_t j = lane; j < c4; j += 4 * TPR) {
            const float4 v0 = load(x4 + j);
            const float4 v1 = (j + TPR < c4) ? load(x4 + j + TPR) : ninf;
            const float4 v2 = (j + 2 * TPR < c4) ? load(x4 + j + 2 * TPR) : ninf;
            const float4 v3 = (j + 3 * TPR < c4) ? load(x4 + j + 3 * TPR) : ninf;
            // one rescale per 16 elements: fold the 16 into the running max first
            float mx = fmaxf(fmaxf(fmaxf(v0.x, v0.y), fmaxf(v0.z, v0.w)), fmaxf(fmaxf(v1.x, v1.y), fmaxf(v1.z, v1.w)));
            mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(v2.x, v2.y), fmaxf(v2.z, v2.w)), fmaxf(fmaxf(v3.x, v3.y), fmaxf(v3.z, v3.w))));
            if (mx > acc.m) {
                acc.s = __fmul_rn(acc.s, fexp(__fsub_rn(acc.m, mx)));
                acc.m = mx;
            }
            if (acc.m == -INFINITY) continue;  // nothing but -inf so far: exp(-inf - -inf) must not be formed
            float s = 0.f;
            s += fexp(v0.x - acc.m) + fexp(v0.y - acc.m) + fexp(v0.z - acc.m) + fexp(v0.w - acc.m);
            s += fexp(v1.x - acc.m) + fexp(v1.y - acc.m) + fexp(v1.z - acc.m) + fexp(v1.w - acc.m);
            s += fexp(v2.x - acc.m) + fexp(v2.y - acc.m) + fexp(v2.z - acc.m) + fexp(v2.w - acc.m);
            s += fexp(v3.x - acc.m) + fexp(v3.y - acc.m) + fexp(v3.z - acc.m) + fexp(v3.w - acc.m);
            acc.s += s;
        }
        for (size_t i = h + (c4 << 2) + (size_t)lane; i < cols; i += TPR)
            if (xr[i] != -INFINITY) online_push(acc, xr[i]);
    }
    return acc;
}

// Second pass over a row: probabilities exp(x - l) written out; MODE 1 also returns this lane's part of the row's loss
// term sum_j -t_j * log(clamp(p_j)); GRAD 1 writes (p - t) / denom to the gradient row, GRAD 2 adds it.  Where the rows
// of all the arrays involved start at the same offset from a 16-byte boundary, the row is walked like row_online walks
// it (head, 16-byte pieces with four in flight per lane, tail); rows of fewer than 8 * TPR columns and rows that start at
// different offsets go value by value.  Each element's arithmetic is the same either way.
template <int TPR, int MODE, int GRAD>
__device__ __forceinline__ float row_probs(const float* xr, const float* tr, float* pr, float* gr, size_t cols, int lane,
                                           float l, float denom, bool fast) {
    float part = 0.f;
    auto element = [&](float x, float t, float g, float& p, float& d) {
        p = fast ? fexp(__fsub_rn(x, l)) : expf(__fsub_rn(x, l));
        if (MODE) {
            if (t != 0.f) {  // a zero target adds t * log(.) = 0: skipping it changes nothing and saves the log
                const float safe = fminf(fmaxf(p, 1e-7f), 1.0f - 1e-7f);
                part = __fsub_rn(part, __fmul_rn(t, logf(safe)));
            }
            if (GRAD) {
                d = __fdiv_rn(__fsub_rn(p, t), denom);
                if (GRAD == 2) d = __fadd_rn(g, d);
            }
        }
    };
    auto scalar = [&](size_t j) {
        float p, dd = 0.f;
        element(xr[j], MODE ? tr[j] : 0.f, GRAD == 2 ? gr[j] : 0.f, p, dd);
        pr[j] = p;
        if (GRAD) gr[j] = dd;
    };
    uintptr_t differ = reinterpret_cast<uintptr_t>(xr) ^ reinterpret_cast<uintptr_t>(pr);
    if (MODE) differ |= reinterpret_cast<uintptr_t>(xr) ^ reinterpret_cast<uintptr_t>(tr);
    if (GRAD) differ |= reinterpret_cast<uintptr_t>(xr) ^ reinterpret_cast<uintptr_t>(gr);
    if ((differ & 15u) != 0 || cols < (size_t)8 * TPR) {
        for (size_t j = lane; j < cols; j += TPR) scalar(j);
        return part;
    }
    const size_t h = row_head(xr, cols);
    for (size_t i = lane; i < h; i += TPR) scalar(i);
    const size_t c4 = (cols - h) >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(xr + h);
    const float4* t4 = reinterpret_cast<const float4*>(MODE ? tr + h : xr + h);
    float4* p4 = reinterpret_cast<float4*>(pr + h);
    float4* g4 = reinterpret_cast<float4*>(GRAD ? gr + h : pr + h);
    constexpr int U = 4;
    for (size_t j0 = lane; j0 < c4; j0 += (size_t)U * TPR) {
        float4 v[U], t[U], g[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t j = j0 + (size_t)u * TPR;
            if (j < c4) {
                v[u] = nt_load(x4 + j);
                if (MODE) t[u] = nt_load(t4 + j);
                if (GRAD == 2) g[u] = nt_load(g4 + j);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t j = j0 + (size_t)u * TPR;
            if (j < c4) {
                float4 p, dd = make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 tt = MODE ? t[u] : dd, gg = GRAD == 2 ? g[u] : dd;
                element(v[u].x, tt.x, gg.x, p.x, dd.x);
                element(v[u].y, tt.y, gg.y, p.y, dd.y);
                element(v[u].z, tt.z, gg.z, p.z, dd.z);
                element(v[u].w, tt.w, gg.w, p.w, dd.w);
                nt_store(p, p4 + j);
                if (GRAD) nt_store(dd, g4 + j);
            }
        }
    }
    for (size_t i = h + (c4 << 2) + (size_t)lane; i < cols; i += TPR) scalar(i);
    return part;
}

template <int TPR>
__device__ __forceinline__ OnlineAccT row_group_reduce(OnlineAccT acc, OnlineAccT* smem) {
    if (TPR <= kWave) return group_reduce<OnlineAcc, (TPR <= kWave ? TPR : kWave)>(acc);
    acc = block_reduce<OnlineAcc>(acc, smem);
    // broadcast wave 0's result to the whole workgroup
    __syncthreads();
    if (threadIdx.x == 0) smem[0] = acc;
    __syncthreads();
    return smem[0];
}

// integer labels: lse[row] and the row's loss term  -log(clamp(p_label, 1e-7, 1 - 1e-7))
template <int TPR>
__global__ __launch_bounds__(kBlock) void smce_label_fwd_kernel(const float* logits, const uint64_t* labels,
                                                                 float* lse, float* row_loss, size_t rows,
                                                                 size_t cols) {
    __shared__ OnlineAccT smem[kBlock / kWave];
    constexpr int kRows = kBlock / TPR;
    const int lane = threadIdx.x % TPR;
    const size_t row = (size_t)blockIdx.x * kRows + threadIdx.x / TPR;
    const bool live = row < rows;
    OnlineAccT acc = OnlineAcc::init();
    if (live) acc = row_online<TPR>(logits + row * cols, cols, lane);
    acc = row_group_reduce<TPR>(acc, smem);
    if (live && lane == 0) {
        const float l = __fadd_rn(acc.m, logf(acc.s));
        lse[row] = l;
        const uint64_t lab = labels[row];
        float term = 0.f;
        if (lab < cols) {
            float p = expf(__fsub_rn(logits[row * cols + lab], l));
            float safe = fminf(fmaxf(p, 1e-7f), 1.0f - 1e-7f);
            term = -logf(safe);
        }
        row_loss[row] = term;
    }
}

// grad (+)= (exp(x - lse[row]) - onehot) / rows, elementwise over the whole matrix, value by value: for operands that
// are not on 16-byte boundaries and rows of fewer than four columns.
template <bool ACC>
__global__ __launch_bounds__(kBlock) void smce_label_bwd_values_kernel(const float* logits, const uint64_t* labels,
                                                                        const float* lse, float* grad, size_t n,
                                                                        size_t cols, float denom) {
    const float inv_denom = __fdiv_rn(1.0f, denom);  // exact for power-of-two batch sizes, else within 1 ulp of x/denom
    const size_t nt = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += nt) {
        const size_t r = i / cols, c = i - r * cols;
        const float d = __fmul_rn(__fsub_rn(fexp(__fsub_rn(logits[i], lse[r])), (c == labels[r]) ? 1.f : 0.f), inv_denom);
        grad[i] = ACC ? __fadd_rn(grad[i], d) : d;
    }
}

// The same update with the matrix walked as one flat array: workgroup b owns float4 b*1024 .. b*1024+1023 of both
// streams, whatever rows they fall in (rows of at least 256 float4, so a piece crosses at most a few row ends).
// Chunks that start every 16 KiB and leave no short chunk at each row's end keep more DRAM pages open than the
// per-row chunks above: 570 -> 515 us for the accumulating form at [8192, 32000].
constexpr int kLabelBwdU = 4;
constexpr size_t kLabelBwdChunk = (size_t)kBlock * kLabelBwdU;
constexpr size_t kLabelBwdMinC4 = 256;
template <bool ACC>
__global__ __launch_bounds__(kBlock) void smce_label_bwd_flat_kernel(const float* logits, const uint64_t* labels,
                                                                      const float* lse, float* grad, size_t n4,
                                                                      size_t c4, float denom) {
    const float inv_denom = __fdiv_rn(1.0f, denom);
    const float4* x4 = reinterpret_cast<const float4*>(logits);
    float4* g4 = reinterpret_cast<float4*>(grad);
    for (size_t c0 = (size_t)blockIdx.x * kLabelBwdChunk; c0 < n4; c0 += (size_t)gridDim.x * kLabelBwdChunk) {
        const size_t r0 = c0 / c4, rem = c0 - r0 * c4;
        float4 v[kLabelBwdU], g[kLabelBwdU];
        float l[kLabelBwdU];
        uint64_t hit[kLabelBwdU];  // label minus the column of the piece's first element: 0..3 marks the one-hot entry
#pragma unroll
        for (int u = 0; u < kLabelBwdU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            size_t o = rem + threadIdx.x + (size_t)u * kBlock, r = r0;
            while (o >= c4) {
                o -= c4;
                r++;
            }
            if (j < n4) {
                v[u] = nt_load(x4 + j);
                if (ACC) g[u] = nt_load(g4 + j);
                l[u] = lse[r];
                hit[u] = labels[r] - 4 * o;  // wraps to a huge value when the label lies before this piece
            }
        }
#pragma unroll
        for (int u = 0; u < kLabelBwdU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            if (j < n4) {
                float d0 = __fmul_rn(__fsub_rn(fexp(__fsub_rn(v[u].x, l[u])), (hit[u] == 0) ? 1.f : 0.f), inv_denom);
                float d1 = __fmul_rn(__fsub_rn(fexp(__fsub_rn(v[u].y, l[u])), (hit[u] == 1) ? 1.f : 0.f), inv_denom);
                float d2 = __fmul_rn(__fsub_rn(fexp(__fsub_rn(v[u].z, l[u])), (hit[u] == 2) ? 1.f : 0.f), inv_denom);
                float d3 = __fmul_rn(__fsub_rn(fexp(__fsub_rn(v[u].w, l[u])), (hit[u] == 3) ? 1.f : 0.f), inv_denom);
                float4 o;
                o.x = ACC ? __fadd_rn(g[u].x, d0) : d0;
                o.y = ACC ? __fadd_rn(g[u].y, d1) : d1;
                o.z = ACC ? __fadd_rn(g[u].z, d2) : d2;
                o.w = ACC ? __fadd_rn(g[u].w, d3) : d3;
                nt_store(o, g4 + j);
            }
        }
    }
}


// The same for rows of any length of at least four columns (both matrices on 16-byte boundaries): the matrix is still
// walked as one flat array of 16-byte pieces, and a piece may end one row and begin the next, so a thread fetches lse
// and label of the row its piece starts in and of the one after, and each of the four values takes the pair of its own
// row.  The n % 4 values after the last whole piece are done one by one.  (One workgroup per row, the form this
// replaces, ran [1048576, 10] at 4 % of 8 TB/s and [8192, 50257] at 50 %.)
template <bool ACC>
__global__ __launch_bounds__(kBlock) void smce_label_bwd_any_kernel(const float* logits, const uint64_t* labels,
                                                                     const float* lse, float* grad, size_t n, size_t cols,
                                                                     size_t rows, float denom) {
    const float inv_denom = __fdiv_rn(1.0f, denom);
    const float4* x4 = reinterpret_cast<const float4*>(logits);
    float4* g4 = reinterpret_cast<float4*>(grad);
    const size_t n4 = n >> 2;
    for (size_t c0 = (size_t)blockIdx.x * kLabelBwdChunk; c0 < n4; c0 += (size_t)gridDim.x * kLabelBwdChunk) {
        const size_t e0 = c0 << 2, r0 = e0 / cols, rem = e0 - r0 * cols;
        float4 v[kLabelBwdU], g[kLabelBwdU];
        float l0[kLabelBwdU], l1[kLabelBwdU];
        uint64_t lab0[kLabelBwdU], lab1[kLabelBwdU];
        size_t col[kLabelBwdU];  // column of the piece's first value
#pragma unroll
        for (int u = 0; u < kLabelBwdU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            size_t o = rem + 4 * (threadIdx.x + (size_t)u * kBlock), r = r0;  // o < cols + 4 * kLabelBwdChunk
            if (cols >= 4 * kLabelBwdChunk) {
                if (o >= cols) {
                    o -= cols;
                    r++;
                }
            } else {
                const uint32_t q = (uint32_t)o / (uint32_t)cols;
                o -= (size_t)q * cols;
                r += q;
            }
            col[u] = o;
            if (j < n4) {
                const size_t r1 = r + 1 < rows ? r + 1 : r;
                v[u] = nt_load(x4 + j);
                if (ACC) g[u] = nt_load(g4 + j);
                l0[u] = lse[r];
                l1[u] = lse[r1];
                lab0[u] = labels[r];
                lab1[u] = labels[r1];
            }
        }
#pragma unroll
        for (int u = 0; u < kLabelBwdU; u++) {
            const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
            if (j < n4) {
                auto value = [&](float x, size_t c) {
                    const bool next = c >= cols;  // at most one row end inside a piece: cols >= 4
                    const float l = next ? l1[u] : l0[u];
                    const uint64_t lab = next ? lab1[u] : lab0[u];
                    const size_t cc = next ? c - cols : c;
                    return __fmul_rn(__fsub_rn(fexp(__fsub_rn(x, l)), (cc == lab) ? 1.f : 0.f), inv_denom);
                };
                const float d0 = value(v[u].x, col[u]), d1 = value(v[u].y, col[u] + 1), d2 = value(v[u].z, col[u] + 2),
                            d3 = value(v[u].w, col[u] + 3);
                float4 o;
                o.x = ACC ? __fadd_rn(g[u].x, d0) : d0;
                o.y = ACC ? __fadd_rn(g[u].y, d1) : d1;
                o.z = ACC ? __fadd_rn(g[u].z, d2) : d2;
                o.w = ACC ? __fadd_rn(g[u].w, d3) : d3;
                nt_store(o, g4 + j);
            }
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t i = (n4 << 2) + threadIdx.x, r = i / cols, c = i - r * cols;
        const float d = __fmul_rn(__fsub_rn(fexp(__fsub_rn(logits[i], lse[r])), (c == labels[r]) ? 1.f : 0.f), inv_denom);
        grad[i] = ACC ? __fadd_rn(grad[i], d) : d;
    }
}


// one-hot targets (the reference's form): probabilities are written out; the row's loss term is
// sum_j -t_j * log(clamp(p_j)).  MODE 0: softmax only (no target, no loss).
template <int TPR, int MODE>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(const float* logits, const float* target, float* probs,
                                                               float* row_loss, size_t rows, size_t cols) {
    __shared__ OnlineAccT smem[kBlock / kWave];
    __shared__ float lsum[kBlock / kWave];
    constexpr int kRows = kBlock / TPR;
    const int lane = threadIdx.x % TPR;
    const size_t row = (size_t)blockIdx.x * kRows + threadIdx.x / TPR;
    const bool live = row < rows;
    OnlineAccT acc = OnlineAcc::init();
    if (live) acc = row_online<TPR, true>(logits + row * cols, cols, lane);
    acc = row_group_reduce<TPR>(acc, smem);
    float part = 0.f;
    if (live) {
        const float l = __fadd_rn(acc.m, logf(acc.s));
        part = row_probs<TPR, MODE, 0>(logits + row * cols, MODE ? target + row * cols : nullptr, probs + row * cols,
                                       nullptr, cols, lane, l, 1.f, false);
    }
    if (MODE) {
        if (TPR <= kWave) {
            part = group_reduce<SumAcc, (TPR <= kWave ? TPR : kWave)>(part);
        } else {
            part = block_reduce<SumAcc>(part, lsum);
        }
        if (live && lane == 0) row_loss[row] = part;
    }
}

// Long rows (1028 to 32768 columns, 16-byte aligned): one workgroup of NT threads per row keeps the whole row in
// registers (at most VEC float4 per thread), so the logits are read from HBM once: max / sum-of-exponentials over
// the registers, one workgroup reduction, then the probabilities (and the loss terms) from the same registers.
// MODE 1 reads the target row as well; its loads are issued before the reduction so they are in flight under it.
// Three shapes by row length, so that a thread has several loads in flight and a compute unit several rows:
// 256 threads x 4 float4 up to 4096 columns, 256 x 8 up to 8192, 1024 x 8 beyond.
constexpr int kLongRowMaxThreads = 1024;
constexpr int kLongRowMaxVec = 8;
// GRAD (with MODE 1): 1 the loss's gradient (p - t) / denom is written to grad as well, 2 it is added to grad: the
// backward pass of the scalar loss in the same pass over the row (smce_bwd_kernel's arithmetic per element).
template <int kLongRowThreads, int kLongRowVec, int MODE, int GRAD = 0>
__global__ __launch_bounds__(kLongRowThreads) void softmax_long_rows_kernel(const float* logits, const float* target,
                                                                            float* probs, float* row_loss,
                                                                            size_t cols, float* grad = nullptr,
                                                                            float denom = 1.f) {
    __shared__ OnlineAccT smem[kLongRowThreads / kWave];
    __shared__ float lsum[kLongRowThreads / kWave];
    __shared__ OnlineAccT total_s;
    const size_t row = blockIdx.x;
    const size_t c4 = cols >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(logits + row * cols);
    const float4* t4 = reinterpret_cast<const float4*>(MODE ? target + row * cols : logits);
    float4* p4 = reinterpret_cast<float4*>(probs + row * cols);
    float4* g4 = reinterpret_cast<float4*>(GRAD ? grad + row * cols : probs);
    const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    float4 v[kLongRowVec], t[kLongRowVec];
#pragma unroll
    for (int u = 0; u < kLongRowVec; u++) {
        const size_t j = threadIdx.x + (size_t)u * kLongRowThreads;
        v[u] = (j < c4) ? nt_load(x4 + j) : ninf;
    }
    if (MODE) {
#pragma unroll
        for (int u = 0; u < kLongRowVec; u++) {
            const size_t j = threadIdx.x + (size_t)u * kLongRowThreads;
            t[u] = (j < c4) ? nt_load(t4 + j) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    OnlineAccT acc = OnlineAcc::init();
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < kLongRowVec; u++) mx = fmaxf(mx, fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)));
    if (mx != -INFINITY) {
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < kLongRowVec; u++)
            sum += fexp(v[u].x - mx) + fexp(v[u].y - mx) + fexp(v[u].z - mx) + fexp(v[u].w - mx);
        acc.m = mx;
        acc.s = sum;
    }
    // workgroup reduction: butterfly inside each wave, then the 16 wave results in wave order by every thread
    acc = group_reduce<OnlineAcc, kWave>(acc);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) smem[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        OnlineAccT tot = smem[0];
        for (int w = 1; w < kLongRowThreads / kWave; w++) tot = OnlineAcc::combine(tot, smem[w]);
        total_s = tot;
    }
    __syncthreads();
    const float l = __fadd_rn(total_s.m, logf(total_s.s));
    float part = 0.f;
#pragma unroll
    for (int u = 0; u < kLongRowVec; u++) {
        const size_t j = threadIdx.x + (size_t)u * kLongRowThreads;
        if (j < c4) {
            float4 p;
            p.x = fexp(__fsub_rn(v[u].x, l));
            p.y = fexp(__fsub_rn(v[u].y, l));
            p.z = fexp(__fsub_rn(v[u].z, l));
            p.w = fexp(__fsub_rn(v[u].w, l));
            nt_store(p, p4 + j);
            if (MODE) {
                const float pv[4] = {p.x, p.y, p.z, p.w}, tv[4] = {t[u].x, t[u].y, t[u].z, t[u].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (tv[e] != 0.f) {
                        const float safe = fminf(fmaxf(pv[e], 1e-7f), 1.0f - 1e-7f);
                        part = __fsub_rn(part, __fmul_rn(tv[e], logf(safe)));
                    }
                }
                if (GRAD) {
                    float4 d;
                    d.x = __fdiv_rn(__fsub_rn(p.x, t[u].x), denom);
                    d.y = __fdiv_rn(__fsub_rn(p.y, t[u].y), denom);
                    d.z = __fdiv_rn(__fsub_rn(p.z, t[u].z), denom);
                    d.w = __fdiv_rn(__fsub_rn(p.w, t[u].w), denom);
                    if (GRAD == 2) {
                        const float4 g = nt_load(g4 + j);
                        d.x = __fadd_rn(g.x, d.x);
                        d.y = __fadd_rn(g.y, d.y);
                        d.z = __fadd_rn(g.z, d.z);
                        d.w = __fadd_rn(g.w, d.w);
                    }
                    nt_store(d, g4 + j);
                }
            }
        }
    }
    if (MODE) {
        part = group_reduce<SumAcc, kWave>(part);
        if (lane == 0) lsum[wave] = part;
        __syncthreads();
        if (threadIdx.x == 0) {
            float tot = lsum[0];
            for (int w = 1; w < kLongRowThreads / kWave; w++) tot = __fadd_rn(tot, lsum[w]);
            row_loss[row] = tot;
        }
    }
}

// Rows of up to 1024 columns (the wide classifier's [4096, 1024] logits): TPR lanes of a wave per row (16 up to 256
// columns, a whole wave beyond) hold the row in registers (at most 4 float4 per lane), so the logits are read once and
// the row's reductions stay inside the wave: three passes of the matrix instead of four, no LDS, no barrier.
constexpr int kWaveRowVec = 4;
// RPG rows per lane group (1, 2 or 4): a row of at most TPR * 4 / RPG pieces leaves a lane's other registers to further
// rows, RPG of them loaded before the first is used.  With one piece per lane a workgroup of 16-lane groups moved 4 KiB
// per trip and the softmax of [4194304, 64] ran at 57 % of 8 TB/s.  The arithmetic of a row does not depend on RPG: the
// pieces a row does not have added exp(-inf) = 0 to its sum.
template <int TPR, int MODE, int GRAD = 0, int RPG = 1>
__global__ __launch_bounds__(kBlock) void softmax_wave_rows_kernel(const float* logits, const float* target, float* probs,
                                                                    float* row_loss, size_t rows, size_t cols,
                                                                    float* grad = nullptr, float denom = 1.f) {
    constexpr int PPL = kWaveRowVec / RPG;  // pieces per lane and row
    constexpr int kGroups = kBlock / TPR;
    const int lane = threadIdx.x & (TPR - 1);
    const size_t row0 = (size_t)blockIdx.x * (kGroups * RPG) + threadIdx.x / TPR;  // this group's rows: row0 + r * kGroups
    if (row0 >= rows) return;  // the lanes of a group leave together: no barrier follows, and shuffles stay inside it
    const size_t c4 = cols >> 2;
    const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    float4 v[kWaveRowVec], t[kWaveRowVec];
#pragma unroll
    for (int r = 0; r < RPG; r++) {
        const size_t row = row0 + (size_t)r * kGroups;
        const float4* x4 = reinterpret_cast<const float4*>(logits + row * cols);
#pragma unroll
        for (int u = 0; u < PPL; u++) {
            const size_t j = lane + (size_t)u * TPR;
            v[r * PPL + u] = (row < rows && j < c4) ? nt_load(x4 + j) : ninf;
        }
    }
    if (MODE) {
#pragma unroll
        for (int r = 0; r < RPG; r++) {
            const size_t row = row0 + (size_t)r * kGroups;
            const float4* t4 = reinterpret_cast<const float4*>(target + row * cols);
#pragma unroll
            for (int u = 0; u < PPL; u++) {
                const size_t j = lane + (size_t)u * TPR;
                t[r * PPL + u] = (row < rows && j < c4) ? nt_load(t4 + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RPG; r++) {
        const size_t row = row0 + (size_t)r * kGroups;
        const bool live = row < rows;  // the same for every lane of the group
        float4* p4 = reinterpret_cast<float4*>(probs + row * cols);
        float4* g4 = reinterpret_cast<float4*>(GRAD ? grad + row * cols : probs);
        OnlineAccT acc = OnlineAcc::init();
        float mx = -INFINITY;
#pragma unroll
        for (int u = 0; u < PPL; u++) {
            const float4 a = v[r * PPL + u];
            mx = fmaxf(mx, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)));
        }
        if (mx != -INFINITY) {
            float sum = 0.f;
#pragma unroll
            for (int u = 0; u < PPL; u++) {
                const float4 a = v[r * PPL + u];
                sum += fexp(a.x - mx) + fexp(a.y - mx) + fexp(a.z - mx) + fexp(a.w - mx);
            }
            acc.m = mx;
            acc.s = sum;
        }
        acc = group_reduce<OnlineAcc, TPR>(acc);
        const float l = __fadd_rn(acc.m, logf(acc.s));
        float part = 0.f;
#pragma unroll
        for (int u = 0; u < PPL; u++) {
            const size_t j = lane + (size_t)u * TPR;
            if (live && j < c4) {
                const float4 a = v[r * PPL + u];
                float4 p;
                p.x = fexp(__fsub_rn(a.x, l));
                p.y = fexp(__fsub_rn(a.y, l));
                p.z = fexp(__fsub_rn(a.z, l));
                p.w = fexp(__fsub_rn(a.w, l));
                nt_store(p, p4 + j);
                if (MODE) {
                    const float4 tt = t[r * PPL + u];
                    const float pv[4] = {p.x, p.y, p.z, p.w}, tv[4] = {tt.x, tt.y, tt.z, tt.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (tv[e] != 0.f) {
                            const float safe = fminf(fmaxf(pv[e], 1e-7f), 1.0f - 1e-7f);
                            part = __fsub_rn(part, __fmul_rn(tv[e], logf(safe)));
                        }
                    }
                    if (GRAD) {
                        float4 dd;
                        dd.x = __fdiv_rn(__fsub_rn(p.x, tt.x), denom);
                        dd.y = __fdiv_rn(__fsub_rn(p.y, tt.y), denom);
                        dd.z = __fdiv_rn(__fsub_rn(p.z, tt.z), denom);
                        dd.w = __fdiv_rn(__fsub_rn(p.w, tt.w), denom);
                        if (GRAD == 2) {
                            const float4 g = nt_load(g4 + j);
                            dd.x = __fadd_rn(g.x, dd.x);
                            dd.y = __fadd_rn(g.y, dd.y);
                            dd.z = __fadd_rn(g.z, dd.z);
                            dd.w = __fadd_rn(g.w, dd.w);
                        }
                        nt_store(dd, g4 + j);
                    }
                }
            }
        }
        if (MODE) {
            part = group_reduce<SumAcc, TPR>(part);
            if (live && lane == 0) row_loss[row] = part;
        }
    }
}

// A handful of very long rows (fewer than two per compute unit, rows of 65536 columns and more): a workgroup per row would
// leave most of the machine idle (32 rows of 1048576 columns: 7 % of 8 TB/s), so a row is cut into segments.  First
// launch: workgroup (s, r) forms the running maximum and sum of segment s of row r (row_online, which places its
// 16-byte pieces by the segment's own address) and leaves it at acc[r * n_seg + s].
__global__ __launch_bounds__(kBlock) void softmax_seg_online_kernel(const float* logits, OnlineAccT* acc_out, size_t cols,
                                                                     size_t seg, int n_seg) {
    __shared__ OnlineAccT smem[kBlock / kWave];
    const size_t s = blockIdx.x, row = blockIdx.y;
    const size_t c0 = s * seg, c1 = c0 + seg < cols ? c0 + seg : cols;
    OnlineAccT acc = row_online<kBlock, true>(logits + row * cols + c0, c1 - c0, threadIdx.x);
    acc = block_reduce<OnlineAcc>(acc, smem);
    if (threadIdx.x == 0) acc_out[row * n_seg + s] = acc;
}

// A row's segments (at most one per thread) combined by the workgroup in the fixed order of its reduction tree: log of
// the sum of the row's exponentials, in every thread.
__device__ __forceinline__ float seg_row_lse(const OnlineAccT* acc, size_t row, int n_seg, OnlineAccT* smem) {
    OnlineAccT a = (int)threadIdx.x < n_seg ? acc[row * n_seg + threadIdx.x] : OnlineAcc::init();
    a = row_group_reduce<kBlock>(a, smem);
    return __fadd_rn(a.m, logf(a.s));
}

// Second launch: workgroup (s, r) writes the probabilities of its segment (row_probs) and, MODE 1, leaves the segment's
// part of the row's loss term at seg_loss[r * n_seg + s].
template <int MODE>
__global__ __launch_bounds__(kBlock) void softmax_seg_probs_kernel(const float* logits, const float* target, float* probs,
                                                                    const OnlineAccT* acc, float* seg_loss, size_t cols,
                                                                    size_t seg, int n_seg) {
    __shared__ float lsum[kBlock / kWave];
    __shared__ OnlineAccT smem[kBlock / kWave];
    const size_t s = blockIdx.x, row = blockIdx.y;
    const size_t c0 = s * seg, c1 = c0 + seg < cols ? c0 + seg : cols;
    const float l = seg_row_lse(acc, row, n_seg, smem);
    const size_t o = row * cols + c0;
    float part = row_probs<kBlock, MODE, 0>(logits + o, MODE ? target + o : nullptr, probs + o, nullptr, c1 - c0,
                                            threadIdx.x, l, 1.f, false);
    if (MODE) {
        part = block_reduce<SumAcc>(part, lsum);
        if (threadIdx.x == 0) seg_loss[row * n_seg + s] = part;
    }
}

// Integer labels: lse[row] and the row's loss term from the row's segments, a workgroup per row.
__global__ __launch_bounds__(kBlock) void label_seg_final_kernel(const float* logits, const uint64_t* labels,
                                                                  const OnlineAccT* acc, float* lse, float* row_loss,
                                                                  size_t rows, size_t cols, int n_seg) {
    __shared__ OnlineAccT smem[kBlock / kWave];
    const size_t row = blockIdx.x;
    const float l = seg_row_lse(acc, row, n_seg, smem);
    if (threadIdx.x != 0) return;
    lse[row] = l;
    const uint64_t lab = labels[row];
    float term = 0.f;
    if (lab < cols) {
        const float p = expf(__fsub_rn(logits[row * cols + lab], l));
        const float safe = fminf(fmaxf(p, 1e-7f), 1.0f - 1e-7f);
        term = -logf(safe);
    }
    row_loss[row] = term;
}

// Segments for `rows` long rows: about two workgroups per compute unit, segments of at least 16384 columns (a multiple of
// 1024), at most one per thread of a workgroup.  0: the rows are not cut.
static int row_segments_for(const zg_hip_ctx* ctx, size_t rows, size_t cols, size_t* seg_out) {
    if (rows >= 2 * (size_t)ctx->n_cu || cols < 65536) return 0;
    size_t n_seg = ceil_div_sz(2 * (size_t)ctx->n_cu, rows);
    if (n_seg > (size_t)kBlock) n_seg = kBlock;
    size_t seg = ceil_div_sz(ceil_div_sz(cols, n_seg), 1024) * 1024;
    if (seg < 16384) seg = 16384;
    n_seg = ceil_div_sz(cols, seg);
    *seg_out = seg;
    return n_seg >= 2 ? (int)n_seg : 0;
}

static bool wave_row_ok(const float* a, const float* b, const float* c, size_t rows, size_t cols) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c);
    return cols <= (size_t)kWave * kWaveRowVec * 4 && cols % 4 == 0 && (bits & 15u) == 0 && rows <= 0x7fffffffull;
}

static bool long_row_ok(const float* a, const float* b, const float* c, size_t rows, size_t cols) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c);
    return cols > 1024 && cols % 4 == 0 && cols <= (size_t)kLongRowMaxThreads * kLongRowMaxVec * 4 && (bits & 15u) == 0 &&
           rows <= 0x7fffffffull;
}

// Launches softmax_wave_rows_kernel<.., MODE, GRAD> with the lanes per row that fit the row length (wave_row_ok holds).
#define ZG_WAVE_ROWS_AS(TPR_, RPG_, MODE, GRAD, ...)                                                                  \
    hipLaunchKernelGGL((softmax_wave_rows_kernel<TPR_, MODE, GRAD, RPG_>),                                             \
                       dim3((unsigned)ceil_div_sz(rows, (size_t)(kBlock / TPR_) * RPG_)), dim3(kBlock), 0, ctx->stream, \
                       __VA_ARGS__)
#define ZG_WAVE_ROWS(MODE, GRAD, ...)                                                                                  \
    do { /* the lanes per row of pick_tpr, which the one-workgroup kernel for small batches follows; rows that leave */ \
        /* registers free share a lane group two or four at a time where that still leaves a thousand workgroups */     \
        /* ([4096, 64] on 64 workgroups instead of 256: 6.9 -> 8.8 us) */                                              \
        const bool many = rows >= 65536;                                                                               \
        if (cols <= 16 && rows >= 4 * 65536) ZG_WAVE_ROWS_AS(4, 4, MODE, GRAD, __VA_ARGS__);                           \
        else if (cols <= 32 && rows >= 2 * 65536) ZG_WAVE_ROWS_AS(4, 2, MODE, GRAD, __VA_ARGS__);                      \
        else if (cols <= 32) ZG_WAVE_ROWS_AS(4, 1, MODE, GRAD, __VA_ARGS__);                                           \
        else if (cols <= 64 && many) ZG_WAVE_ROWS_AS(16, 4, MODE, GRAD, __VA_ARGS__);                                  \
        else if (cols <= 128 && many) ZG_WAVE_ROWS_AS(16, 2, MODE, GRAD, __VA_ARGS__);                                 \
        else if (cols <= 16 * kWaveRowVec * 4) ZG_WAVE_ROWS_AS(16, 1, MODE, GRAD, __VA_ARGS__);                        \
        else if (cols <= 512 && rows >= 8192) ZG_WAVE_ROWS_AS(kWave, 2, MODE, GRAD, __VA_ARGS__);                      \
        else ZG_WAVE_ROWS_AS(kWave, 1, MODE, GRAD, __VA_ARGS__);                                                       \
    } while (0)

// Launches softmax_long_rows_kernel<.., MODE, GRAD> in the shape that fits the row length (long_row_ok holds).
#define ZG_LONG_ROWS(MODE, GRAD, ...)                                                                                  \
    do {                                                                                                               \
        if (cols <= 4096)                                                                                              \
            hipLaunchKernelGGL((softmax_long_rows_kernel<256, 4, MODE, GRAD>), dim3((unsigned)rows), dim3(256), 0, ctx->stream, \
                               __VA_ARGS__);                                                                           \
        else if (cols <= 8192)                                                                                         \
            hipLaunchKernelGGL((softmax_long_rows_kernel<256, 8, MODE, GRAD>), dim3((unsigned)rows), dim3(256), 0, ctx->stream, \
                               __VA_ARGS__);                                                                           \
        else                                                                                                           \
            hipLaunchKernelGGL((softmax_long_rows_kernel<1024, 8, MODE, GRAD>), dim3((unsigned)rows), dim3(1024), 0,   \
                               ctx->stream, __VA_ARGS__);                                                              \
    } while (0)

// src/nn/loss.zig:150-159.  ACC false: the gradient is written, not accumulated (same values as accumulating
// into zeros, without reading them).
// A workgroup owns kSmceBwdChunk consecutive float4 of every stream (16 KiB each) and has all of them in flight
// before its first store: with three or four streams, consecutive workgroups on consecutive chunks keep the
// DRAM pages of each stream open far better than a grid-stride walk does (4.6 -> 5.9 TB/s on four streams).
constexpr int kSmceBwdU = 4;
constexpr size_t kSmceBwdChunk = (size_t)kBlock * kSmceBwdU;
constexpr size_t kSmceBwdMaxGrid = 0x7fffffffull;
template <bool ACC>
__global__ __launch_bounds__(kBlock) void smce_bwd_kernel(const float* probs, const float* target, float* grad, size_t n,
                                                           float denom) {
    const bool vec = ((reinterpret_cast<uintptr_t>(probs) | reinterpret_cast<uintptr_t>(target) |
                       reinterpret_cast<uintptr_t>(grad)) & 15u) == 0;
    auto term = [&](float g, float p, float t) {
        const float d = __fdiv_rn(__fsub_rn(p, t), denom);
        return ACC ? __fadd_rn(g, d) : d;
    };
    if (vec) {
        const size_t n4 = n >> 2;
        const float4* p4 = reinterpret_cast<const float4*>(probs);
        const float4* t4 = reinterpret_cast<const float4*>(target);
        float4* g4 = reinterpret_cast<float4*>(grad);
        const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
        for (size_t c0 = (size_t)blockIdx.x * kSmceBwdChunk; c0 < n4; c0 += (size_t)gridDim.x * kSmceBwdChunk) {
            float4 p[kSmceBwdU], t[kSmceBwdU], g[kSmceBwdU];
#pragma unroll
            for (int u = 0; u < kSmceBwdU; u++) {
                const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
                g[u] = zero4;
                if (j < n4) {
                    p[u] = nt_load(p4 + j);
                    t[u] = nt_load(t4 + j);
                    if (ACC) g[u] = nt_load(g4 + j);
                }
            }
#pragma unroll
            for (int u = 0; u < kSmceBwdU; u++) {
                const size_t j = c0 + threadIdx.x + (size_t)u * kBlock;
                if (j < n4) {
                    float4 o;
                    o.x = term(g[u].x, p[u].x, t[u].x);
                    o.y = term(g[u].y, p[u].y, t[u].y);
                    o.z = term(g[u].z, p[u].z, t[u].z);
                    o.w = term(g[u].w, p[u].w, t[u].w);
                    nt_store(o, g4 + j);
                }
            }
        }
        const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x, nt = (size_t)gridDim.x * kBlock;
        for (size_t j = (n4 << 2) + i; j < n; j += nt) grad[j] = term(ACC ? grad[j] : 0.f, probs[j], target[j]);
    } else {
        const size_t nt = (size_t)gridDim.x * kBlock;
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += nt)
            grad[i] = term(ACC ? grad[i] : 0.f, probs[i], target[i]);
    }
}

static unsigned smce_bwd_grid(size_t n) {
    size_t blocks = ceil_div_sz(n, kSmceBwdChunk * 4);
    if (blocks > kSmceBwdMaxGrid) blocks = kSmceBwdMaxGrid;
    return (unsigned)(blocks ? blocks : 1);
}

// smce_fwd and the loss's backward (upstream gradient 1) of a batch small enough for one workgroup, in one launch:
// kFlatSingle / TPR rows of at most 4096 columns (rows of more than 1024 columns that the register-resident row kernels
// take go there instead: 8 x 4096 21 us here, 7.7 us through them and the reduction of the row terms).  Per row the
// arithmetic is that of the row kernel a larger batch of such rows takes (softmax_rows_kernel, or the lanes-per-row
// kernel with its exponential), per gradient element smce_bwd_kernel's, and the mean over the rows is formed as
// flat_single_kernel forms it.  GRAD: 0 no gradient (smce_fwd alone), 1 written, 2 added to.
template <int TPR, int GRAD>
__global__ __launch_bounds__(kFlatSingle) void smce_small_kernel(const float* logits, const float* target, float* probs,
                                                                 float* loss, float* grad, size_t rows, size_t cols) {
    static_assert(TPR <= kWave, "a row is reduced inside one wave");
    __shared__ __align__(16) float row_loss[kFlatSingle / TPR];
    __shared__ float smem[kFlatSingle / kWave];
    const int lane = threadIdx.x % TPR;
    const size_t row = threadIdx.x / TPR;
    const bool live = row < rows;
    const float denom = (float)rows;
    OnlineAccT acc = OnlineAcc::init();
    if (live) acc = row_online<TPR, true>(logits + row * cols, cols, lane);
    acc = group_reduce<OnlineAcc, TPR>(acc);
    float part = 0.f;
    // rows the register-resident kernels take in a larger batch (wave_row_ok) get their exponential, so that a row's
    // probabilities do not depend on the size of the batch it arrives in
    const bool fast = cols % 4 == 0 && ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(target) |
                                         reinterpret_cast<uintptr_t>(probs)) & 15u) == 0;
    if (live) {
        const float l = __fadd_rn(acc.m, logf(acc.s));
        part = row_probs<TPR, 1, GRAD>(logits + row * cols, target + row * cols, probs + row * cols,
                                       GRAD ? grad + row * cols : nullptr, cols, lane, l, denom, fast);
    }
    part = group_reduce<SumAcc, TPR>(part);
    if (live && lane == 0) row_loss[row] = part;
    __syncthreads();
    float s = flat_accumulate<TermId, 1>(row_loss, nullptr, rows, 0.f, threadIdx.x, blockDim.x);
    s = block_reduce<SumAcc>(s, smem);
    if (threadIdx.x == 0) FinDivN{loss, denom}(s);
}

// The two passes of the softmax backward over one row (or one segment of a row) of `cols` values, TPR lanes on it.
// Rows of the three operands that start at the same offset from a 16-byte boundary are walked in 16-byte pieces, the
// values before the first boundary and after the last whole piece dealt to the lanes one by one (rows of 32001 columns
// value by value: 31 % of 8 TB/s); rows of fewer than eight pieces per lane and rows at different offsets go value by
// value.
template <int TPR>
__device__ __forceinline__ bool bwd_row_in_pieces(const float* yr, const float* gr, const float* xr, size_t cols) {
    return cols >= (size_t)8 * TPR && (((reinterpret_cast<uintptr_t>(yr) ^ reinterpret_cast<uintptr_t>(gr)) |
                                        (reinterpret_cast<uintptr_t>(yr) ^ reinterpret_cast<uintptr_t>(xr))) & 15u) == 0;
}
// this lane's part of sum_j y_j * y_g_j
template <int TPR>
__device__ __forceinline__ float bwd_row_dot(const float* yr, const float* gr, size_t cols, int lane, bool pieces) {
    float part = 0.f;
    if (!pieces) {
        for (size_t j = lane; j < cols; j += TPR) part = __fadd_rn(part, __fmul_rn(yr[j], gr[j]));
        return part;
    }
    const size_t h = row_head(yr, cols), c4 = (cols - h) >> 2;
    const float4* y4 = reinterpret_cast<const float4*>(yr + h);
    const float4* q4 = reinterpret_cast<const float4*>(gr + h);
    auto dot4 = [](float4 a, float4 b) {
        return __fadd_rn(__fadd_rn(__fmul_rn(a.x, b.x), __fmul_rn(a.y, b.y)), __fadd_rn(__fmul_rn(a.z, b.z), __fmul_rn(a.w, b.w)));
    };
    for (size_t i = lane; i < h; i += TPR) part = __fadd_rn(part, __fmul_rn(yr[i], gr[i]));
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (size_t j = lane; j < c4; j += 4 * TPR) {
        const bool in1 = j + TPR < c4, in2 = j + 2 * TPR < c4, in3 = j + 3 * TPR < c4;
        // plain loads: the second pass reads both rows again
        const float4 a0 = y4[j], b0 = q4[j];
        const float4 a1 = in1 ? y4[j + TPR] : zero, b1 = in1 ? q4[j + TPR] : zero;
        const float4 a2 = in2 ? y4[j + 2 * TPR] : zero, b2 = in2 ? q4[j + 2 * TPR] : zero;
        const float4 a3 = in3 ? y4[j + 3 * TPR] : zero, b3 = in3 ? q4[j + 3 * TPR] : zero;
        s0 = __fadd_rn(s0, dot4(a0, b0));
        s1 = __fadd_rn(s1, dot4(a1, b1));
        s2 = __fadd_rn(s2, dot4(a2, b2));
        s3 = __fadd_rn(s3, dot4(a3, b3));
    }
    part = __fadd_rn(part, __fadd_rn(__fadd_rn(s0, s1), __fadd_rn(s2, s3)));
    for (size_t i = h + (c4 << 2) + (size_t)lane; i < cols; i += TPR) part = __fadd_rn(part, __fmul_rn(yr[i], gr[i]));
    return part;
}
// x_g += y * (y_g - dot) over the row
template <int TPR>
__device__ __forceinline__ void bwd_row_apply(const float* yr, const float* gr, float* xr, size_t cols, int lane, float dot,
                                              bool pieces) {
    if (!pieces) {
        for (size_t j = lane; j < cols; j += TPR) xr[j] = __fadd_rn(xr[j], __fmul_rn(yr[j], __fsub_rn(gr[j], dot)));
        return;
    }
    const size_t h = row_head(yr, cols), c4 = (cols - h) >> 2;
    const float4* y4 = reinterpret_cast<const float4*>(yr + h);
    const float4* q4 = reinterpret_cast<const float4*>(gr + h);
    float4* x4 = reinterpret_cast<float4*>(xr + h);
    for (size_t i = lane; i < h; i += TPR) xr[i] = __fadd_rn(xr[i], __fmul_rn(yr[i], __fsub_rn(gr[i], dot)));
    for (size_t j0 = lane; j0 < c4; j0 += 2 * TPR) {
        const size_t j1 = j0 + TPR;
        const bool in1 = j1 < c4;
        const float4 a0 = nt_load(y4 + j0), b0 = nt_load(q4 + j0), x0 = nt_load(x4 + j0);
        float4 a1 = a0, b1 = b0, x1 = x0;
        if (in1) {
            a1 = nt_load(y4 + j1);
            b1 = nt_load(q4 + j1);
            x1 = nt_load(x4 + j1);
        }
        auto upd = [&](float4 a, float4 b, float4 x) {
            float4 o;
            o.x = __fadd_rn(x.x, __fmul_rn(a.x, __fsub_rn(b.x, dot)));
            o.y = __fadd_rn(x.y, __fmul_rn(a.y, __fsub_rn(b.y, dot)));
            o.z = __fadd_rn(x.z, __fmul_rn(a.z, __fsub_rn(b.z, dot)));
            o.w = __fadd_rn(x.w, __fmul_rn(a.w, __fsub_rn(b.w, dot)));
            return o;
        };
        nt_store(upd(a0, b0, x0), x4 + j0);
        if (in1) nt_store(upd(a1, b1, x1), x4 + j1);
    }
    for (size_t i = h + (c4 << 2) + (size_t)lane; i < cols; i += TPR)
        xr[i] = __fadd_rn(xr[i], __fmul_rn(yr[i], __fsub_rn(gr[i], dot)));
}

// src/nn/loss.zig:232-245: x_g += y * (y_g - sum_j y_j * y_g_j) per row
template <int TPR>
__global__ __launch_bounds__(kBlock) void softmax_bwd_kernel(const float* y, const float* y_g, float* x_g, size_t rows,
                                                              size_t cols) {
    __shared__ float smem[kBlock / kWave];
    __shared__ float bcast;
    constexpr int kRows = kBlock / TPR;
    const int lane = threadIdx.x % TPR;
    const size_t row = (size_t)blockIdx.x * kRows + threadIdx.x / TPR;
    const bool live = row < rows;
    const float* yr = y + row * cols;
    const float* gr = y_g + row * cols;
    float* xr = x_g + row * cols;
    const bool pieces = live && bwd_row_in_pieces<TPR>(yr, gr, xr, cols);
    float part = live ? bwd_row_dot<TPR>(yr, gr, cols, lane, pieces) : 0.f;
    if (TPR <= kWave) {
        part = group_reduce<SumAcc, (TPR <= kWave ? TPR : kWave)>(part);
    } else {
        part = block_reduce<SumAcc>(part, smem);
        __syncthreads();
        if (threadIdx.x == 0) bcast = part;
        __syncthreads();
        part = bcast;
    }
    if (live) bwd_row_apply<TPR>(yr, gr, xr, cols, lane, part, pieces);
}

// A handful of very long rows, cut into segments like the forward kernels cut them: the first launch leaves each
// segment's part of the row's sum at dots[r * n_seg + s], the second adds a row's parts up in a workgroup (the fixed order
// of its reduction tree) and updates its segment.
__global__ __launch_bounds__(kBlock) void softmax_bwd_seg_dot_kernel(const float* y, const float* y_g, const float* x_g,
                                                                      float* dots, size_t cols, size_t seg, int n_seg) {
    __shared__ float smem[kBlock / kWave];
    const size_t s = blockIdx.x, row = blockIdx.y;
    const size_t c0 = s * seg, c1 = c0 + seg < cols ? c0 + seg : cols, o = row * cols + c0;
    const bool pieces = bwd_row_in_pieces<kBlock>(y + o, y_g + o, x_g + o, c1 - c0);
    float part = bwd_row_dot<kBlock>(y + o, y_g + o, c1 - c0, threadIdx.x, pieces);
    part = block_reduce<SumAcc>(part, smem);
    if (threadIdx.x == 0) dots[row * n_seg + s] = part;
}
__global__ __launch_bounds__(kBlock) void softmax_bwd_seg_apply_kernel(const float* y, const float* y_g, float* x_g,
                                                                        const float* dots, size_t cols, size_t seg,
                                                                        int n_seg) {
    __shared__ float smem[kBlock / kWave];
    __shared__ float bcast;
    const size_t s = blockIdx.x, row = blockIdx.y;
    const size_t c0 = s * seg, c1 = c0 + seg < cols ? c0 + seg : cols, o = row * cols + c0;
    float dot = (int)threadIdx.x < n_seg ? dots[row * n_seg + threadIdx.x] : 0.f;
    dot = block_reduce<SumAcc>(dot, smem);
    __syncthreads();
    if (threadIdx.x == 0) bcast = dot;
    __syncthreads();
    dot = bcast;
    const bool pieces = bwd_row_in_pieces<kBlock>(y + o, y_g + o, x_g + o, c1 - c0);
    bwd_row_apply<kBlock>(y + o, y_g + o, x_g + o, c1 - c0, threadIdx.x, dot, pieces);
}

// The same with the rows of y and y_g held in registers (16-byte aligned rows of up to 32768 columns): NT threads per row
// (lanes of a wave up to 1024 columns, a workgroup beyond), at most VEC float4 of each operand per thread, all loads of
// the row in flight at once: one pass over the three operands instead of two passes of single values.
template <int NT, int VEC>
__global__ __launch_bounds__(NT <= kWave ? kBlock : NT) void softmax_bwd_rows_kernel(const float* y, const float* y_g,
                                                                                      float* x_g, size_t rows, size_t cols) {
    constexpr int kThreads = NT <= kWave ? kBlock : NT;
    __shared__ float smem[kThreads / kWave];
    __shared__ float bcast;
    const int lane = threadIdx.x % NT;
    const size_t row = (size_t)blockIdx.x * (kThreads / NT) + threadIdx.x / NT;
    const bool live = row < rows;  // a workgroup per row (NT > 64) is always live: every thread reaches the barriers
    const size_t c4 = cols >> 2;
    const float4* a4 = reinterpret_cast<const float4*>(y + (live ? row : 0) * cols);
    const float4* b4 = reinterpret_cast<const float4*>(y_g + (live ? row : 0) * cols);
    float4* g4 = reinterpret_cast<float4*>(x_g + (live ? row : 0) * cols);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 a[VEC], b[VEC], g[VEC];
#pragma unroll
    for (int u = 0; u < VEC; u++) {
        const size_t j = lane + (size_t)u * NT;
        const bool in = live && j < c4;
        a[u] = in ? nt_load(a4 + j) : zero;
        b[u] = in ? nt_load(b4 + j) : zero;
        g[u] = in ? nt_load(g4 + j) : zero;
    }
    float part = 0.f;
#pragma unroll
    for (int u = 0; u < VEC; u++) {
        part = __fadd_rn(part, __fmul_rn(a[u].x, b[u].x));
        part = __fadd_rn(part, __fmul_rn(a[u].y, b[u].y));
        part = __fadd_rn(part, __fmul_rn(a[u].z, b[u].z));
        part = __fadd_rn(part, __fmul_rn(a[u].w, b[u].w));
    }
    if (NT <= kWave) {
        part = group_reduce<SumAcc, (NT <= kWave ? NT : kWave)>(part);
    } else {
        part = block_reduce<SumAcc>(part, smem);
        __syncthreads();
        if (threadIdx.x == 0) bcast = part;
        __syncthreads();
        part = bcast;
    }
#pragma unroll
    for (int u = 0; u < VEC; u++) {
        const size_t j = lane + (size_t)u * NT;
        if (live && j < c4) {
            float4 o;
            o.x = __fadd_rn(g[u].x, __fmul_rn(a[u].x, __fsub_rn(b[u].x, part)));
            o.y = __fadd_rn(g[u].y, __fmul_rn(a[u].y, __fsub_rn(b[u].y, part)));
            o.z = __fadd_rn(g[u].z, __fmul_rn(a[u].z, __fsub_rn(b[u].z, part)));
            o.w = __fadd_rn(g[u].w, __fmul_rn(a[u].w, __fsub_rn(b[u].w, part)));
            nt_store(o, g4 + j);
        }
    }
}

static int pick_tpr(size_t cols) {
    if (cols <= 32) return 4;
    if (cols <= 256) return 16;
    if (cols <= 4096) return 64;
    return 256;
}

// The integer-label forward has no other kernel whose rows its own must equal, so short rows get fewer lanes: the
// combining of running maxima and sums across lanes (two exponentials a step) is most of a short row's work.
static int label_tpr(size_t rows, size_t cols) {
    // ([3355443, 10]: 96 -> 51 us, [524288, 64]: 75 -> 39 us, [262144, 128]: 43 -> 31 us, [32768, 1000]: 31 -> 28 us);
    // only where that still leaves a thousand workgroups ([1000, 1000] on 63 instead of 250: 7.0 -> 8.6 us)
    const int few = cols < 16 ? 1 : cols < 32 ? 2 : cols < 96 ? 4 : cols < 512 ? 8 : cols <= 1024 ? 16 : pick_tpr(cols);
    const int usual = pick_tpr(cols);
    return (few < usual && rows / (size_t)(kBlock / few) >= 1024) ? few : usual;
}

#define ZG_TPR_DISPATCH(tpr, CALL) \
    switch (tpr) {                 \
        case 1: { constexpr int T = 1; CALL; } break;     \
        case 2: { constexpr int T = 2; CALL; } break;     \
        case 8: { constexpr int T = 8; CALL; } break;     \
        case 4: { constexpr int T = 4; CALL; } break;     \
        case 16: { constexpr int T = 16; CALL; } break;   \
        case 64: { constexpr int T = 64; CALL; } break;   \
        default: { constexpr int T = 256; CALL; } break;  \
    }

// Scratch of the entry point that allocates nothing (zg_hip_smce_label_fwd_noalloc): the per-row loss terms, then
// the per-workgroup partials of their sum.  One copy per GPU for the life of the process; every call on a GPU uses
// it, so calls that overlap on one GPU race.  Nothing in it has to start at zero: each call writes every entry it
// later reads.
constexpr size_t kNoAllocMaxRows = (size_t)1 << 18;
constexpr size_t kNoAllocRowBytes = kNoAllocMaxRows * sizeof(float);
constexpr size_t kNoAllocBytes = kNoAllocRowBytes + kMaxPartials * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kNoAllocBytes];

// `scratch` is a host-side stand-in in host code, not a device address: the address on the current device is
// looked up once per context (zg_hip_init calls this with the context's device current) and used from then on.
int noalloc_setup(zg_hip_ctx* ctx) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        set_error("init: hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
        return ZG_HIP_ERUNTIME;
    }
    ctx->noalloc_scratch = p;
    ctx->noalloc_scratch_bytes = kNoAllocBytes;
    return ZG_HIP_OK;
}

static int check_rows(const char* name, size_t rows, size_t cols) {
    ZG_REQUIRE(rows > 0 && cols > 0, "%s: empty matrix (%zu x %zu)", name, rows, cols);
    ZG_REQUIRE(rows <= 0x7fffffffull * 64, "%s: too many rows", name);
    return ZG_HIP_OK;
}

}  // namespace zg

using namespace zg;

ZG_API int zg_hip_smce_label_fwd(zg_hip_ctx* ctx, const float* logits, const uint64_t* labels, float* lse, float* loss,
                                 size_t rows, size_t cols) {
    ZG_CTX(ctx);
    ZG_REQUIRE(logits && labels && lse && loss, "smce_label_fwd: null pointer");
    if (int rc = check_rows("smce_label_fwd", rows, cols)) return rc;
    size_t seg = 0;
    if (const int n_seg = row_segments_for(ctx, rows, cols, &seg)) {
        char* mem = (char*)workspace(ctx, rows * sizeof(float) + rows * n_seg * sizeof(OnlineAccT));
        if (!mem) return ZG_HIP_EOOM;
        OnlineAccT* acc = (OnlineAccT*)mem;
        float* row_loss = (float*)(mem + rows * n_seg * sizeof(OnlineAccT));
        hipLaunchKernelGGL(softmax_seg_online_kernel, dim3((unsigned)n_seg, (unsigned)rows), dim3(kBlock), 0, ctx->stream,
                           logits, acc, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(label_seg_final_kernel, dim3((unsigned)rows), dim3(kBlock), 0, ctx->stream,
                           logits, labels, acc, lse, row_loss, rows, cols, n_seg);
        ZG_LAUNCH_CHECK();
        return flat_reduce<TermId, 1>(ctx, row_loss, nullptr, rows, 0.f, FinDivN{loss, (float)rows});
    }
    float* row_loss = (float*)workspace(ctx, rows * sizeof(float));
    if (!row_loss) return ZG_HIP_EOOM;
    const int tpr = label_tpr(rows, cols);
    const unsigned grid = (unsigned)ceil_div_sz(rows, kBlock / tpr);
    ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((smce_label_fwd_kernel<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, logits,
                                            labels, lse, row_loss, rows, cols));
    ZG_LAUNCH_CHECK();
    return flat_reduce<TermId, 1>(ctx, row_loss, nullptr, rows, 0.f, FinDivN{loss, (float)rows});
}

ZG_API int zg_hip_smce_label_fwd_noalloc(zg_hip_ctx* ctx, const float* logits, const uint64_t* labels, float* lse,
                                         float* loss, size_t rows, size_t cols) {
    // work that earlier calls left waiting is launched by ZG_CTX below, without an allocation (a waiting product reserved
    // its workspace when it was queued): the count of driver allocations is compared before any kernel of this call is
    // queued, so a call that reports a difference has launched nothing of its own
    const uint64_t allocs_before = ctx ? ctx->n_device_allocs : 0;
    ZG_CTX(ctx);
    if (ctx->n_device_allocs != allocs_before) {
        set_error("smce_label_fwd_noalloc: %llu driver allocation(s) were made while waiting work was launched",
                  (unsigned long long)(ctx->n_device_allocs - allocs_before));
        return ZG_HIP_ERUNTIME;
    }
    ZG_REQUIRE(logits && labels && lse && loss, "smce_label_fwd_noalloc: null pointer");
    if (int rc = check_rows("smce_label_fwd_noalloc", rows, cols)) return rc;
    ZG_REQUIRE(rows <= kNoAllocMaxRows, "smce_label_fwd_noalloc: %zu rows exceed the fixed scratch (at most %zu rows)",
               rows, kNoAllocMaxRows);
    ZG_REQUIRE(ctx->noalloc_scratch != nullptr, "smce_label_fwd_noalloc: the context has no scratch address");
    float* row_loss = (float*)ctx->noalloc_scratch;
    void* partials = (char*)ctx->noalloc_scratch + kNoAllocRowBytes;
    const int tpr = label_tpr(rows, cols);
    const unsigned grid = (unsigned)ceil_div_sz(rows, kBlock / tpr);
    ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((smce_label_fwd_kernel<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, logits,
                                            labels, lse, row_loss, rows, cols));
    ZG_LAUNCH_CHECK();
    return flat_reduce_into<TermId, 1>(ctx, row_loss, nullptr, rows, 0.f, FinDivN{loss, (float)rows}, partials);
}

ZG_API int zg_hip_smce_label_bwd(zg_hip_ctx* ctx, const float* logits, const uint64_t* labels, const float* lse,
                                 float* grad, size_t rows, size_t cols, int accumulate) {
    ZG_CTX(ctx);  // (a gradient fill that is still waiting is launched here: this form is not the reference's own)
    ZG_REQUIRE(logits && labels && lse && grad, "smce_label_bwd: null pointer");
    if (int rc = check_rows("smce_label_bwd", rows, cols)) return rc;
    const bool aligned = ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(grad)) & 15u) == 0;
    if (aligned && cols % 4 == 0 && cols / 4 >= kLabelBwdMinC4) {
        const size_t n4 = rows * (cols / 4);
        size_t blocks = ceil_div_sz(n4, kLabelBwdChunk);
        if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
        if (accumulate)
            hipLaunchKernelGGL((smce_label_bwd_flat_kernel<true>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream,
                               logits, labels, lse, grad, n4, cols / 4, (float)rows);
        else
            hipLaunchKernelGGL((smce_label_bwd_flat_kernel<false>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream,
                               logits, labels, lse, grad, n4, cols / 4, (float)rows);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    const size_t n = rows * cols;
    if (aligned && cols >= 4 && cols < 0xffffffffull) {
        size_t blocks = ceil_div_sz(n >> 2, kLabelBwdChunk);
        if (blocks < 1) blocks = 1;
        if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
        if (accumulate)
            hipLaunchKernelGGL((smce_label_bwd_any_kernel<true>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream,
                               logits, labels, lse, grad, n, cols, rows, (float)rows);
        else
            hipLaunchKernelGGL((smce_label_bwd_any_kernel<false>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream,
                               logits, labels, lse, grad, n, cols, rows, (float)rows);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    size_t blocks = ceil_div_sz(n, kBlock);
    if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
    if (accumulate)
        hipLaunchKernelGGL((smce_label_bwd_values_kernel<true>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream, logits,
                           labels, lse, grad, n, cols, (float)rows);
    else
        hipLaunchKernelGGL((smce_label_bwd_values_kernel<false>), dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream,
                           logits, labels, lse, grad, n, cols, (float)rows);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_smce_fwd(zg_hip_ctx* ctx, const float* logits, const float* target, float* probs, float* loss,
                           size_t rows, size_t cols) {
    ZG_CTX(ctx);
    ZG_REQUIRE(logits && target && probs && loss, "smce_fwd: null pointer");
    if (int rc = check_rows("smce_fwd", rows, cols)) return rc;
    {
        // a batch small enough for one workgroup: rows and their mean in one launch
        const int tpr = pick_tpr(cols);
        if (tpr <= kWave && rows <= (size_t)(kFlatSingle / tpr) && !long_row_ok(logits, target, probs, rows, cols)) {
            ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((smce_small_kernel<(T <= kWave ? T : kWave), 0>), dim3(1), dim3(kFlatSingle),
                                                    0, ctx->stream, logits, target, probs, loss, (float*)nullptr, rows, cols));
            ZG_LAUNCH_CHECK();
            return ZG_HIP_OK;
        }
    }
    size_t seg = 0;
    if (const int n_seg = row_segments_for(ctx, rows, cols, &seg)) {
        char* mem = (char*)workspace(ctx, rows * n_seg * (sizeof(float) + sizeof(OnlineAccT)));
        if (!mem) return ZG_HIP_EOOM;
        OnlineAccT* acc = (OnlineAccT*)mem;
        float* seg_loss = (float*)(mem + rows * n_seg * sizeof(OnlineAccT));
        const dim3 grid((unsigned)n_seg, (unsigned)rows);
        hipLaunchKernelGGL(softmax_seg_online_kernel, grid, dim3(kBlock), 0, ctx->stream, logits, acc, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(softmax_seg_probs_kernel<1>, grid, dim3(kBlock), 0, ctx->stream, logits, target, probs, acc,
                           seg_loss, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        return flat_reduce<TermId, 1>(ctx, seg_loss, nullptr, rows * n_seg, 0.f, FinDivN{loss, (float)rows});
    }
    float* row_loss = (float*)workspace(ctx, rows * sizeof(float));
    if (!row_loss) return ZG_HIP_EOOM;
    if (long_row_ok(logits, target, probs, rows, cols)) {
        ZG_LONG_ROWS(1, 0, logits, target, probs, row_loss, cols, (float*)nullptr, 1.f);
    } else if (wave_row_ok(logits, target, probs, rows, cols)) {
        ZG_WAVE_ROWS(1, 0, logits, target, probs, row_loss, rows, cols, (float*)nullptr, 1.f);
    } else {
        const int tpr = pick_tpr(cols);
        const unsigned grid = (unsigned)ceil_div_sz(rows, kBlock / tpr);
        ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((softmax_rows_kernel<T, 1>), dim3(grid), dim3(kBlock), 0, ctx->stream,
                                                logits, target, probs, row_loss, rows, cols));
    }
    ZG_LAUNCH_CHECK();
    return flat_reduce<TermId, 1>(ctx, row_loss, nullptr, rows, 0.f, FinDivN{loss, (float)rows});
}

ZG_API int zg_hip_smce_bwd(zg_hip_ctx* ctx, const float* probs, const float* target, float* grad, size_t rows,
                           size_t cols) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    if (rows == 0 || cols == 0) return ZG_HIP_OK;  // the host's loop over no rows (src/nn/loss.zig:157-171)
    ZG_REQUIRE(probs && target && grad, "smce_bwd: null pointer");
    if (int rc = check_rows("smce_bwd", rows, cols)) return rc;
    // the gradient's zero fill (ensure_grad(0), src/ndtensor.zig:221-228) may still be waiting: then write, not add
    const bool fresh = absorb_zero_fill(ctx, grad, rows * cols);
    {
        // a fill that meets none of the three operands keeps waiting (the loss's upstream gradient is filled right
        // before this call and read by nobody: src/nn/loss.zig:150-159 folds it into the 1/rows factor)
        const void* ops[3] = {probs, target, grad};
        const size_t bytes[3] = {rows * cols * sizeof(float), rows * cols * sizeof(float), rows * cols * sizeof(float)};
        if (int rc = flush_pending_but_fills(ctx, ops, bytes, 3)) {
            if (fresh) (void)zg_hip_mem_fill(ctx, grad, rows * cols, 0.f);
            return rc;
        }
    }
    const size_t n = rows * cols;
    const unsigned blocks = smce_bwd_grid(n);
    if (fresh)
        hipLaunchKernelGGL(smce_bwd_kernel<false>, dim3(blocks), dim3(kBlock), 0, ctx->stream, probs, target, grad, n,
                           (float)rows);
    else
        hipLaunchKernelGGL(smce_bwd_kernel<true>, dim3(blocks), dim3(kBlock), 0, ctx->stream, probs, target, grad, n,
                           (float)rows);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_smce_fwd_bwd(zg_hip_ctx* ctx, const float* logits, const float* target, float* probs, float* loss,
                               float* grad, size_t rows, size_t cols, int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(logits && target && probs && loss && grad, "smce_fwd_bwd: null pointer");
    if (int rc = check_rows("smce_fwd_bwd", rows, cols)) return rc;
    const int tpr = pick_tpr(cols);
    if (tpr <= kWave && rows <= (size_t)(kFlatSingle / tpr) && !long_row_ok(logits, target, probs, rows, cols)) {
#define ZG_SMALL(T)                                                                                                    \
    if (accumulate)                                                                                                    \
        hipLaunchKernelGGL((smce_small_kernel<T, 2>), dim3(1), dim3(kFlatSingle), 0, ctx->stream, logits, target,      \
                           probs, loss, grad, rows, cols);                                                             \
    else                                                                                                               \
        hipLaunchKernelGGL((smce_small_kernel<T, 1>), dim3(1), dim3(kFlatSingle), 0, ctx->stream, logits, target,      \
                           probs, loss, grad, rows, cols)
        if (tpr == 4) { ZG_SMALL(4); }
        else if (tpr == 16) { ZG_SMALL(16); }
        else { ZG_SMALL(64); }
#undef ZG_SMALL
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    // rows a wave or a workgroup holds in registers: probabilities, loss terms and gradient in one pass over the logits
    // and the target (four streams instead of the six of forward + backward); the gradient must not lie on the inputs
    const size_t n = rows * cols;
    auto apart = [&](const float* a) { return a + n <= grad || grad + n <= a; };
    const bool one_pass = aligned16(grad) && apart(logits) && apart(target) && apart(probs) &&
                          (long_row_ok(logits, target, probs, rows, cols) || wave_row_ok(logits, target, probs, rows, cols));
    if (one_pass) {
        float* row_loss = (float*)workspace(ctx, rows * sizeof(float));
        if (!row_loss) return ZG_HIP_EOOM;
        const float denom = (float)rows;
        if (long_row_ok(logits, target, probs, rows, cols)) {
            if (accumulate) ZG_LONG_ROWS(1, 2, logits, target, probs, row_loss, cols, grad, denom);
            else ZG_LONG_ROWS(1, 1, logits, target, probs, row_loss, cols, grad, denom);
        } else {
            if (accumulate) ZG_WAVE_ROWS(1, 2, logits, target, probs, row_loss, rows, cols, grad, denom);
            else ZG_WAVE_ROWS(1, 1, logits, target, probs, row_loss, rows, cols, grad, denom);
        }
        ZG_LAUNCH_CHECK();
        return flat_reduce<TermId, 1>(ctx, row_loss, nullptr, rows, 0.f, FinDivN{loss, denom});
    }
    if (int rc = zg_hip_smce_fwd(ctx, logits, target, probs, loss, rows, cols)) return rc;
    const unsigned blocks = smce_bwd_grid(n);
    if (accumulate)
        hipLaunchKernelGGL(smce_bwd_kernel<true>, dim3(blocks), dim3(kBlock), 0, ctx->stream, probs, target, grad,
                           n, (float)rows);
    else
        hipLaunchKernelGGL(smce_bwd_kernel<false>, dim3(blocks), dim3(kBlock), 0, ctx->stream, probs, target,
                           grad, n, (float)rows);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_softmax_fwd(zg_hip_ctx* ctx, const float* x, float* y, size_t rows, size_t cols) {
    ZG_CTX(ctx);
    if (rows == 0 || cols == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && y, "softmax_fwd: null pointer");
    if (int rc = check_rows("softmax_fwd", rows, cols)) return rc;
    size_t seg = 0;
    if (const int n_seg = row_segments_for(ctx, rows, cols, &seg)) {
        OnlineAccT* acc = (OnlineAccT*)workspace(ctx, rows * n_seg * sizeof(OnlineAccT));
        if (!acc) return ZG_HIP_EOOM;
        const dim3 grid((unsigned)n_seg, (unsigned)rows);
        hipLaunchKernelGGL(softmax_seg_online_kernel, grid, dim3(kBlock), 0, ctx->stream, x, acc, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(softmax_seg_probs_kernel<0>, grid, dim3(kBlock), 0, ctx->stream, x, (const float*)nullptr, y, acc,
                           (float*)nullptr, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (long_row_ok(x, x, y, rows, cols)) {
        ZG_LONG_ROWS(0, 0, x, (const float*)nullptr, y, (float*)nullptr, cols, (float*)nullptr, 1.f);
    } else if (wave_row_ok(x, x, y, rows, cols)) {
        ZG_WAVE_ROWS(0, 0, x, (const float*)nullptr, y, (float*)nullptr, rows, cols, (float*)nullptr, 1.f);
    } else {
        const int tpr = pick_tpr(cols);
        const unsigned grid = (unsigned)ceil_div_sz(rows, kBlock / tpr);
        ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((softmax_rows_kernel<T, 0>), dim3(grid), dim3(kBlock), 0, ctx->stream, x,
                                                (const float*)nullptr, y, (float*)nullptr, rows, cols));
    }
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_softmax_bwd(zg_hip_ctx* ctx, const float* y, const float* y_g, float* x_g, size_t rows, size_t cols) {
    ZG_CTX(ctx);
    if (rows == 0 || cols == 0) return ZG_HIP_OK;
    ZG_REQUIRE(y && y_g && x_g, "softmax_bwd: null pointer");
    if (int rc = check_rows("softmax_bwd", rows, cols)) return rc;
    size_t seg = 0;
    if (const int n_seg = row_segments_for(ctx, rows, cols, &seg)) {
        float* dots = (float*)workspace(ctx, rows * n_seg * sizeof(float));
        if (!dots) return ZG_HIP_EOOM;
        const dim3 grid((unsigned)n_seg, (unsigned)rows);
        hipLaunchKernelGGL(softmax_bwd_seg_dot_kernel, grid, dim3(kBlock), 0, ctx->stream, y, y_g, x_g, dots, cols, seg, n_seg);
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(softmax_bwd_seg_apply_kernel, grid, dim3(kBlock), 0, ctx->stream, y, y_g, x_g, dots, cols, seg,
                           n_seg);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(y_g) | reinterpret_cast<uintptr_t>(x_g);
    if (cols % 4 == 0 && (bits & 15u) == 0 && cols <= 32768 && rows <= 0x7fffffffull) {
#define ZG_BWD_ROWS(NT, VEC, ROWS_PER_WG)                                                                              \
    hipLaunchKernelGGL((softmax_bwd_rows_kernel<NT, VEC>), dim3((unsigned)ceil_div_sz(rows, ROWS_PER_WG)),             \
                       dim3(NT <= kWave ? kBlock : NT), 0, ctx->stream, y, y_g, x_g, rows, cols)
        if (cols <= 256) ZG_BWD_ROWS(16, 4, kBlock / 16);
        else if (cols <= 1024) ZG_BWD_ROWS(64, 4, kBlock / 64);
        else if (cols <= 4096) ZG_BWD_ROWS(256, 4, 1);
        else if (cols <= 8192) ZG_BWD_ROWS(256, 8, 1);
        else ZG_BWD_ROWS(1024, 8, 1);
#undef ZG_BWD_ROWS
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    // rows the register kernel does not take (off the 16-byte grid, or longer than 32768 columns); sixteen lanes from 13
    // columns on (four lanes on 31 columns, eight values each one after the other: 16 % of 8 TB/s)
    const int tpr = (cols > 12 && cols <= 32) ? 16 : pick_tpr(cols);
    const unsigned grid = (unsigned)ceil_div_sz(rows, kBlock / tpr);
    ZG_TPR_DISPATCH(tpr, hipLaunchKernelGGL((softmax_bwd_kernel<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, y, y_g,
                                            x_g, rows, cols));
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}
