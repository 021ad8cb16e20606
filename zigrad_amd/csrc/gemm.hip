// fp32 GEMM family on the CDNA4 matrix cores: matmul, bmm_acc (all four transpose variants, alpha/beta,
// explicit leading dimensions), matvec, outer, transpose.
//
// Reference semantics: cblas_sgemm(RowMajor, ...) as called from src/device/host_device.zig:242-250 and
// the batch loop of :277-313.
//
// Kernel shape: a workgroup of 4 waves (2 x 2) owns a BM x BN tile of C.  Each wave owns a
// (BM/2) x (BN/2) sub-tile as a grid of 32x32 accumulator blocks fed by v_mfma_f32_32x32x2_f32.
// Operand tiles of BK = 16 along k are staged through LDS in a k-major layout ([k][m] and [k][n]), so
// a wave's fragment read (32 consecutive m or n for one k) is one conflict-free row segment, whatever
// the operand's layout in HBM.  LDS is double buffered: the global loads of tile t+1 are in flight
// while the MFMAs of tile t run, with one barrier per tile.  Workgroup ids are remapped so that the
// workgroups resident on one XCD (ids congruent modulo 8) cover a compact patch of C and share their
// A rows / B columns in that XCD's L2.
#include "common.h"

#include <type_traits>

namespace zg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));  // first-class vector: stays in registers

constexpr int BK = 16;
constexpr int kGemmThreads = 256;

#ifndef ZG_GEMM_MNMAP
#define ZG_GEMM_MNMAP 0
#endif


// One operand tile: `BMN` rows in the m (or n) direction by BK along k.
// KMAJOR: element (mn, k) lives at ptr[mn * ld + k]   (A not transposed, B transposed)
// else  : element (mn, k) lives at ptr[k * ld + mn]   (A transposed, B not transposed)
// LDS layout is always [k][mn] with row stride LD floats.
template <int BMN, bool KMAJOR>
struct Tile {
    static constexpr int LD = BMN + 4;
    static constexpr int NV = BMN * BK / 4 / kGemmThreads;
    floatx4 r[NV];

    // which float4 of the tile thread `threadIdx.x` handles in its i-th access: (mn, k) of its first element
    static __device__ __forceinline__ void coords(int i, int& mn, int& k) {
        const int f = threadIdx.x + i * kGemmThreads;
        if (KMAJOR) {
            mn = f / (BK / 4);
            k = (f % (BK / 4)) * 4;
        } else {
#if ZG_GEMM_MNMAP
            constexpr int L = BMN / 32;  // 128-byte lines per k-row of the tile
            constexpr int NL = BK * L;   // lines in the tile
            const int hl = f >> 2, sub = f & 3;
            const int line = hl % NL, pass = hl / NL;
            const int half = (pass + line) & 1;
            k = line / L;
            mn = ((line % L) * 8 + half * 4 + sub) * 4;
#else
            k = f / (BMN / 4);
            mn = (f % (BMN / 4)) * 4;
#endif
        }
    }

    template <bool SAFE>
    __device__ __forceinline__ void load(const float* __restrict__ p, size_t ld, size_t mn0, size_t k0, size_t MN,
                                         size_t K, bool vec_ok) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int tmn, tk;
            coords(i, tmn, tk);
            const size_t mn = mn0 + tmn, k = k0 + tk;
            const float* q = KMAJOR ? p + mn * ld + k : p + k * ld + mn;
            if (!SAFE) {
                r[i] = *reinterpret_cast<const floatx4*>(q);
            } else {
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (KMAJOR) {
                    if (mn < MN) {
                        if (vec_ok && k + 4 <= K) {
                            v = *reinterpret_cast<const floatx4*>(q);
                        } else {
                            if (k + 0 < K) v.x = q[0];
                            if (k + 1 < K) v.y = q[1];
                            if (k + 2 < K) v.z = q[2];
                            if (k + 3 < K) v.w = q[3];
                        }
                    }
                } else {
                    if (k < K) {
                        if (vec_ok && mn + 4 <= MN) {
                            v = *reinterpret_cast<const floatx4*>(q);
                        } else {
                            if (mn + 0 < MN) v.x = q[0];
                            if (mn + 1 < MN) v.y = q[1];
                            if (mn + 2 < MN) v.z = q[2];
                            if (mn + 3 < MN) v.w = q[3];
                        }
                    }
                }
                r[i] = v;
            }
        }
    }

    // LDS write instructions this thread issues per tile: 4 scalar writes per float4 for a k-major operand
    // (the transposing store), one 128-bit write otherwise
    static constexpr int NW = NV * (KMAJOR ? 4 : 1);

    // the op-th of those writes
    __device__ __forceinline__ void store_op(float* __restrict__ lds, int op) const {
        const int i = KMAJOR ? op / 4 : op;
        int mn, k;
        coords(i, mn, k);
        if (KMAJOR) {
            const int c = op % 4;
            lds[(k + c) * LD + mn] = r[i][c];
        } else {
            *reinterpret_cast<floatx4*>(lds + k * LD + mn) = r[i];
        }
    }

    __device__ __forceinline__ void store(float* __restrict__ lds) const {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int mn, k;
            coords(i, mn, k);
            if (KMAJOR) {
                lds[(k + 0) * LD + mn] = r[i].x;
                lds[(k + 1) * LD + mn] = r[i].y;
                lds[(k + 2) * LD + mn] = r[i].z;
                lds[(k + 3) * LD + mn] = r[i].w;
            } else {
                *reinterpret_cast<floatx4*>(lds + k * LD + mn) = r[i];
            }
        }
    }
};

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    size_t M, N, K;
    size_t lda, ldb, ldc;
    float alpha, beta;
    // batching: operand batch index = z % n_batch_{a,b}
    size_t nba, nbb;
    size_t a_chunk, b_chunk, c_chunk;
    unsigned tiles_m, tiles_n;
    int a_vec, b_vec;  // 16-byte vector loads are legal for this operand
};

// Logical tile id from the hardware workgroup id.  Hardware deals consecutive ids round-robin to the 8
// XCDs; give each XCD a contiguous run of logical ids, then walk C in column groups of 8 tile-rows.
__device__ __forceinline__ void tile_coords(unsigned pid, unsigned tiles_m, unsigned tiles_n, unsigned& tm,
                                            unsigned& tn) {
    const unsigned total = tiles_m * tiles_n;
    unsigned id = pid;
    if ((total & 7u) == 0) id = (pid & 7u) * (total >> 3) + (pid >> 3);
    constexpr unsigned GM = 8;
    const unsigned per_group = GM * tiles_n;
    const unsigned group = id / per_group;
    const unsigned first_m = group * GM;
    const unsigned gsize = (tiles_m - first_m < GM) ? (tiles_m - first_m) : GM;
    const unsigned in_group = id % per_group;
    tm = first_m + in_group % gsize;
    tn = in_group / gsize;
}

template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, bool SAFE>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmArgs g) {
    using TA = Tile<BM, A_KMAJOR>;
    using TB = Tile<BN, B_KMAJOR>;
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_ELEMS = BK * TA::LD, B_ELEMS = BK * TB::LD;
    __shared__ __attribute__((aligned(16))) float lds[2 * (A_ELEMS + B_ELEMS)];
    float* As0 = lds;
    float* Bs0 = lds + 2 * A_ELEMS;

    unsigned tm, tn;
    tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
    const size_t z = blockIdx.z;
    const float* A = g.A + (z % g.nba) * g.a_chunk;
    const float* B = g.B + (z % g.nbb) * g.b_chunk;
    float* C = g.C + z * g.c_chunk;
    const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int l32 = lane & 31, lk = lane >> 5;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const size_t KT = (g.K + BK - 1) / BK;
    constexpr int NP = BK / 2;   // k-pairs (one MFMA step each) per tile
    constexpr int NM = TM * TN;  // MFMAs per k-pair
    constexpr int NW = TA::NW + TB::NW;
    constexpr int WPM = (NW + NM - 1) / NM;  // LDS writes placed in front of each MFMA of the last pair

    // A wave issues in order and one fp32 MFMA keeps the matrix pipe busy for 64 cycles, so whatever has to
    // overlap with it must sit between MFMAs in the instruction stream.  The schedule is written out by hand
    // and pinned with sched_barrier (left alone, the scheduler sinks every load next to its use and exposes
    // the LDS and L2 latencies):
    //   tile start : read the fragments of pair 0, issue the global loads of the next tile
    //   pair p     : read the fragments of pair p+1 (second register set), then the MFMAs of pair p
    //   last pair  : the LDS writes of the next tile are dealt out in front of its MFMAs
    float fa[2][TM], fb[2][TN];
    auto read_frag = [&](int set, const float* As, const float* Bs, int kk) {
#pragma unroll
        for (int i = 0; i < TM; i++) fa[set][i] = As[(kk + lk) * TA::LD + wm0 + i * 32 + l32];
#pragma unroll
        for (int j = 0; j < TN; j++) fb[set][j] = Bs[(kk + lk) * TB::LD + wn0 + j * 32 + l32];
    };
    TA ta;
    TB tb;
    auto tile_step = [&](size_t kt, auto more_tag) {
        constexpr bool MORE = decltype(more_tag)::value;
        const int cur = (int)(kt & 1);
        const float* As = As0 + cur * A_ELEMS;
        const float* Bs = Bs0 + cur * B_ELEMS;
        float* As_next = As0 + (cur ^ 1) * A_ELEMS;
        float* Bs_next = Bs0 + (cur ^ 1) * B_ELEMS;
        read_frag(0, As, Bs, 0);
        if (MORE) {
            ta.template load<SAFE>(A, g.lda, m0, (kt + 1) * BK, g.M, g.K, g.a_vec != 0);
            tb.template load<SAFE>(B, g.ldb, n0, (kt + 1) * BK, g.N, g.K, g.b_vec != 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < NP; p++) {
            if (p + 1 < NP) read_frag((p + 1) & 1, As, Bs, 2 * (p + 1));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < NM; q++) {
                if (MORE && p == NP - 1) {
#pragma unroll
                    for (int w = q * WPM; w < (q + 1) * WPM && w < NW; w++) {
                        if (w < TA::NW) ta.store_op(As_next, w);
                        else tb.store_op(Bs_next, w - TA::NW);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                const int i = q / TN, j = q % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[p & 1][i], fb[p & 1][j], acc[i][j], 0, 0, 0);
                if (MORE && p == NP - 1) __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };

    ta.template load<SAFE>(A, g.lda, m0, 0, g.M, g.K, g.a_vec != 0);
    tb.template load<SAFE>(B, g.ldb, n0, 0, g.N, g.K, g.b_vec != 0);
    ta.store(As0);
    tb.store(Bs0);
    __syncthreads();
    for (size_t kt = 0; kt + 1 < KT; kt++) tile_step(kt, std::true_type{});
    tile_step(KT - 1, std::false_type{});

    // epilogue: accumulator register r of lane l holds C[(r/4)*8 + (l/32)*4 + r%4][l%32] of its 32x32 block
    const float alpha = g.alpha, beta = g.beta;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const size_t col = n0 + wn0 + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const size_t row = m0 + wm0 + i * 32 + (r >> 2) * 8 + lk * 4 + (r & 3);
                if (!SAFE || (row < g.M && col < g.N)) {
                    float* c = C + row * g.ldc + col;
                    float v = alpha * acc[i][j][r];
                    if (beta != 0.f) v += beta * (*c);  // C is not read when beta == 0
                    *c = v;
                }
            }
        }
    }
}

template <int BM, int BN>
static int launch_gemm(zg_hip_ctx* ctx, GemmArgs& g, bool a_kmajor, bool b_kmajor, bool safe, size_t batches) {
    g.tiles_m = (unsigned)ceil_div_sz(g.M, BM);
    g.tiles_n = (unsigned)ceil_div_sz(g.N, BN);
    dim3 grid(g.tiles_m * g.tiles_n, 1, (unsigned)batches), block(kGemmThreads);
#define ZG_GEMM(AK, BKM, SF) \
    hipLaunchKernelGGL((gemm_kernel<BM, BN, AK, BKM, SF>), grid, block, 0, ctx->stream, g)
    if (safe) {
        if (a_kmajor && b_kmajor) ZG_GEMM(true, true, true);
        else if (a_kmajor && !b_kmajor) ZG_GEMM(true, false, true);
        else if (!a_kmajor && b_kmajor) ZG_GEMM(false, true, true);
        else ZG_GEMM(false, false, true);
    } else {
        if (a_kmajor && b_kmajor) ZG_GEMM(true, true, false);
        else if (a_kmajor && !b_kmajor) ZG_GEMM(true, false, false);
        else if (!a_kmajor && b_kmajor) ZG_GEMM(false, true, false);
        else ZG_GEMM(false, false, false);
    }
#undef ZG_GEMM
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// C *= beta (or 0) when k == 0 or alpha == 0: BLAS leaves beta*C
__global__ void scale_c_kernel(float* C, size_t M, size_t N, size_t ldc, float beta, size_t c_chunk) {
    float* c = C + (size_t)blockIdx.z * c_chunk;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; i < M * N; i += nt) {
        size_t r = i / N, col = i % N;
        c[r * ldc + col] = (beta == 0.f) ? 0.f : beta * c[r * ldc + col];
    }
}

static int gemm_dispatch(zg_hip_ctx* ctx, const char* name, const float* A, const float* B, float* C, size_t m, size_t n,
                         size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta,
                         size_t batches, size_t nba, size_t nbb, size_t a_chunk, size_t b_chunk, size_t c_chunk) {
    if (m == 0 || n == 0 || batches == 0) return ZG_HIP_OK;
    ZG_REQUIRE(A && B && C, "%s: null pointer", name);
    // cblas argument rules for row-major storage
    ZG_REQUIRE(lda >= (trans_a ? m : k) && lda >= 1, "%s: lda %zu too small", name, lda);
    ZG_REQUIRE(ldb >= (trans_b ? k : n) && ldb >= 1, "%s: ldb %zu too small", name, ldb);
    ZG_REQUIRE(ldc >= n, "%s: ldc %zu < n %zu", name, ldc, n);
    ZG_REQUIRE(batches <= 65535, "%s: more than 65535 batches", name);
    ZG_REQUIRE(nba >= 1 && nbb >= 1, "%s: zero operand batches", name);
    if (k == 0 || alpha == 0.f) {
        if (beta == 1.f) return ZG_HIP_OK;
        size_t blocks = ceil_div_sz(m * n, 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(scale_c_kernel, dim3((unsigned)blocks, 1, (unsigned)batches), dim3(256), 0, ctx->stream, C, m,
                           n, ldc, beta, c_chunk);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    GemmArgs g;
    g.A = A;
    g.B = B;
    g.C = C;
    g.M = m;
    g.N = n;
    g.K = k;
    g.lda = lda;
    g.ldb = ldb;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    g.nba = nba;
    g.nbb = nbb;
    g.a_chunk = a_chunk;
    g.b_chunk = b_chunk;
    g.c_chunk = c_chunk;
    const bool a_kmajor = !trans_a, b_kmajor = trans_b != 0;
    g.a_vec = aligned16(A) && lda % 4 == 0 && a_chunk % 4 == 0;
    g.b_vec = aligned16(B) && ldb % 4 == 0 && b_chunk % 4 == 0;

    // tile choice: the largest tile that still gives every CU a workgroup
    const size_t t128 = ceil_div_sz(m, 128) * ceil_div_sz(n, 128) * batches;
    const size_t t256 = ceil_div_sz(m, 256) * ceil_div_sz(n, 128) * batches;
    const bool big = t256 >= (size_t)ctx->n_cu * 2;
    (void)t128;
    if (big) {
        const bool safe = !(g.a_vec && g.b_vec && m % 256 == 0 && n % 128 == 0 && k % BK == 0);
        return launch_gemm<256, 128>(ctx, g, a_kmajor, b_kmajor, safe, batches);
    }
    if (m > 64 && n > 64) {
        const bool safe = !(g.a_vec && g.b_vec && m % 128 == 0 && n % 128 == 0 && k % BK == 0);
        return launch_gemm<128, 128>(ctx, g, a_kmajor, b_kmajor, safe, batches);
    }
    const bool safe = !(g.a_vec && g.b_vec && m % 64 == 0 && n % 64 == 0 && k % BK == 0);
    return launch_gemm<64, 64>(ctx, g, a_kmajor, b_kmajor, safe, batches);
}

// ------------------------------------------------------------------------------------------------
// matvec / outer / transpose
// ------------------------------------------------------------------------------------------------

// y = alpha * A x + beta * y, A is [m, n] row-major: one wave per row
__global__ __launch_bounds__(256) void gemv_n_kernel(const float* A, const float* x, float* y, size_t m, size_t n,
                                                      float alpha, float beta) {
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m) return;
    const int lane = threadIdx.x & 63;
    const float* a = A + row * n;
    float s = 0.f;
    for (size_t j = lane; j < n; j += 64) s += a[j] * x[j];
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
    if (lane == 0) y[row] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[row];
}

// y = alpha * A^T x + beta * y, A is [m, n] row-major, y has n entries: thread per column, rows in order
__global__ __launch_bounds__(256) void gemv_t_kernel(const float* A, const float* x, float* y, size_t m, size_t n,
                                                      float alpha, float beta) {
    const size_t col = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= n) return;
    float s = 0.f;
    for (size_t i = 0; i < m; i++) s += A[i * n + col] * x[i];
    y[col] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[col];
}

// A += alpha * x y^T   (cblas_sger, src/device/host_device.zig:252-258)
__global__ __launch_bounds__(256) void ger_kernel(const float* x, size_t xl, const float* y, size_t yl, float* A,
                                                   float alpha) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, nt = (size_t)gridDim.x * 256;
    for (; i < xl * yl; i += nt) {
        size_t r = i / yl, c = i % yl;
        A[i] = __fadd_rn(A[i], __fmul_rn(__fmul_rn(alpha, x[r]), y[c]));
    }
}

// B = A^T + alpha * B through a 32x33 LDS tile so both the read of A and the write of B are coalesced.
// B is not read when alpha == 0.
__global__ __launch_bounds__(256) void transpose_kernel(const float* A, float* B, size_t m, size_t n, float alpha) {
    __shared__ float tile[32][33];
    const size_t bi = (size_t)blockIdx.y * 32, bj = (size_t)blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8) {
        size_t i = bi + r, j = bj + tx;
        if (i < m && j < n) tile[r][tx] = A[i * n + j];
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        size_t j = bj + r, i = bi + tx;  // B[j, i]
        if (i < m && j < n) {
            float v = tile[tx][r];
            float* b = B + j * m + i;
            *b = (alpha == 0.f) ? v : __fadd_rn(v, __fmul_rn(alpha, *b));
        }
    }
}

}  // namespace zg

using namespace zg;

ZG_API int zg_hip_matmul(zg_hip_ctx* ctx, const float* A, const float* B, float* C, size_t m, size_t n, size_t k,
                         int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    ZG_CTX(ctx);
    return gemm_dispatch(ctx, "matmul", A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, 1, 1, 1, 0, 0, 0);
}

ZG_API int zg_hip_bmm_acc(zg_hip_ctx* ctx, const float* A, const uint64_t* A_shape, const float* B,
                          const uint64_t* B_shape, float* C, const uint64_t* C_shape, int trans_a, int trans_b,
                          size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    ZG_CTX(ctx);
    ZG_REQUIRE(A_shape && B_shape && C_shape, "bmm_acc: null shape");
    const size_t nba = A_shape[0], nbb = B_shape[0], nbc = C_shape[0];
    const size_t m = C_shape[1], n = C_shape[2], k = A_shape[2];
    ZG_REQUIRE(A_shape[1] == m, "bmm_acc: A rows %llu != C rows %zu", (unsigned long long)A_shape[1], m);
    ZG_REQUIRE(B_shape[1] == k && B_shape[2] == n, "bmm_acc: B shape does not match [%zu, %zu]", k, n);
    if (nbc == 0) return ZG_HIP_OK;
    ZG_REQUIRE(nba >= 1 && nbb >= 1, "bmm_acc: zero operand batches");
    return gemm_dispatch(ctx, "bmm_acc", A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, nbc, nba, nbb,
                         A_shape[1] * A_shape[2], B_shape[1] * B_shape[2], C_shape[1] * C_shape[2]);
}

ZG_API int zg_hip_matvec(zg_hip_ctx* ctx, const float* A, const float* x, float* y, size_t m, size_t n, int trans_a,
                         float alpha, float beta) {
    ZG_CTX(ctx);
    if (m == 0 || n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(A && x && y, "matvec: null pointer");
    if (!trans_a)
        hipLaunchKernelGGL(gemv_n_kernel, dim3((unsigned)ceil_div_sz(m, 4)), dim3(256), 0, ctx->stream, A, x, y, m, n,
                           alpha, beta);
    else
        hipLaunchKernelGGL(gemv_t_kernel, dim3((unsigned)ceil_div_sz(n, 256)), dim3(256), 0, ctx->stream, A, x, y, m, n,
                           alpha, beta);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_outer(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* A, float alpha) {
    ZG_CTX(ctx);
    if (xl == 0 || yl == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && y && A, "outer: null pointer");
    size_t blocks = ceil_div_sz(xl * yl, 256);
    if (blocks > (size_t)ctx->n_cu * 16) blocks = (size_t)ctx->n_cu * 16;
    hipLaunchKernelGGL(ger_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, x, xl, y, yl, A, alpha);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_transpose(zg_hip_ctx* ctx, const float* A, float* B, size_t m, size_t n, float alpha) {
    ZG_CTX(ctx);
    if (m == 0 || n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(A && B, "transpose: null pointer");
    ZG_REQUIRE(A != B, "transpose: in-place transpose is not supported");
    dim3 grid((unsigned)ceil_div_sz(n, 32), (unsigned)ceil_div_sz(m, 32));
    ZG_REQUIRE(grid.y <= 65535, "transpose: too many rows");
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, ctx->stream, A, B, m, n, alpha);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}
