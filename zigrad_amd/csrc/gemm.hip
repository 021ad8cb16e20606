// fp32 GEMM family on the CDNA4 matrix cores: matmul, bmm_acc (all four transpose variants, alpha/beta,
// explicit leading dimensions), the fused Linear entry points built on them (forward with bias and ReLU in the
// epilogue, masked input gradient, a small layer's whole backward in one launch), matvec, outer, transpose.
//
// Reference semantics: cblas_sgemm(RowMajor, ...) as called from src/device/host_device.zig:242-250 and
// the batch loop of :277-313.
//
// Kernel shape: a workgroup of 4 waves (2 x 2) owns a BM x BN tile of C.  Each wave owns a
// (BM/2) x (BN/2) sub-tile as a grid of 32x32 accumulator blocks fed by v_mfma_f32_32x32x2_f32.
// Operand tiles of BK = 16 along k are staged through LDS, double buffered, one barrier per tile.
//
// A wave cannot overlap its own non-MFMA instructions with its MFMAs to any useful degree (measured: every
// LDS or global instruction in the loop costs about its issue time), so the loop is built to need few of them:
//   * LDS keeps each operand tile in the orientation it has in HBM ([mn][k] for a k-contiguous operand,
//     [k][mn] otherwise), so a tile moves HBM -> registers -> LDS with 16-byte loads and 16-byte LDS writes only;
//     the [mn][k] form is XOR-swizzled, the other padded, so that no LDS access conflicts on banks.
//   * An MFMA sums over two k values, one per lane half, and it does not matter which two as long as A and B
//     agree.  Lane half h takes k = 8g + 4h + c in step c of k-group g.  A lane of a k-contiguous operand then
//     reads its 4 steps of one 32-row block with one ds_read_b128; a lane of the other kind reads, per step,
//     its T consecutive rows (block row b <-> tile rows b*T .. b*T+T-1) with one ds_read_b128 / b64.
//   * All LDS addresses are a per-thread base plus immediates; global addresses are a scalar base plus a
//     per-thread 32-bit offset.
// Workgroup ids are remapped so that the workgroups resident on one XCD (ids congruent modulo 8) cover a
// compact patch of C and share their A rows / B columns in that XCD's L2.
#include "common.h"
#include "reduce_device.h"

#include <type_traits>

namespace zg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));  // first-class vector: stays in registers

constexpr int kGemmThreads = 256;

constexpr int kBK = 16;  // tile depth along k: two k-groups of 8

template <int T>
struct VecOf;
template <>
struct VecOf<1> {
    typedef float type;
};
template <>
struct VecOf<2> {
    typedef float type __attribute__((ext_vector_type(2)));
};
template <>
struct VecOf<4> {
    typedef floatx4 type;
};

// One operand tile: `BMN` rows in the m (or n) direction by kBK along k.
// KMAJOR: element (mn, k) lives at ptr[mn * ld + k]   (A not transposed, B transposed); LDS holds [mn][k]
// else  : element (mn, k) lives at ptr[k * ld + mn]   (A transposed, B not transposed); LDS holds [k][mn]
// [k][mn] rows carry 4 floats of padding.  [mn][k] rows are 16 floats with no padding; the 16-byte piece kq of row
// mn sits at column kq ^ ((mn >> 2) & 3), so that both the LDS writes (4 pieces of 4 adjacent rows per 16 lanes) and
// the fragment reads (one piece of 16 adjacent rows per 16 lanes) touch 64 distinct banks.
template <int BMN, bool KMAJOR>
struct Tile {
    static constexpr int LD = KMAJOR ? kBK : BMN + 4;                // LDS row stride in floats
    static constexpr int ELEMS = KMAJOR ? BMN * LD : kBK * LD;       // floats per LDS buffer
    static constexpr int NV = BMN * kBK / 4 / kGemmThreads;          // 16-byte pieces per thread
    floatx4 r[NV];

    // (mn, k) of the first element of the i-th piece of thread `threadIdx.x`
    static __device__ __forceinline__ void coords(int i, int& mn, int& k) {
        const int f = threadIdx.x + i * kGemmThreads;
        if (KMAJOR) {
            mn = f / (kBK / 4);
            k = (f % (kBK / 4)) * 4;
        } else {
            k = f / (BMN / 4);
            mn = (f % (BMN / 4)) * 4;
        }
    }
    // element offset of piece i from the tile origin in HBM / in LDS
    static __device__ __forceinline__ size_t gmem_offset(int i, size_t ld) {
        int mn, k;
        coords(i, mn, k);
        return KMAJOR ? mn * ld + k : k * ld + mn;
    }
    static __device__ __forceinline__ int lds_offset(int i) {
        int mn, k;
        coords(i, mn, k);
        return KMAJOR ? mn * LD + (((k >> 2) ^ ((mn >> 2) & 3)) << 2) : k * LD + mn;
    }

    // fast path: `base` is the tile origin (uniform), `off` this thread's byte offset of piece i.  A buffer load
    // takes the base as a scalar resource and the offset as one 32-bit VGPR, so moving along k costs scalar adds
    // only (a flat global load needs a 64-bit vector add per piece and tile).
    // `bytes` = size of the buffer from `base` on: a load that starts beyond it returns zeros instead of touching
    // memory (the loads of the last tiles of a k that ends inside a tile can pass the end of the operand).
    __device__ __forceinline__ void load_fast(int i, const float* __restrict__ base, unsigned off,
                                              unsigned bytes = 0xffffffffu) {
        typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)bytes, 0x00020000);
        r[i] = __builtin_bit_cast(floatx4, (uintx4)__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    }

    // checked path: zero fill outside [0, MN) x [0, K), scalar loads where 16-byte loads are not legal
    __device__ __forceinline__ void load_safe(int i, const float* __restrict__ p, size_t ld, size_t mn0, size_t k0,
                                              size_t MN, size_t K, bool vec_ok) {
        int tmn, tk;
        coords(i, tmn, tk);
        const size_t mn = mn0 + tmn, k = k0 + tk;
        const float* q = KMAJOR ? p + mn * ld + k : p + k * ld + mn;
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

    __device__ __forceinline__ void store_op(float* __restrict__ lds_thread_base, int i) const {
        // lds_thread_base = buffer + lds_offset(0); the further pieces sit at compile-time distances
        constexpr int STEP = KMAJOR ? (kGemmThreads / (kBK / 4)) * LD : (kGemmThreads / (BMN / 4)) * LD;
        *reinterpret_cast<floatx4*>(lds_thread_base + i * STEP) = r[i];
    }
    // the same store for a tile that starts at k0 and may reach past k_end: values at k >= k_end become zero
    __device__ __forceinline__ void store_masked(float* __restrict__ lds_thread_base, int i, size_t k0,
                                                 size_t k_end) const {
        constexpr int STEP = KMAJOR ? (kGemmThreads / (kBK / 4)) * LD : (kGemmThreads / (BMN / 4)) * LD;
        int tmn, tk;
        coords(i, tmn, tk);
        const size_t k = k0 + tk;
        floatx4 v = r[i];
        if (KMAJOR) {
            if (k + 0 >= k_end) v.x = 0.f;
            if (k + 1 >= k_end) v.y = 0.f;
            if (k + 2 >= k_end) v.z = 0.f;
            if (k + 3 >= k_end) v.w = 0.f;
        } else if (k >= k_end) {
            v = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        *reinterpret_cast<floatx4*>(lds_thread_base + i * STEP) = v;
    }
};

// The fragments one lane feeds to the MFMAs of one k-group (4 steps) for its T blocks of 32 rows.
template <int BMN, bool KMAJOR, int T>
struct Frag {
    using Tl = Tile<BMN, KMAJOR>;
    using V = std::conditional_t<KMAJOR, floatx4, typename VecOf<T>::type>;
    static constexpr int N = KMAJOR ? T : 4;  // LDS reads per k-group
    V v[N];

    // this lane's read base inside an LDS buffer for k-group g: w0 = first row of the wave's slab.  A k-contiguous
    // tile is swizzled (see Tile), which makes the column of piece 2g + lk a per-lane constant for each g; the other
    // layout reaches group g through an immediate offset, so its two bases are the same.
    static __device__ __forceinline__ int lane_base(int w0, int l32, int lk, int g) {
        const int row = w0 + l32;
        return KMAJOR ? row * Tl::LD + ((((g << 1) + lk) ^ ((row >> 2) & 3)) << 2) : (lk * 4) * Tl::LD + w0 + l32 * T;
    }
    // n-th read of k-group g; lane_ptr = buffer + lane_base(.., g)
    __device__ __forceinline__ void read_op(int n, const float* __restrict__ lane_ptr, int g) {
        if (KMAJOR) v[n] = *reinterpret_cast<const V*>(lane_ptr + n * 32 * Tl::LD);
        else v[n] = *reinterpret_cast<const V*>(lane_ptr + (g * 8 + n) * Tl::LD);
    }
    // operand of block t in step c
    __device__ __forceinline__ float get(int t, int c) const {
        if constexpr (KMAJOR) return v[t][c];
        else if constexpr (T == 1) return v[c];
        else return v[c][t];
    }
    // tile row (or column) that block t, block-row b stands for
    static __device__ __forceinline__ int index_of(int t, int b) { return KMAJOR ? t * 32 + b : b * T + t; }
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
    unsigned flat_batches;  // staged kernels: number of batches folded into grid.x (0: the batch is grid.z)
    // split-K: workgroup y handles k-tiles [y * split_tiles, (y + 1) * split_tiles) and writes its C tile at
    // C + y * split_stride (the launcher points C at a buffer of partial products); one split = the whole of k
    size_t split_tiles, split_stride;
    // Tail in pieces (staged kernels, one unbatched product of whole tiles; tail_splits == 0: off).  The first
    // tail_first workgroups (a whole number of rounds of the CUs) compute whole tiles as ever; the tiles that would
    // start one more round are cut along k instead, tail_splits workgroups per tile with split_tiles k-tiles each,
    // and piece p of tail tile t goes to tail_part + (t * tail_splits + p) * BM * BN as a dense BM x BN block with no
    // epilogue arithmetic; gemm_tail_reduce_kernel adds a tile's pieces in piece order and applies alpha, beta and the
    // extras.  Every CU then carries the same work instead of a quarter of them carrying one tile more.
    unsigned tail_first, tail_splits;
    float* tail_part;
    int a_vec, b_vec;  // 16-byte vector loads are legal for this operand
    int c_vec;         // vector stores to C are legal (alignment, ldc and n multiples of 4)
    int bounded_tail;  // edge kernels: an m or n that ends inside a 16-byte piece reads a few floats past the
                       // operand's end in the last k rows, so the last tiles must load through bounded descriptors
    // Optional epilogue of the fused Linear entry points, applied to v = alpha * acc + beta * C in this order:
    // v += bias[col]; v = max(v, 0) when relu; v = 0 where gate[row][col] <= 0 (gate laid out like C, only with
    // beta == 0).  All null / 0 for the plain products.
    const float* bias;
    const float* gate;
    int relu;
};

// the epilogue extras on one value (the rounding of the separate add / relu / mask kernels: one IEEE add, selects)
__device__ __forceinline__ float gemm_extras(float v, bool has_bias, float bias, bool relu) {
    if (has_bias) v = __fadd_rn(v, bias);
    if (relu) v = v > 0.f ? v : 0.f;
    return v;
}

// Logical tile id from the hardware workgroup id.  Hardware deals consecutive ids round-robin to the 8
// XCDs; give each XCD a contiguous run of logical ids, then walk C in column groups of GM tile-rows.
// GM = 4: the two workgroups that share a CU do not advance at the same speed (the one placed first wins the
// arbitration and runs about 17 % ahead), so an XCD's resident workgroups split into an early and a late half
// that stop sharing L2 lines after a few dozen k-tiles.  Each half is a run of 32 consecutive ids; 4 rows x 8
// columns is the shape of such a run with the fewest A and B panel bytes for the 256 x 128 tile (8 rows x 4
// columns fetched 47 % more from the fabric, measured with FETCH_SIZE).
__device__ __forceinline__ unsigned xcd_contiguous(unsigned pid, unsigned total) {
    return ((total & 7u) == 0) ? (pid & 7u) * (total >> 3) + (pid >> 3) : pid;
}
__device__ __forceinline__ void tile_coords(unsigned id, unsigned tiles_m, unsigned tiles_n, unsigned& tm,
                                            unsigned& tn) {
    constexpr unsigned GM = 4;
    const unsigned per_group = GM * tiles_n;
    const unsigned group = id / per_group;
    const unsigned first_m = group * GM;
    const unsigned gsize = (tiles_m - first_m < GM) ? (tiles_m - first_m) : GM;
    const unsigned in_group = id % per_group;
    tm = first_m + in_group % gsize;
    tn = in_group / gsize;
}

// MODE 0 (fast): whole tiles in m and n, C fit for vector stores; no bounds checks in the loop.  A k that is not a whole
//                number of tile pairs is handled by the last two pairs of steps: their loads see the operand's true
//                size (buffer bounds: nothing past the end is touched) and their LDS writes zero what lies past k.
// MODE 1 (edge): as fast, but M and N may end inside a tile and C may need scalar stores: the per-thread load
//                offsets are clamped once, before the loop, to the last valid row or to the 16-byte piece that holds
//                it (rows and columns past the edge then hold copies of valid data or whatever follows the edge in
//                memory, which only reach C elements that are never stored), and the epilogue checks bounds.  When
//                such a piece sticks out of the operand (M or N not a multiple of 4 with a non-k-contiguous operand)
//                the last tiles load through bounded descriptors like the tail of a ragged k.  The loop is the fast loop.
// MODE 2 (checked): every load checked and zero-filled; only for leading dimensions beyond 32-bit byte offsets.
// TAILS: the launch has its tail in pieces (GemmArgs::tail_part); instantiated for the 128 x 128 and 64 x 64 tiles only
// (the 256 x 128 kernels' register budget has no room for it, and the planner never asks them).
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int MODE, bool TAILS = false>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmArgs g) {
    constexpr bool SAFE = MODE == 2;
    constexpr int BK = kBK;
    using TA = Tile<BM, A_KMAJOR>;
    using TB = Tile<BN, B_KMAJOR>;
    constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;
    using FA = Frag<BM, A_KMAJOR, TM>;
    using FB = Frag<BN, B_KMAJOR, TN>;
    extern __shared__ __attribute__((aligned(16))) float lds[];  // A buffers 0/1, then B buffers 0/1
    float* const As0 = lds;
    float* const Bs0 = lds + 2 * TA::ELEMS;

    // Batched products with few tiles per batch fold the batch into grid.x (flat_batches != 0): the contiguous run of
    // logical ids an XCD gets then holds whole batches, so the tiles that share a batch's A and B panels share an L2.
    // With the batch in grid.z the hardware deals the tiles of one batch out over all eight XCDs and every tile
    // fetches its panels alone (32 x 512 x 512 x 4096: 513 -> 46x us).
    unsigned tm, tn;
    size_t z = blockIdx.z;
    unsigned split = blockIdx.y;
    bool piece = false;     // a k range of a tail tile: goes to the partial buffer as it is
    unsigned piece_id = 0;
    if constexpr (TAILS) {
        if (blockIdx.x < g.tail_first) {
            tile_coords(xcd_contiguous(blockIdx.x, g.tail_first), g.tiles_m, g.tiles_n, tm, tn);
        } else {
            piece = true;
            piece_id = blockIdx.x - g.tail_first;
            split = piece_id % g.tail_splits;
            tile_coords(g.tail_first + piece_id / g.tail_splits, g.tiles_m, g.tiles_n, tm, tn);
        }
    } else {
        const unsigned per_batch = g.tiles_m * g.tiles_n;
        if (g.flat_batches) {
            const unsigned id = xcd_contiguous(blockIdx.x, per_batch * g.flat_batches);
            z = id / per_batch;
            tile_coords(id % per_batch, g.tiles_m, g.tiles_n, tm, tn);
        } else {
            tile_coords(xcd_contiguous(blockIdx.x, per_batch), g.tiles_m, g.tiles_n, tm, tn);
        }
    }
    const float* A = g.A + (z % g.nba) * g.a_chunk;
    const float* B = g.B + (z % g.nbb) * g.b_chunk;
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

    // this workgroup's range of k
    const bool whole_k = TAILS && !piece;
    const size_t k_begin = whole_k ? 0 : (size_t)split * g.split_tiles * BK;
    const size_t k_end = (whole_k || k_begin + g.split_tiles * BK >= g.K) ? g.K : k_begin + g.split_tiles * BK;
    // 32-bit tile counter: there is no scalar 64-bit ordered compare, and a vector compare in the loop costs MFMA time
    const unsigned KT = (unsigned)((k_end - k_begin + BK - 1) / BK);
    // fast / edge kernels: a k range that is not a whole number of tile pairs ends in tiles whose values past k_end
    // are zeroed on their way into LDS (the last two pairs of steps run the masking variant of the step)
    const bool ragged_k = !SAFE && ((k_end - k_begin) % (2 * BK) != 0 || (MODE == 1 && g.bounded_tail != 0));
    constexpr int NM = TM * TN;         // MFMAs per step
    constexpr int NMF = 4 * NM;         // MFMAs per k-group
    constexpr int NR = FA::N + FB::N;   // fragment reads per k-group
    constexpr int NL = TA::NV + TB::NV; // 16-byte global loads (and LDS writes) per thread per tile

    // per-thread constants: where this thread's pieces go in LDS, where its lane reads fragments, and (fast
    // path) the byte offsets of its pieces from the tile origin in HBM
    float* const a_wr = As0 + TA::lds_offset(0);
    float* const b_wr = Bs0 + TB::lds_offset(0);
    const float* const a_rd[2] = {As0 + FA::lane_base(wm0, l32, lk, 0), As0 + FA::lane_base(wm0, l32, lk, 1)};
    const float* const b_rd[2] = {Bs0 + FB::lane_base(wn0, l32, lk, 0), Bs0 + FB::lane_base(wn0, l32, lk, 1)};
    unsigned a_off[TA::NV], b_off[TB::NV];
#pragma unroll
    for (int i = 0; i < TA::NV; i++) {
        int tmn, tk;
        TA::coords(i, tmn, tk);
        if (MODE == 1) {
            const size_t last = A_KMAJOR ? g.M - 1 : (g.M - 1) / 4 * 4;  // the row, or the piece that holds row M - 1
            if (m0 + tmn > last) tmn = (int)(last - m0);
        }
        a_off[i] = (unsigned)((A_KMAJOR ? tmn * g.lda + tk : tk * g.lda + tmn) * sizeof(float));
    }
#pragma unroll
    for (int i = 0; i < TB::NV; i++) {
        int tmn, tk;
        TB::coords(i, tmn, tk);
        if (MODE == 1) {
            const size_t last = B_KMAJOR ? g.N - 1 : (g.N - 1) / 4 * 4;
            if (n0 + tmn > last) tmn = (int)(last - n0);
        }
        b_off[i] = (unsigned)((B_KMAJOR ? tmn * g.ldb + tk : tk * g.ldb + tmn) * sizeof(float));
    }
    const float* const a_org = A_KMAJOR ? A + m0 * g.lda : A + m0;  // tile origin at k = 0
    const float* const b_org = B_KMAJOR ? B + n0 * g.ldb : B + n0;
    // one past the last element of each operand
    const float* const a_end = A_KMAJOR ? A + (g.M - 1) * g.lda + g.K : A + (g.K - 1) * g.lda + g.M;
    const float* const b_end = B_KMAJOR ? B + (g.N - 1) * g.ldb + g.K : B + (g.K - 1) * g.ldb + g.N;
    auto bytes_left = [](const float* base, const float* end) {
        const size_t n = base < end ? (size_t)(end - base) * sizeof(float) : 0;
        return (unsigned)(n < 0xffffffffull ? n : 0xffffffffull);
    };

    // Tiles wait in registers for two tile times between their global loads and their LDS writes (slot t % 2),
    // which covers the HBM latency also when a workgroup has a CU to itself.
    TA ta[2];
    TB tb[2];
    // Fast / edge kernels: a k-contiguous operand is addressed through a running tile-origin pointer (a_tile, b_tile)
    // that tile_step moves along k with one scalar add; a strided operand's origin is recomputed from k0 for every
    // tile.  (Running pointers for the strided operands as well save a few scalar instructions per tile and 0.5 % of
    // the TN product's time, but its workgroups then drift apart in k and the L2 of each XCD misses 1.6 x as many
    // bytes: measured 509 -> 790..950 MiB per 4096-cubed product.)  The checked kernels address through k0.
    const float* a_tile = a_org;
    const float* b_tile = b_org;
    const size_t a_step = A_KMAJOR ? (size_t)BK : (size_t)BK * g.lda;  // elements between the origins of two tiles
    const size_t b_step = B_KMAJOR ? (size_t)BK : (size_t)BK * g.ldb;
    auto load_op = [&](auto slot_tag, int v, size_t k0, auto bounded_tag) {
        constexpr int S = decltype(slot_tag)::value;
        constexpr bool BOUNDED = decltype(bounded_tag)::value;  // give the buffer its true size (last tiles only)
        if (v < TA::NV) {
            if (!SAFE) {
                const float* org = A_KMAJOR ? a_tile : a_org + k0 * g.lda;
                ta[S].load_fast(v, org, a_off[v], BOUNDED ? bytes_left(org, a_end) : 0xffffffffu);
            } else ta[S].load_safe(v, A, g.lda, m0, k0, g.M, k_end, g.a_vec != 0);
        } else {
            if (!SAFE) {
                const float* org = B_KMAJOR ? b_tile : b_org + k0 * g.ldb;
                tb[S].load_fast(v - TA::NV, org, b_off[v - TA::NV], BOUNDED ? bytes_left(org, b_end) : 0xffffffffu);
            } else tb[S].load_safe(v - TA::NV, B, g.ldb, n0, k0, g.N, k_end, g.b_vec != 0);
        }
    };
    // k0: first k of the tile being stored (used by the masking variant only)
    auto store_op = [&](auto slot_tag, int w, int buf, size_t k0, auto masked_tag) {
        constexpr int S = decltype(slot_tag)::value;
        if constexpr (decltype(masked_tag)::value) {
            if (w < TA::NV) ta[S].store_masked(a_wr + buf * TA::ELEMS, w, k0, k_end);
            else tb[S].store_masked(b_wr + buf * TB::ELEMS, w - TA::NV, k0, k_end);
        } else {
            if (w < TA::NV) ta[S].store_op(a_wr + buf * TA::ELEMS, w);
            else tb[S].store_op(b_wr + buf * TB::ELEMS, w - TA::NV);
        }
    };
    // fragment register sets: k-group 0 of a tile lives in set 0, k-group 1 in set 1
    FA fa[2];
    FB fb[2];
    auto read_op = [&](int set, int n, int buf, int grp) {
        if (n < FA::N) fa[set].read_op(n, a_rd[grp] + buf * TA::ELEMS, grp);
        else fb[set].read_op(n - FA::N, b_rd[grp] + buf * TB::ELEMS, grp);
    };

    // One tile = two k-groups of 4 steps of NM MFMAs.  The other instructions are dealt out behind the MFMAs,
    // pinned with sched_barrier (left alone, the scheduler sinks every load next to its use):
    //   group 0: global loads of tile t+2, fragment reads of group 1, LDS writes of tile t+1; then the barrier
    //   group 1: fragment reads of group 0 of tile t+1
    // Every tile runs the same code, the last ones included: past the end of k the fast and edge kernels repeat the
    // loads of the last tile, the checked kernels load zeros, and the LDS writes and the barrier still happen.  One
    // loop body without peeled tails keeps the accumulators in one place.  The tile's parity is a template
    // argument, so all LDS addresses are immediates.  The masking variant of the step (second template flag) is the
    // same instruction stream with bounded loads and k-masked LDS writes; it only runs for the last two pairs of
    // steps of a ragged k range.
    constexpr int E0 = NL + NR + NL;
    constexpr int PER0 = (E0 + NMF - 1) / NMF;
    constexpr int PER1 = (NR + (NMF + 1) / 2 - 1) / ((NMF + 1) / 2);  // reads land in the first half of group 1
    auto tile_step = [&](unsigned kt, auto parity_tag, auto masked_tag) {
        constexpr int S = decltype(parity_tag)::value;  // kt % 2: LDS buffer and register slot of this tile
        using SCur = std::integral_constant<int, S>;
        using SNext = std::integral_constant<int, S ^ 1>;
        // this step loads tile min(kt + 2, KT - 1) (the checked kernels: tile kt + 2, zeros past the end)
        const size_t k_load = k_begin + (size_t)((SAFE || kt + 2 < KT) ? kt + 2 : KT - 1) * BK;
        const size_t k_store = k_begin + (size_t)(kt + 1) * BK;
#pragma unroll
        for (int grp = 0; grp < 2; grp++) {
#pragma unroll
            for (int n = 0; n < NMF; n++) {
                const int c = n / NM, q = n % NM;
                const int i = q / TN, j = q % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[grp].get(i, c), fb[grp].get(j, c), acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (grp == 0) {
#pragma unroll
                    for (int e = n * PER0; e < (n + 1) * PER0 && e < E0; e++) {
                        if (e < NL) load_op(SCur{}, e, k_load, masked_tag);  // slot S is free: tile kt is in LDS
                        else if (e < NL + NR) read_op(1, e - NL, S, 1);
                        else store_op(SNext{}, e - NL - NR, S ^ 1, k_store, masked_tag);
                    }
                } else {
#pragma unroll
                    for (int e = n * PER1; e < (n + 1) * PER1 && e < NR; e++) read_op(0, e, S ^ 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (grp == 0) {
                if (!SAFE && kt + 3 < KT) {  // the loads of this step are out: move on to the next step's tile
                    a_tile += a_step;
                    b_tile += b_step;
                }
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using Plain = std::false_type;
    using Masked = std::true_type;

    // prologue: tile 0 goes straight to LDS buffer 0, tile 1 starts its flight in slot 1
    a_tile += (A_KMAJOR ? k_begin : k_begin * g.lda);
    b_tile += (B_KMAJOR ? k_begin : k_begin * g.ldb);
    auto advance = [&](unsigned next_tile) {  // to the origin of tile min(next_tile, KT - 1)
        if (!SAFE && next_tile < KT) {
            a_tile += a_step;
            b_tile += b_step;
        }
    };
    if (__builtin_expect(ragged_k, 0)) {
#pragma unroll
        for (int v = 0; v < NL; v++) load_op(P0{}, v, k_begin, Masked{});
        advance(1);
#pragma unroll
        for (int v = 0; v < NL; v++) load_op(P1{}, v, k_begin + ((SAFE || KT > 1) ? BK : 0), Masked{});
#pragma unroll
        for (int w = 0; w < NL; w++) store_op(P0{}, w, 0, k_begin, Masked{});
    } else {
#pragma unroll
        for (int v = 0; v < NL; v++) load_op(P0{}, v, k_begin, Plain{});
        advance(1);
#pragma unroll
        for (int v = 0; v < NL; v++) load_op(P1{}, v, k_begin + ((SAFE || KT > 1) ? BK : 0), Plain{});
#pragma unroll
        for (int w = 0; w < NL; w++) store_op(P0{}, w, 0, k_begin, Plain{});
    }
    advance(2);
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NR; n++) read_op(0, n, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // Tiles go in pairs so that the loop body is one straight run of MFMAs.  A tile past the end of k adds nothing:
    // the masking steps zero it on its way into LDS, the checked kernels load it as zeros.
    const unsigned kt_plain = !ragged_k ? KT : (KT > 4 ? ((KT + 1) & ~1u) - 4 : 0);
    unsigned kt = 0;
    for (; kt < kt_plain; kt += 2) {
        tile_step(kt, P0{}, Plain{});
        tile_step(kt + 1, P1{}, Plain{});
    }
    if constexpr (!SAFE) {
        if (__builtin_expect(kt < KT, 0)) {  // ragged k only: the last two pairs, whose stores may hold values past k_end
            do {
                tile_step(kt, P0{}, Masked{});
                tile_step(kt + 1, P1{}, Masked{});
                kt += 2;
            } while (kt < KT);
        }
    }

    // epilogue.  Accumulator register r of lane l belongs to block row (r/4)*8 + (l/32)*4 + r%4 and block
    // column l%32; Frag::index_of turns those into tile rows and columns.  With B k-contiguous a store
    // instruction writes two 128-byte row segments; otherwise a lane owns TN adjacent columns and stores them as
    // one vector.  With beta != 0 the old values of a row of blocks are read together before any is used; C is
    // not read at all when beta == 0.
    // where the tile's element (0, 0) is stored, and the row pitch there
    float* const c_org = piece ? g.tail_part + (size_t)piece_id * (BM * BN)
                               : g.C + z * g.c_chunk + (size_t)split * g.split_stride + m0 * g.ldc + n0;
    const size_t c_ld = piece ? (size_t)BN : g.ldc;
    const float alpha = piece ? 1.f : g.alpha, beta = piece ? 0.f : g.beta;
    const bool use_c = beta != 0.f;
    // gated implies !use_c
    const bool has_bias = !piece && g.bias != nullptr, relu = !piece && g.relu != 0, gated = !piece && g.gate != nullptr;
    // the gate value of a C element sits at the same offset from g.gate as the element from g.C
    const ptrdiff_t gate_bytes = gated ? reinterpret_cast<const char*>(g.gate) - reinterpret_cast<const char*>(g.C) : 0;

    const bool use_old = use_c || gated;
    const bool any_extras = has_bias || relu || gated;
    // The accumulators are taken out of their AGPRs one row of blocks at a time through an explicit
    // v_accvgpr_read (the "a" constraint pins the value in an AGPR up to that point).  Left to itself the
    // register allocator copies all of them to VGPRs at the loop exit, which doubles the kernel's register
    // count and halves its occupancy.  The instruction is opaque to the hazard recogniser, so the wait states an
    // AGPR read needs after the MFMA that wrote it are spent explicitly first.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    constexpr bool VEC_C = !SAFE && !B_KMAJOR && TN > 1;
    using VC = typename VecOf<VEC_C ? TN : 1>::type;
    const bool vec_c = VEC_C && (MODE == 0 || g.c_vec != 0 || piece);  // edge kernels also serve a C that needs scalar stores
#pragma unroll
    for (int i = 0; i < TM; i++) {
        float res[TN][16], old[TN][16];
        float* cptr[TN];
        const float* optr[TN];  // where the old values come from: C itself, or the gate
        float bias_v[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const size_t col = n0 + wn0 + FB::index_of(j, l32);
            cptr[j] = c_org + (size_t)(wm0 + FA::index_of(i, lk * 4)) * c_ld + (col - n0);
            optr[j] = reinterpret_cast<const float*>(reinterpret_cast<const char*>(cptr[j]) + gate_bytes);
            bias_v[j] = (has_bias && (MODE == 0 || col < g.N)) ? g.bias[col] : 0.f;
        }
        constexpr int RSTEP = A_KMAJOR ? 1 : TM;  // tile rows between consecutive block rows
        auto row_of = [&](int r) { return ((r >> 2) * 8 + (r & 3)) * RSTEP; };  // relative to block row lk*4
        auto in_range = [&](int j, int r) {
            if (MODE == 0 || piece) return true;  // a piece is a whole dense tile in the partial buffer
            const size_t row = m0 + wm0 + FA::index_of(i, lk * 4 + (r >> 2) * 8 + (r & 3));
            const size_t col = n0 + wn0 + FB::index_of(j, l32);
            return row < g.M && col < g.N;
        };
        if (use_old) {  // the old C values, or the gate values when gated
#pragma unroll
            for (int r = 0; r < 16; r++) {
                if (vec_c) {
                    VC o = {};
                    if (in_range(0, r)) o = *reinterpret_cast<const VC*>(optr[0] + (size_t)row_of(r) * c_ld);
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        if constexpr (VEC_C) old[j][r] = o[j];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        old[j][r] = in_range(j, r) ? optr[j][(size_t)row_of(r) * c_ld] : 0.f;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(res[j][r]) : "a"(acc[i][j][r]));
#pragma unroll
        for (int r = 0; r < 16; r++) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                float v = alpha * res[j][r];
                if (use_c) v += beta * old[j][r];
                res[j][r] = v;
            }
        }
        if (any_extras) {  // one uniform branch: the plain products skip all of it
#pragma unroll
            for (int r = 0; r < 16; r++) {
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    float v = gemm_extras(res[j][r], has_bias, bias_v[j], relu);
                    if (gated) v = old[j][r] <= 0.f ? 0.f : v;
                    res[j][r] = v;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            if (vec_c) {
                VC o;
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    if constexpr (VEC_C) o[j] = res[j][r];
                }
                if (in_range(0, r)) *reinterpret_cast<VC*>(cptr[0] + (size_t)row_of(r) * c_ld) = o;
            } else {
#pragma unroll
                for (int j = 0; j < TN; j++)
                    if (in_range(j, r)) cptr[j][(size_t)row_of(r) * c_ld] = res[j][r];
            }
        }
        // one row of blocks at a time
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int BM, int BN>
static int launch_gemm(zg_hip_ctx* ctx, GemmArgs& g, bool a_kmajor, bool b_kmajor, int mode, size_t batches) {
    g.tiles_m = (unsigned)ceil_div_sz(g.M, BM);
    g.tiles_n = (unsigned)ceil_div_sz(g.N, BN);
    const size_t kt_total = ceil_div_sz(g.K, kBK);
    dim3 grid(g.tiles_m * g.tiles_n, (unsigned)ceil_div_sz(kt_total, g.split_tiles), (unsigned)batches), block(kGemmThreads);
    if (g.tail_splits) grid = dim3(g.tail_first + (g.tiles_m * g.tiles_n - g.tail_first) * g.tail_splits, 1, 1);
    const size_t flat = (size_t)grid.x * batches;
    g.flat_batches = 0;
    if (!g.tail_splits && batches > 1 && grid.y == 1 && flat % 8 == 0 && flat < 0x7fffffffull) {
        g.flat_batches = (unsigned)batches;
        grid = dim3((unsigned)flat, 1, 1);
    }
#define ZG_GEMM(AK, BKM, MD)                                                                                        \
    do {                                                                                                            \
        constexpr size_t lds_bytes = 2 * (size_t)(Tile<BM, AK>::ELEMS + Tile<BN, BKM>::ELEMS) * sizeof(float);       \
        static_assert(lds_bytes <= 64 * 1024, "tile buffers exceed the default dynamic LDS limit");                 \
        if constexpr (BM * BN <= 128 * 128 && MD != 2) {                                                            \
            if (g.tail_splits) {                                                                                    \
                hipLaunchKernelGGL((gemm_kernel<BM, BN, AK, BKM, MD, true>), grid, block, lds_bytes, ctx->stream, g); \
                break;                                                                                              \
            }                                                                                                       \
        }                                                                                                           \
        hipLaunchKernelGGL((gemm_kernel<BM, BN, AK, BKM, MD>), grid, block, lds_bytes, ctx->stream, g);             \
    } while (0)
#define ZG_GEMM_LAYOUT(MD)                                      \
    do {                                                        \
        if (a_kmajor && b_kmajor) ZG_GEMM(true, true, MD);      \
        else if (a_kmajor && !b_kmajor) ZG_GEMM(true, false, MD); \
        else if (!a_kmajor && b_kmajor) ZG_GEMM(false, true, MD); \
        else ZG_GEMM(false, false, MD);                         \
    } while (0)
    if (mode == 0) {
        ZG_GEMM_LAYOUT(0);
    } else if (mode == 1) {
        ZG_GEMM_LAYOUT(1);
    } else {
        // the checked kernels exist for the 64 x 64 tile only: they serve leading dimensions beyond 32-bit byte offsets
        if constexpr (BM == 64 && BN == 64) ZG_GEMM_LAYOUT(2);
        else ZG_REQUIRE(false, "gemm: no checked kernel for this tile");
    }
#undef ZG_GEMM_LAYOUT
#undef ZG_GEMM
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// Small products (k <= 256, at most a few hundred 32x32 blocks of C): the staged kernel's fixed costs (two tiles of
// prologue, LDS round trips, a barrier per tile) dominate there.  Here a workgroup owns one 32x32 block of C and
// its four waves split k between them in groups of 8 (wave w takes groups w, w+4, ...).  Operands go straight
// from memory to the MFMA operand registers with the same k assignment as the staged kernel (lane half h, step c
// of group g: k = 8g + 4h + c), so a k-contiguous operand is one 16-byte load per lane and group; every load is
// guarded and zero-filled, so any shape and alignment is served.  The four partial blocks are added in wave
// order through LDS: the result does not depend on scheduling.
// `block` is the 32x32 block of C (row-major over tiles_n), z the batch, `part` 16 KiB of the caller's LDS.  With
// g.split_tiles != 0 the workgroup takes the groups [split * split_tiles, (split + 1) * split_tiles) of k only and
// writes its block at C + split * split_stride (the launcher points C at a buffer of partial products).
template <bool A_KMAJOR, bool B_KMAJOR>
__device__ __forceinline__ void gemm_tiny_block(const GemmArgs& g, unsigned block, unsigned split, size_t z,
                                                float (*part)[16][64]) {
    const size_t m0 = (size_t)(block / g.tiles_n) * 32, n0 = (size_t)(block % g.tiles_n) * 32;
    const float* A = g.A + (z % g.nba) * g.a_chunk;
    const float* B = g.B + (z % g.nbb) * g.b_chunk;
    float* C = g.C + z * g.c_chunk + (size_t)split * g.split_stride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const size_t K = g.K, groups = (K + 7) / 8;
    const size_t grp_begin = (size_t)split * g.split_tiles;
    const size_t grp_end = (g.split_tiles && grp_begin + g.split_tiles < groups) ? grp_begin + g.split_tiles : groups;

    auto fragment = [&](const float* P, bool kmajor, size_t ld, size_t idx, size_t limit, bool vec_ok, size_t grp) {
        floatx4 v = {0.f, 0.f, 0.f, 0.f};
        const size_t k0 = grp * 8 + (size_t)lk * 4;
        if (idx < limit && grp < grp_end && k0 < K) {
            if (kmajor) {
                const float* q = P + idx * ld + k0;
                if (vec_ok && k0 + 4 <= K) {
                    v = *reinterpret_cast<const floatx4*>(q);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        if (k0 + c < K) v[c] = q[c];
                }
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (k0 + c < K) v[c] = P[(k0 + c) * ld + idx];
            }
        }
        return v;
    };
    auto frag_a = [&](size_t grp) { return fragment(A, A_KMAJOR, g.lda, m0 + l32, g.M, g.a_vec != 0, grp); };
    auto frag_b = [&](size_t grp) { return fragment(B, B_KMAJOR, g.ldb, n0 + l32, g.N, g.b_vec != 0, grp); };

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    // 32 groups (k = 256) per round, 8 per wave: all of a wave's operand loads of a round are issued before its first
    // MFMA, so a round costs one memory round trip instead of one per group.  Most callers need a single round.
    constexpr int kMaxGroups = 8;
    for (size_t base = grp_begin; base < grp_end; base += 4 * kMaxGroups) {
        floatx4 a_frag[kMaxGroups], b_frag[kMaxGroups];
#pragma unroll
        for (int i = 0; i < kMaxGroups; i++) {
            const size_t grp = base + (size_t)wave + 4 * (size_t)i;
            a_frag[i] = frag_a(grp);  // zero beyond the range
            b_frag[i] = frag_b(grp);
        }
#pragma unroll
        for (int i = 0; i < kMaxGroups; i++) {
            if (base + (size_t)wave + 4 * (size_t)i < grp_end) {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_frag[i][c], b_frag[i][c], acc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 16; r++) part[wave][r][lane] = acc[r];
    __syncthreads();
    const float alpha = g.alpha, beta = g.beta;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int e = threadIdx.x + q * kGemmThreads, r = e >> 6, ln = e & 63;
        float s = part[0][r][ln];
        s += part[1][r][ln];
        s += part[2][r][ln];
        s += part[3][r][ln];
        const size_t row = m0 + (r >> 2) * 8 + (ln >> 5) * 4 + (r & 3), col = n0 + (ln & 31);
        if (row < g.M && col < g.N) {
            float v = alpha * s;
            if (beta != 0.f) v += beta * C[row * g.ldc + col];
            v = gemm_extras(v, g.bias != nullptr, g.bias ? g.bias[col] : 0.f, g.relu != 0);
            if (g.gate && g.gate[z * g.c_chunk + row * g.ldc + col] <= 0.f) v = 0.f;
            C[row * g.ldc + col] = v;
        }
    }
}

template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kGemmThreads) void gemm_tiny_kernel(GemmArgs g) {
    __shared__ float part[4][16][64];
    gemm_tiny_block<A_KMAJOR, B_KMAJOR>(g, blockIdx.x, blockIdx.y, blockIdx.z, part);
}

// The backward of a small Linear layer in one launch: the workgroups of the weight-gradient product (gw += gy^T x),
// those of the input-gradient product (gx = gy w, masked by the ReLU output that fed the layer) and those of the bias
// gradient (gb += column sums of gy) side by side.  Each workgroup runs the block of gemm_tiny_kernel or of
// col_reduce_kernel it would run in the separate launches, so the values are the same; the three results are
// independent of each other.
struct LinearBwdArgs {
    GemmArgs gw, gx;
    unsigned n_w, n_x;  // workgroups of the two products (n_x = 0: no input gradient)
    const float* gy;    // [R, inner]
    float* gb;          // null: no bias gradient
    float gb_beta;      // 1: gb += sums; 0: gb = sums (its zero fill was taken over)
    size_t R, inner;
    int log2_cx;
};
template <int V>
__global__ __launch_bounds__(kGemmThreads) void linear_bwd_small_kernel(LinearBwdArgs a) {
    __shared__ float part[4][16][64];
    static_assert(sizeof(part) >= sizeof(float) * kBlock * V && kBlock == kGemmThreads, "LDS of the column sums");
    const unsigned b = blockIdx.x;
    if (b < a.n_w) gemm_tiny_block<false, false>(a.gw, b, 0, 0, part);
    else if (b < a.n_w + a.n_x) gemm_tiny_block<true, false>(a.gx, b - a.n_w, 0, 0, part);
    else
        col_reduce_block<AxisSum, V>(a.gy, a.gb, nullptr, a.R, a.inner, a.log2_cx, a.R, 1.f, a.gb_beta, b - a.n_w - a.n_x, 0, 0,
                                     1, &part[0][0][0]);
}

// Thousands of very small products (m, n <= 8, k <= 64: per-sample transforms): a workgroup per product spends its
// launch on a block that is 1/16 full (65536 products of 8 x 8 x 8: 280 us, 2 % of 8 TB/s), so here a thread owns one
// element of one product and walks k; the threads of a product read the same few cache lines.  No epilogue extras.
template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(256) void gemm_micro_kernel(GemmArgs g, size_t batches) {
    const size_t mn = g.M * g.N, total = batches * mn;
    const size_t nt = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += nt) {
        const size_t z = i / mn, e = i - z * mn, r = e / g.N, c = e - r * g.N;
        const float* a = g.A + (z % g.nba) * g.a_chunk;
        const float* b = g.B + (z % g.nbb) * g.b_chunk;
        float acc = 0.f;
        for (size_t kk = 0; kk < g.K; kk++) {
            const float av = A_KMAJOR ? a[r * g.lda + kk] : a[kk * g.lda + r];
            const float bv = B_KMAJOR ? b[c * g.ldb + kk] : b[kk * g.ldb + c];
            acc = fmaf(av, bv, acc);
        }
        float* cp = g.C + z * g.c_chunk + r * g.ldc + c;
        float v = g.alpha * acc;
        if (g.beta != 0.f) v += g.beta * *cp;
        *cp = v;
    }
}
static bool gemm_is_micro(size_t m, size_t n, size_t k, size_t batches, const GemmArgs& g) {
    // up to 8 x 8 (16 x 16 x 16 with a k-contiguous B: 250 us a workgroup per product, 481 us this way)
    return batches >= 4096 && m <= 8 && n <= 8 && k <= 64 && !g.bias && !g.gate && !g.relu;
}
static int launch_gemm_micro(zg_hip_ctx* ctx, const GemmArgs& g, bool a_kmajor, bool b_kmajor, size_t batches) {
    size_t blocks = ceil_div_sz(batches * g.M * g.N, 256);
    if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
    const dim3 grid((unsigned)blocks), block(256);
    if (a_kmajor && b_kmajor) hipLaunchKernelGGL((gemm_micro_kernel<true, true>), grid, block, 0, ctx->stream, g, batches);
    else if (a_kmajor) hipLaunchKernelGGL((gemm_micro_kernel<true, false>), grid, block, 0, ctx->stream, g, batches);
    else if (b_kmajor) hipLaunchKernelGGL((gemm_micro_kernel<false, true>), grid, block, 0, ctx->stream, g, batches);
    else hipLaunchKernelGGL((gemm_micro_kernel<false, false>), grid, block, 0, ctx->stream, g, batches);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

static int launch_gemm_tiny(zg_hip_ctx* ctx, GemmArgs& g, bool a_kmajor, bool b_kmajor, size_t batches,
                            size_t splits = 1) {
    g.tiles_m = (unsigned)ceil_div_sz(g.M, 32);
    g.tiles_n = (unsigned)ceil_div_sz(g.N, 32);
    if (splits == 1) g.split_tiles = g.split_stride = 0;  // the whole of k in one workgroup per block
    dim3 grid(g.tiles_m * g.tiles_n, (unsigned)splits, (unsigned)batches), block(kGemmThreads);
    if (a_kmajor && b_kmajor) hipLaunchKernelGGL((gemm_tiny_kernel<true, true>), grid, block, 0, ctx->stream, g);
    else if (a_kmajor && !b_kmajor) hipLaunchKernelGGL((gemm_tiny_kernel<true, false>), grid, block, 0, ctx->stream, g);
    else if (!a_kmajor && b_kmajor) hipLaunchKernelGGL((gemm_tiny_kernel<false, true>), grid, block, 0, ctx->stream, g);
    else hipLaunchKernelGGL((gemm_tiny_kernel<false, false>), grid, block, 0, ctx->stream, g);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// Deep products on a few blocks (a Linear layer's forward at a small batch: 64 x 128 over k = 784; the graph
// convolution's first layer, 2708 x 16 over k = 1433): C = alpha * A B^T + beta * C with both operands k-contiguous, one
// 16 x 16 block of C per workgroup, so that even 64 x 128 gives 32 workgroups something to fetch.  The four waves deal
// k out in chunks of 16 (wave w takes chunks w, w + 4, ...); lane (r, q) of a wave loads values 4 q .. 4 q + 3 of its
// chunk for row r of A and for column r of B, sixteen bytes each, twelve chunks' loads in flight before the first is
// used, and element c of the two pieces feeds MFMA c of the chunk (v_mfma_f32_16x16x4_f32 adds over q in hardware).
// The waves' blocks are added in wave order through LDS; thread t finishes C element (t / 16, t % 16).  One launch
// where cutting k over workgroups takes two: 64 x 128 x 784 7.8 -> 5.4 us, 2708 x 16 x 1433 12.3 -> 7.8 us,
// 256 x 256 x 1024 9.9 -> 6.6 us.
constexpr int kDeepBatch = 12;  // chunks in flight per wave

__global__ __launch_bounds__(256) void gemm_deep_kernel(GemmArgs g) {
    __shared__ float part[4][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    const size_t tm = blockIdx.x / g.tiles_n, tn = blockIdx.x % g.tiles_n;
    size_t row = tm * 16 + r, col = tn * 16 + r;
    if (row >= g.M) row = g.M - 1;  // rows and columns past the edge repeat the last one; their sums are never stored
    if (col >= g.N) col = g.N - 1;
    // 16-byte buffer loads (served at any 4-byte alignment) from the block's first row, lane offsets in bytes
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
    const float* a_rows = g.A + tm * 16 * g.lda;
    const float* b_rows = g.B + tn * 16 * g.ldb;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a_rows), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(b_rows), 0, -1, 0x00020000);
    const unsigned a_off = (unsigned)(((row - tm * 16) * g.lda + 4 * q) * sizeof(float));
    const unsigned b_off = (unsigned)(((col - tn * 16) * g.ldb + 4 * q) * sizeof(float));
    const unsigned chunks = (unsigned)((g.K + 15) / 16);
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    // four values of k from chunk * 16 + 4 q on, zeros past K (the one chunk that K ends in loads value by value)
    auto piece = [&](__amdgpu_buffer_rsrc_t rsrc, const float* rows, unsigned off, unsigned chunk) {
        const unsigned k0 = chunk * 16 + 4 * (unsigned)q;
        if (k0 + 4 <= g.K) return __builtin_bit_cast(floatx4, (uintx4)__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(off + chunk * 64), 0, 0));
        floatx4 p;
#pragma unroll
        for (int c = 0; c < 4; c++) p[c] = (k0 + c < g.K) ? rows[off / 4 + chunk * 16 + c] : 0.f;
        return p;
    };
    for (unsigned c0 = wave; c0 < chunks; c0 += 4 * kDeepBatch) {
        floatx4 av[kDeepBatch], bv[kDeepBatch];
#pragma unroll
        for (int i = 0; i < kDeepBatch; i++) {
            const unsigned chunk = c0 + 4 * i;
            if (chunk < chunks) {
                av[i] = piece(a_rsrc, a_rows, a_off, chunk);
                bv[i] = piece(b_rsrc, b_rows, b_off, chunk);
            }
        }
#pragma unroll
        for (int i = 0; i < kDeepBatch; i++) {
            if (c0 + 4 * i < chunks) {
#pragma unroll
                for (int c = 0; c < 4; c++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i][c], bv[i][c], acc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) part[wave][lane][i] = acc[i];
    __syncthreads();
    // accumulator i of lane (r, q) is C element (4 q + i, r) of the block
    const int er = threadIdx.x >> 4, ec = threadIdx.x & 15;
    const int src_lane = (er >> 2) * 16 + ec, src_i = er & 3;
    float sum = part[0][src_lane][src_i];
#pragma unroll
    for (int w = 1; w < 4; w++) sum += part[w][src_lane][src_i];
    const size_t orow = tm * 16 + er, ocol = tn * 16 + ec;
    if (orow >= g.M || ocol >= g.N) return;
    const size_t at = orow * g.ldc + ocol;
    float v = g.alpha * sum;
    if (g.beta != 0.f) v += g.beta * g.C[at];
    v = gemm_extras(v, g.bias != nullptr, g.bias ? g.bias[ocol] : 0.f, g.relu != 0);
    if (g.gate && g.gate[at] <= 0.f) v = 0.f;
    g.C[at] = v;
}

// C = alpha * (sum of the split-K partial products, in split order) + beta * C.  P is [batch][split][M][N] dense.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* P, float* C, size_t M, size_t N, size_t ldc,
                                                            int splits, float alpha, float beta, size_t c_chunk,
                                                            const float* bias, const float* gate, int relu) {
    const size_t z = blockIdx.z;
    const float* p = P + z * (size_t)splits * M * N;
    float* c = C + z * c_chunk;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; i < M * N; i += nt) {
        float acc = p[i];
        for (int s0 = 1; s0 < splits; s0 += 8) {  // eight loads in flight, added in split order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (s0 + u < splits) v[u] = p[(size_t)(s0 + u) * M * N + i];
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (s0 + u < splits) acc += v[u];
        }
        const size_t r = i / N, col = i % N;
        float v = alpha * acc;
        if (beta != 0.f) v += beta * c[r * ldc + col];
        v = gemm_extras(v, bias != nullptr, bias ? bias[col] : 0.f, relu != 0);
        if (gate && gate[z * c_chunk + r * ldc + col] <= 0.f) v = 0.f;
        c[r * ldc + col] = v;
    }
}

// The same sum for many partial products (more than 16: a very long k): a workgroup takes 64 adjacent elements, wave w adds
// partial products w, w + 4, ... in that order with sixteen loads in flight, and the four wave sums are added in wave
// order.  (A thread walking 256 partial products eight at a time took 38 us for a 64 x 64 block.)
__global__ __launch_bounds__(256) void splitk_reduce_many_kernel(const float* P, float* C, size_t M, size_t N, size_t ldc,
                                                                 int splits, float alpha, float beta, size_t c_chunk,
                                                                 const float* bias, const float* gate, int relu) {
    __shared__ float smem[4][64];
    const size_t z = blockIdx.z;
    const float* p = P + z * (size_t)splits * M * N;
    float* c = C + z * c_chunk;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const size_t i = (size_t)blockIdx.x * 64 + lane;
    float acc = 0.f;
    if (i < M * N) {
        bool first = true;
        for (int s0 = w; s0 < splits; s0 += 4 * 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; u++)
                if (s0 + 4 * u < splits) v[u] = p[(size_t)(s0 + 4 * u) * M * N + i];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                if (s0 + 4 * u < splits) {
                    acc = first ? v[u] : acc + v[u];
                    first = false;
                }
            }
        }
    }
    smem[w][lane] = acc;
    __syncthreads();
    if (w == 0 && i < M * N) {
        const float sum = ((smem[0][lane] + smem[1][lane]) + smem[2][lane]) + smem[3][lane];
        const size_t r = i / N, col = i % N;
        float v = alpha * sum;
        if (beta != 0.f) v += beta * c[r * ldc + col];
        v = gemm_extras(v, bias != nullptr, bias ? bias[col] : 0.f, relu != 0);
        if (gate && gate[z * c_chunk + r * ldc + col] <= 0.f) v = 0.f;
        c[r * ldc + col] = v;
    }
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

// The same sum, four columns per thread: for a C fit for 16-byte accesses and no gate.
__global__ __launch_bounds__(256) void splitk_reduce_vec4_kernel(const float* P, float* C, size_t M, size_t N, size_t ldc,
                                                                 int splits, float alpha, float beta, size_t c_chunk,
                                                                 const float* bias, int relu) {
    const size_t z = blockIdx.z;
    const float4* p = reinterpret_cast<const float4*>(P + z * (size_t)splits * M * N);
    float* c = C + z * c_chunk;
    const size_t n4 = M * N / 4, stride4 = M * N / 4;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; i < n4; i += nt) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s0 = 0; s0 < splits; s0 += 8) {  // eight partial tiles' loads in flight, added in split order
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (s0 + u < splits) v[u] = p[(size_t)(s0 + u) * stride4 + i];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (s0 + u < splits) {
                    if (s0 + u == 0) {
                        acc = v[u];  // the first partial tile starts the sum (no 0 + x: keeps a -0 as it is)
                    } else {
                        acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w;
                    }
                }
            }
        }
        const size_t e = 4 * i, r = e / N, col = e % N;  // N is a multiple of 4: the four share a row
        float4* cp = reinterpret_cast<float4*>(c + r * ldc + col);
        float4 v = make_float4(alpha * acc.x, alpha * acc.y, alpha * acc.z, alpha * acc.w);
        if (beta != 0.f) {
            const float4 o = *cp;
            v.x += beta * o.x; v.y += beta * o.y; v.z += beta * o.z; v.w += beta * o.w;
        }
        const bool hb = bias != nullptr;
        v.x = gemm_extras(v.x, hb, hb ? bias[col] : 0.f, relu != 0);
        v.y = gemm_extras(v.y, hb, hb ? bias[col + 1] : 0.f, relu != 0);
        v.z = gemm_extras(v.z, hb, hb ? bias[col + 2] : 0.f, relu != 0);
        v.w = gemm_extras(v.w, hb, hb ? bias[col + 3] : 0.f, relu != 0);
        *cp = v;
    }
}

// The tail tiles of a product launched with its tail in pieces (GemmArgs::tail_part): C tile = alpha * (the tile's
// pieces, added in piece order) + beta * C, then the extras.  A thread owns four adjacent columns of one row; where C
// is not fit for 16-byte accesses, or the four columns reach past n, it handles them one by one.
template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tail_reduce_kernel(GemmArgs g) {
    constexpr unsigned V4 = BM * BN / 4, PER_TILE = V4 / 256;
    const unsigned t = blockIdx.x / PER_TILE, q = (blockIdx.x % PER_TILE) * 256 + threadIdx.x;
    unsigned tm, tn;
    tile_coords(g.tail_first + t, g.tiles_m, g.tiles_n, tm, tn);
    const size_t row = (size_t)tm * BM + q / (BN / 4), col = (size_t)tn * BN + (q % (BN / 4)) * 4;
    if (row >= g.M || col >= g.N) return;
    const float4* p = reinterpret_cast<const float4*>(g.tail_part + (size_t)t * g.tail_splits * (BM * BN)) + q;
    float4 acc = p[0];
    for (unsigned s0 = 1; s0 < g.tail_splits; s0 += 8) {  // eight pieces' loads in flight, added in piece order
        float4 v[8];
#pragma unroll
        for (unsigned u = 0; u < 8; u++)
            if (s0 + u < g.tail_splits) v[u] = p[(size_t)(s0 + u) * V4];
#pragma unroll
        for (unsigned u = 0; u < 8; u++) {
            if (s0 + u < g.tail_splits) {
                acc.x += v[u].x;
                acc.y += v[u].y;
                acc.z += v[u].z;
                acc.w += v[u].w;
            }
        }
    }
    const size_t at = row * g.ldc + col;
    const bool vec = g.c_vec != 0 && col + 4 <= g.N;
    const int live = vec ? 4 : (int)(g.N - col < 4 ? g.N - col : 4);
    float r[4] = {g.alpha * acc.x, g.alpha * acc.y, g.alpha * acc.z, g.alpha * acc.w};
    if (g.beta != 0.f) {
        float old[4] = {0.f, 0.f, 0.f, 0.f};
        if (vec) {
            const float4 o = *reinterpret_cast<const float4*>(g.C + at);
            old[0] = o.x, old[1] = o.y, old[2] = o.z, old[3] = o.w;
        } else {
            for (int j = 0; j < live; j++) old[j] = g.C[at + j];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) r[j] += g.beta * old[j];
    }
    if (g.bias || g.relu) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            r[j] = gemm_extras(r[j], g.bias != nullptr, (g.bias && j < live) ? g.bias[col + j] : 0.f, g.relu != 0);
    }
    if (g.gate) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (j < live && g.gate[at + j] <= 0.f) r[j] = 0.f;
    }
    if (vec) {
        *reinterpret_cast<float4*>(g.C + at) = make_float4(r[0], r[1], r[2], r[3]);
    } else {
        for (int j = 0; j < live; j++) g.C[at + j] = r[j];
    }
}

// ------------------------------------------------------------------------------------------------
// Launch planning for the staged kernels.  A CU works through its workgroups at a rate that depends on the tile
// shape but hardly on how many of them share the CU, so a launch takes (rounds the grid needs) x (time of one tile)
// plus a fixed cost (launch, first loads, the write of C by workgroups that all finish together).  When the tile
// count leaves the last round mostly empty, two other shapes of launch are priced with the same model: k cut over
// several workgroups per tile with a second kernel adding the partial tiles in a fixed order, and C cut into a block
// of whole large tiles that fills whole rounds plus one or two strips that are products of their own.  Plans depend
// on the shape only and are kept per context.
// ------------------------------------------------------------------------------------------------
struct GemmTileKind {
    size_t bm, bn;
    double eff;  // fraction of a CU's MFMA peak inside the loop
};
static const GemmTileKind kGemmTiles[3] = {{256, 128, 0.975}, {128, 128, 0.90}, {64, 64, 0.82}};
constexpr double kCuFlopsPerUs = 2.4e9 * 256 / 1e6;  // one CU: 256 fp32 MFMA FLOP per clock at 2.4 GHz
constexpr double kLaunchFixedUs = 8.0;
constexpr double kReduceFixedUs = 4.0, kReduceBytesPerUs = 4.0e6;

struct GemmPlan {
    enum Kind { kPlain, kSplit, kParts, kTail } kind = kPlain;
    int tile = 2;
    size_t splits = 1, per = 0;  // kSplit, kTail: number of k ranges and k-tiles per range
    size_t whole = 0;            // kTail: tiles computed whole (a whole number of rounds)
    size_t rm = 0, rn = 0;       // kParts: the main block is rm x rn tiles of 256 x 128
    double us = 0;               // the model's estimate
};

struct GemmPlanKey {
    size_t m, n, k, batches;
    int layout;
    bool operator<(const GemmPlanKey& o) const {
        if (m != o.m) return m < o.m;
        if (n != o.n) return n < o.n;
        if (k != o.k) return k < o.k;
        if (batches != o.batches) return batches < o.batches;
        return layout < o.layout;
    }
};
struct GemmPlanCache {
    std::map<GemmPlanKey, GemmPlan> plans;
    // zg_hip_gemm_timing: event pairs around every product launched while it is on
    bool timing = false, in_bracket = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pairs;
    size_t used = 0;
};

void gemm_plans_destroy(zg_hip_ctx* ctx) {
    if (ctx->gemm_plans)
        for (auto& pr : ctx->gemm_plans->pairs) {
            (void)hipEventDestroy(pr.first);
            (void)hipEventDestroy(pr.second);
        }
    delete ctx->gemm_plans;
    ctx->gemm_plans = nullptr;
}

static double gemm_tile_us(int tile, size_t kk) {
    const GemmTileKind& t = kGemmTiles[tile];
    return 2.0 * (double)(t.bm * t.bn) * (double)kk / (kCuFlopsPerUs * t.eff);
}
static size_t gemm_tiles_of(int tile, size_t m, size_t n, size_t batches) {
    return ceil_div_sz(m, kGemmTiles[tile].bm) * ceil_div_sz(n, kGemmTiles[tile].bn) * batches;
}

// Other shapes of launch are priced only when the model puts the plan in hand more than 12 % above the time the
// product would take with every CU busy at the large tile's rate.
static bool gemm_plan_is_slow(double us, size_t m, size_t n, size_t k, size_t batches, size_t n_cu) {
    const double ideal = 2.0 * (double)m * (double)n * (double)k * (double)batches / ((double)n_cu * kCuFlopsPerUs * 0.975);
    return us > 1.12 * ideal + kLaunchFixedUs;
}

static GemmPlan gemm_plan_compute_untailed(size_t n_cu, size_t m, size_t n, size_t k, size_t batches, int depth);

// One launch (plus the reduction when k is cut) for the whole product: the choice made before planning existed
// (`legacy`: rounds x padded tile work over 0.92 / 0.89 / 0.79, and the 64 x 64 split for few tiles and a deep k), and,
// when the model finds that slow, the best cut of k for any tile if the model prices it at least 8 % faster.
static GemmPlan gemm_plan_single(size_t m, size_t n, size_t k, size_t batches, size_t n_cu) {
    const size_t kt_total = ceil_div_sz(k, kBK);
    static const double legacy_eff[3] = {0.92, 0.89, 0.79};
    GemmPlan lp;
    double best = 0;
    for (int t = 0; t < 3; t++) {
        const double c = (double)ceil_div_sz(gemm_tiles_of(t, m, n, batches), n_cu) *
                         (double)(kGemmTiles[t].bm * kGemmTiles[t].bn) / legacy_eff[t];
        if (t == 0 || c < best) {  // ties go to the larger tile
            best = c;
            lp.tile = t;
        }
    }
    auto model = [&](int tile, size_t splits, size_t per) {
        const size_t wgs = gemm_tiles_of(tile, m, n, batches) * splits;
        double us = (double)ceil_div_sz(wgs, n_cu) * gemm_tile_us(tile, splits == 1 ? k : per * kBK) + kLaunchFixedUs;
        if (splits > 1) us += kReduceFixedUs + (double)(splits + 2) * (double)(m * n * batches) * 4.0 / kReduceBytesPerUs;
        return us;
    };
    if (lp.tile == 2) {
        const size_t t64 = gemm_tiles_of(2, m, n, batches);
        if (t64 < n_cu && kt_total >= 16) {
            // a range of k per CU for up to 32 tiles, two per CU beyond (500 x 256 x 2048, 32 tiles: 15.5 us in 16 ranges,
            // 12.9 us in 8), and at most 16 ranges: shorter ones are mostly prologue and the reduction reads them all
            // (256 x 256 x 4096: 17.0 us in 64 ranges of 64 values of k, 13.1 us in 16 of 256)
            // A very long k (a small layer's weight gradient over a batch of 65536 rows and more) keeps ranges of at least
            // 512 values of k and takes up to 256 of them: sixteen workgroups stream 30 GB/s each, whatever is left to
            // read (64 x 64 x 65536: 88 us in 16 ranges, 4.8 % of 8 TB/s).
            size_t splits = ceil_div_sz((t64 <= 32 ? 1 : 2) * n_cu, t64);
            if (splits > kt_total / 4) splits = kt_total / 4;
            size_t cap = kt_total / 16;
            if (cap < 16) cap = 16;
            if (cap > 256) cap = 256;
            if (splits > cap) splits = cap;
            size_t per = ceil_div_sz(kt_total, splits);
            per += per & 1;
            splits = ceil_div_sz(kt_total, per);
            // Worth it only when the k-tiles saved on the busiest CU outweigh the second launch and the short loops:
            // a 64x64 k-tile step takes about 0.27 us, the split's fixed costs about 4 us when every range has a CU
            // to itself (500 x 64 x 385: 12.4 us whole, 8.2 us in five ranges) and 6 us when the ranges take a second
            // round (768-cubed: 15.5 us whole, 20 us split four ways; 1024 x 500 x 512: 11.4 against 14.6).
            const double whole = (double)kt_total, busiest = (double)(ceil_div_sz(t64 * splits, n_cu) * per);
            const double fixed_us = t64 * splits <= n_cu ? 4.0 : 6.0;
            if (splits >= 2 && (whole - busiest) * 0.27 > fixed_us) {
                lp.kind = GemmPlan::kSplit;
                lp.splits = splits;
                lp.per = per;
            }
        }
    }
    lp.us = model(lp.tile, lp.splits, lp.per);
    if (lp.kind == GemmPlan::kSplit) return lp;
    if (!gemm_plan_is_slow(lp.us, m, n, k, batches, n_cu) || kt_total < 32) return lp;
    GemmPlan bp = lp;
    for (int t = 0; t < 3; t++) {
        for (size_t want = 2; want <= 16; want++) {
            size_t per = ceil_div_sz(kt_total, want);
            per += per & 1;
            if (per < 8) break;  // ranges shorter than 128 values of k are all prologue
            const size_t splits = ceil_div_sz(kt_total, per);
            if (splits < 2) continue;
            const double us = model(t, splits, per);
            if (us < bp.us) {
                bp.kind = GemmPlan::kSplit;
                bp.tile = t;
                bp.splits = splits;
                bp.per = per;
                bp.us = us;
            }
        }
    }
    return (bp.us < 0.92 * lp.us) ? bp : lp;
}

// The tail in pieces (GemmArgs::tail_part) for one unbatched product of whole tiles that needs more than one round:
// with T tiles on n_cu CUs, R = T / n_cu whole rounds and L = T % n_cu tiles left over, a plain launch takes R + 1
// tile times although the last round keeps only L of the CUs busy.  Cutting each left-over tile into s ranges of k
// gives L * s pieces of 1 / s tile each, spread over all CUs: R + ceil(L * s / n_cu) / s tile times, plus the second
// kernel that adds the pieces.  Measured per-round efficiencies (fraction of a CU's MFMA peak while a round runs: 0.975
// / 0.98 / 0.92 for the three tiles) are about equal, so what separates the tiles in this range of sizes is how much
// of the last round is empty, and with the tail in pieces the larger tiles win again: 1536-cubed 69 -> 58 us
// (64 x 64, s = 4), 2560-cubed 285 -> 243 us (64 x 64, s = 4), 3072-cubed 412 (in parts) -> 395 us (128 x 128, s = 4),
// 3584-cubed 93.5 % of the matrix peak (128 x 128, s = 8).
// (the 64 x 64 tile reads four times the operand bytes per flop of the 128 x 128 tile and falls to 0.85 when the
// operands outgrow what the L2s and the Infinity Cache keep of them between tiles: 3000-cubed and up)
static const double kRoundEff[3] = {0.975, 0.98, 0.92};
constexpr double kSmallTileBigOperandsEff = 0.85;
constexpr size_t kSmallTileBigOperands = (size_t)64 << 20;
constexpr double kPieceFixedUs = 1.5, kTailReduceFixedUs = 3.0;

static double gemm_rounds_us(int tile, double rounds, size_t m, size_t n, size_t k) {
    const GemmTileKind& t = kGemmTiles[tile];
    const double eff = (tile == 2 && (m + n) * k * sizeof(float) > kSmallTileBigOperands) ? kSmallTileBigOperandsEff
                                                                                           : kRoundEff[tile];
    return kLaunchFixedUs + rounds * 2.0 * (double)(t.bm * t.bn) * (double)k / (kCuFlopsPerUs * eff);
}

static bool gemm_plan_tail(size_t m, size_t n, size_t k, size_t n_cu, GemmPlan* out) {
    const size_t kt_total = ceil_div_sz(k, kBK);
    bool found = false;
    for (int t = 1; t < 3; t++) {  // the 128 x 128 and 64 x 64 kernels
        const size_t bm = kGemmTiles[t].bm, bn = kGemmTiles[t].bn;
        const size_t T = ceil_div_sz(m, bm) * ceil_div_sz(n, bn), R = T / n_cu, L = T % n_cu;
        if (R == 0 || L == 0 || T >= 0x7fffffffull / 16) continue;
        // Two 128 x 128 workgroups share a CU, and a CU that finishes early takes the next two in line: past three rounds
        // the CUs have drifted far enough apart that the pieces pile up on a few of them (4608-cubed, five rounds: 1537 us
        // against 1350 in parts; 5632-cubed, seven rounds: 2558 against 2502 whole).  The 64 x 64 tile runs six to eight
        // workgroups per CU and keeps its gain (2560-cubed, six rounds: 286 -> 258 us).
        if (t == 1 && R > 3) continue;
        for (size_t want = 2; want <= 8; want++) {
            size_t per = ceil_div_sz(kt_total, want);
            per += per & 1;
            if (per < 8) break;  // ranges shorter than 128 values of k are all prologue
            const size_t s = ceil_div_sz(kt_total, per);
            if (s < 2) continue;
            const size_t piece_rounds = ceil_div_sz(L * s, n_cu);
            const double us = gemm_rounds_us(t, (double)R + (double)piece_rounds * (double)per / (double)kt_total, m, n, k) +
                              kPieceFixedUs * (double)piece_rounds + kTailReduceFixedUs +
                              (double)((s + 1) * L * bm * bn) * 4.0 / kReduceBytesPerUs;
            if (!found || us < out->us) {
                found = true;
                out->kind = GemmPlan::kTail;
                out->tile = t;
                out->splits = s;
                out->per = per;
                out->whole = R * n_cu;
                out->us = us;
            }
        }
    }
    return found;
}

static GemmPlan gemm_plan_compute(size_t n_cu, size_t m, size_t n, size_t k, size_t batches, int depth) {
    GemmPlan best = gemm_plan_compute_untailed(n_cu, m, n, k, batches, depth);
    GemmPlan tail;
    if (batches == 1 && depth == 0 && gemm_plan_tail(m, n, k, n_cu, &tail)) {
        // against the plan in hand priced the same way (a plain launch: its rounds at the measured efficiencies)
        double in_hand = best.us;
        if (best.kind == GemmPlan::kPlain)
            in_hand = gemm_rounds_us(best.tile, (double)ceil_div_sz(gemm_tiles_of(best.tile, m, n, 1), n_cu), m, n, k);
        // Tiles that end inside C take the edge kernels, where the gain is less regular (4100 x 4100 x 1030 measured
        // none at all with any tile or number of pieces, 3000-cubed 438 -> 391 us): the model has to promise more there.
        const bool whole_tiles = m % kGemmTiles[tail.tile].bm == 0 && n % kGemmTiles[tail.tile].bn == 0;
        if (tail.us < (whole_tiles ? 0.97 : 0.92) * in_hand) return tail;
    }
    return best;
}

static GemmPlan gemm_plan_compute_untailed(size_t n_cu, size_t m, size_t n, size_t k, size_t batches, int depth) {
    GemmPlan best = gemm_plan_single(m, n, k, batches, n_cu);
    // C in parts: only for one product (no batch), at the top level, when the single launch is slow by the model
    const size_t tm_f = m / 256, tn_f = n / 128;
    if (depth == 0 && batches == 1 && tm_f >= 1 && tn_f >= 1) {
        if (gemm_plan_is_slow(best.us, m, n, k, 1, n_cu)) {
            GemmPlan bp = best;
            const size_t rm_lo = tm_f > 6 ? tm_f - 6 : 1, rn_lo = tn_f > 6 ? tn_f - 6 : 1;
            for (size_t rm = tm_f; rm >= rm_lo; rm--) {
                for (size_t rn = tn_f; rn >= rn_lo; rn--) {
                    const size_t main_tiles = rm * rn;
                    const double main_fill = (double)main_tiles / (double)(ceil_div_sz(main_tiles, n_cu) * n_cu);
                    if (main_fill < 0.95) continue;
                    double us = (double)ceil_div_sz(main_tiles, n_cu) * gemm_tile_us(0, k) + kLaunchFixedUs;
                    const size_t m1 = rm * 256, n1 = rn * 128;
                    if (n > n1) us += gemm_plan_single(m1, n - n1, k, 1, n_cu).us;
                    if (m > m1) us += gemm_plan_single(m - m1, n, k, 1, n_cu).us;
                    if (us < bp.us) {
                        bp.kind = GemmPlan::kParts;
                        bp.rm = rm;
                        bp.rn = rn;
                        bp.us = us;
                    }
                }
            }
            if (bp.us < 0.92 * best.us) best = bp;
        }
    }
    return best;
}

static GemmPlan gemm_plan(zg_hip_ctx* ctx, size_t m, size_t n, size_t k, size_t batches, bool a_kmajor, bool b_kmajor,
                          int depth) {
    if (!ctx->gemm_plans) ctx->gemm_plans = new GemmPlanCache();
    const GemmPlanKey key{m, n, k, batches, (a_kmajor ? 1 : 0) | (b_kmajor ? 2 : 0) | (depth ? 4 : 0)};
    auto it = ctx->gemm_plans->plans.find(key);
    if (it != ctx->gemm_plans->plans.end()) return it->second;
    const GemmPlan best = gemm_plan_compute((size_t)ctx->n_cu, m, n, k, batches, depth);
    ctx->gemm_plans->plans[key] = best;
    return best;
}

struct GemmExtras {
    const float* bias;
    const float* gate;
    int relu;
};

// the operand fields every kernel reads (the staged kernels' launcher adds the tile geometry and the split)
static GemmArgs gemm_args(const float* A, const float* B, float* C, size_t m, size_t n, size_t k, int trans_a, int trans_b,
                          size_t lda, size_t ldb, size_t ldc, float alpha, float beta, size_t nba, size_t nbb,
                          size_t a_chunk, size_t b_chunk, size_t c_chunk, const GemmExtras* extras) {
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
    g.bias = extras ? extras->bias : nullptr;
    g.gate = extras ? extras->gate : nullptr;
    g.relu = extras ? extras->relu : 0;
    g.nba = nba;
    g.nbb = nbb;
    g.a_chunk = a_chunk;
    g.b_chunk = b_chunk;
    g.c_chunk = c_chunk;
    g.a_vec = aligned16(A) && lda % 4 == 0 && a_chunk % 4 == 0;
    g.b_vec = aligned16(B) && ldb % 4 == 0 && b_chunk % 4 == 0;
    g.tiles_m = (unsigned)ceil_div_sz(m, 32);  // the unstaged kernel's blocks; the staged launcher sets its own
    g.tiles_n = (unsigned)ceil_div_sz(n, 32);
    g.flat_batches = 0;
    g.split_tiles = 0;
    g.split_stride = 0;
    g.tail_first = g.tail_splits = 0;
    g.tail_part = nullptr;
    g.c_vec = 0;
    g.bounded_tail = 0;
    return g;
}

// The unstaged kernel serves short k on up to one 32 x 32 block of C per CU, or k up to 512 when C is only a handful
// of blocks.  Beyond that the split product is faster even with its second launch (64 x 128 x 784, the first layer
// of the batch-64 MLP: 7.6 us of kernel time split and reduced against 11 us unstaged; 128 x 128 x 1024: 8.6 against
// 16).  Cutting k over several workgroups inside the unstaged kernel, with the last one to arrive adding the partial
// blocks, was measured too: the device-scope fences it needs write back and invalidate the L2, 10 us for 32
// workgroups and 65 us for 500.
static bool gemm_is_tiny(size_t m, size_t n, size_t k, size_t batches, size_t lda, size_t ldb, size_t n_cu) {
    const size_t blocks = ceil_div_sz(m, 32) * ceil_div_sz(n, 32) * batches;
    const bool small_ld = lda < ((size_t)1 << 21) && ldb < ((size_t)1 << 21);
    return small_ld && ((k <= 256 && blocks <= n_cu) || (k <= 512 && blocks <= 16));
}

// Ranges of k for the skinny weight-gradient products (see gemm_dispatch_body): groups of 8 values of k, a round of 32
// groups per workgroup at least; at most 32 ranges, or two workgroups per compute unit where k is long enough for
// ranges of 2048 values and more (16 x 16 over a million rows: 413 us in 32 ranges).  `per`: groups per range.
static size_t gemm_skinny_splits(size_t m, size_t n, size_t k, size_t n_cu, size_t* per_out) {
    const size_t groups = ceil_div_sz(k, 8);
    size_t splits = ceil_div_sz(groups, 32);
    size_t cap = 2 * n_cu / (ceil_div_sz(m, 32) * ceil_div_sz(n, 32));
    if (cap > groups / 256) cap = groups / 256;
    if (cap < 32) cap = 32;
    if (splits > cap) splits = cap;
    size_t per = ceil_div_sz(groups, splits);
    per = (per + 3) & ~(size_t)3;  // whole turns of the four waves
    *per_out = per;
    return ceil_div_sz(groups, per);
}

// One unbatched product of k-contiguous operands with a long k on at most a CU's worth of 16 x 16 blocks: gemm_deep_kernel.
// It goes before the unstaged kernel where both apply (k of 384 to 512 on up to 16 blocks of 32 x 32: 64 x 64 x 512
// 8.1 -> 5.6 us, 128 x 64 x 512 8.2 -> 4.8 us).
// (Below k = 384 the unstaged kernel or one round of 64 x 64 tiles does as well.  A load instruction of this kernel
// touches 64 bytes in each of 16 rows, which the memory system serves slowly when the rows are far apart: at k = 4096
// a workgroup's loads take 19 us and the staged kernels with k cut over workgroups win again; measured break-even
// between k = 2048 and 3072.)
static bool gemm_is_deep(size_t m, size_t n, size_t k, size_t batches, bool a_kmajor, bool b_kmajor, size_t n_cu) {
    return batches == 1 && a_kmajor && b_kmajor && k >= 384 && k <= 2048 && ceil_div_sz(m, 16) * ceil_div_sz(n, 16) <= n_cu;
}

static int gemm_validate(const char* name, const float* A, const float* B, const float* C, size_t m, size_t n, size_t k,
                         int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc) {
    ZG_REQUIRE(C && (k == 0 || (A && B)), "%s: null pointer", name);  // with k == 0 the operands are not read: C = beta C
    // cblas argument rules for row-major storage
    ZG_REQUIRE(lda >= (trans_a ? m : k) && lda >= 1, "%s: lda %zu too small", name, lda);
    ZG_REQUIRE(ldb >= (trans_b ? k : n) && ldb >= 1, "%s: ldb %zu too small", name, ldb);
    ZG_REQUIRE(ldc >= n, "%s: ldc %zu < n %zu", name, ldc, n);
    return ZG_HIP_OK;
}

static int gemm_dispatch_body(zg_hip_ctx* ctx, const char* name, const float* A, const float* B, float* C, size_t m,
                              size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha,
                              float beta, size_t batches, size_t nba, size_t nbb, size_t a_chunk, size_t b_chunk,
                              size_t c_chunk, int depth, const GemmExtras* extras);

// One launch for the backward of a small Linear layer (linear_bwd_small_kernel): gw = gw_beta * gw + gy^T x (x with
// leading dimension ldx), gx = gy w masked by act_in (w with leading dimension ldw; gx null: none), gb += column sums of
// gy (gb null: none).  The caller has checked that each job is one the kernel's blocks take.
static int launch_linear_bwd_small(zg_hip_ctx* ctx, const float* gy, const float* x, size_t ldx, const float* w, size_t ldw,
                                   const float* act_in, float* gw, float gw_beta, float* gb, float gb_beta, float* gx,
                                   size_t batch, size_t fan_in, size_t fan_out) {
    LinearBwdArgs a;
    a.gw = gemm_args(gy, x, gw, fan_out, fan_in, batch, 1, 0, fan_out, ldx, fan_in, 1.f, gw_beta, 1, 1, 0, 0, 0, nullptr);
    a.n_w = a.gw.tiles_m * a.gw.tiles_n;
    a.gx = a.gw;
    a.n_x = 0;
    if (gx) {
        const GemmExtras ex = {nullptr, act_in, 0};
        a.gx = gemm_args(gy, w, gx, batch, fan_in, fan_out, 0, 0, fan_out, ldw, fan_in, 1.f, 0.f, 1, 1, 0, 0, 0,
                         act_in ? &ex : nullptr);
        a.n_x = a.gx.tiles_m * a.gx.tiles_n;
    }
    const ColReduceShape cs = col_reduce_shape(gy, fan_out);
    a.gy = gy;
    a.gb = gb;
    a.gb_beta = gb_beta;
    a.R = batch;
    a.inner = fan_out;
    a.log2_cx = cs.log2_cx;
    const unsigned grid = a.n_w + a.n_x + (gb ? (unsigned)cs.gx : 0u);
    if (cs.V == 4) hipLaunchKernelGGL(linear_bwd_small_kernel<4>, dim3(grid), dim3(kGemmThreads), 0, ctx->stream, a);
    else hipLaunchKernelGGL(linear_bwd_small_kernel<1>, dim3(grid), dim3(kGemmThreads), 0, ctx->stream, a);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// Every product goes through here.  With zg_hip_gemm_timing on, the launches of one product (its kernel, and the
// reduction or the strips when it is cut) are bracketed by a pair of events on the context's stream.
static int gemm_dispatch(zg_hip_ctx* ctx, const char* name, const float* A, const float* B, float* C, size_t m, size_t n,
                         size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta,
                         size_t batches, size_t nba, size_t nbb, size_t a_chunk, size_t b_chunk, size_t c_chunk,
                         int depth = 0, const GemmExtras* extras = nullptr) {
    GemmPlanCache* pc = ctx->gemm_plans;
    const bool bracket = pc && pc->timing && !pc->in_bracket && !ctx->capturing && m > 0 && n > 0 && batches > 0;
    if (!bracket)
        return gemm_dispatch_body(ctx, name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, batches, nba, nbb,
                                  a_chunk, b_chunk, c_chunk, depth, extras);
    if (pc->used == pc->pairs.size()) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        ZG_HIP_TRY(hipEventCreate(&e0));
        ZG_HIP_TRY(hipEventCreate(&e1));
        pc->pairs.emplace_back(e0, e1);
    }
    auto& pr = pc->pairs[pc->used];
    ZG_HIP_TRY(hipEventRecord(pr.first, ctx->stream));
    pc->in_bracket = true;
    const int rc = gemm_dispatch_body(ctx, name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, batches, nba,
                                      nbb, a_chunk, b_chunk, c_chunk, depth, extras);
    pc->in_bracket = false;
    if (rc) return rc;
    ZG_HIP_TRY(hipEventRecord(pr.second, ctx->stream));
    pc->used++;
    return ZG_HIP_OK;
}

static int gemm_dispatch_body(zg_hip_ctx* ctx, const char* name, const float* A, const float* B, float* C, size_t m,
                              size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha,
                              float beta, size_t batches, size_t nba, size_t nbb, size_t a_chunk, size_t b_chunk,
                              size_t c_chunk, int depth, const GemmExtras* extras) {
    if (m == 0 || n == 0 || batches == 0) return ZG_HIP_OK;
    if (int rc = gemm_validate(name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc)) return rc;
    ZG_REQUIRE(nba >= 1 && nbb >= 1, "%s: zero operand batches", name);
    if (batches > 65535) {
        // the batch index is the grid's z dimension (at most 65535): longer batches go in runs.  The operand batch
        // index of run-relative batch z is (z0 + z) % nb; a run that starts at a multiple of nb, or an operand with a
        // single batch, keeps the kernel's own z % nb valid, which a run length that nba and nbb both divide ensures.
        ZG_REQUIRE((nba == 1 || nba == batches) && (nbb == 1 || nbb == batches),
                   "%s: more than 65535 batches with operands that repeat every %zu / %zu batches", name, nba, nbb);
        for (size_t z0 = 0; z0 < batches; z0 += 65535) {
            const size_t run = batches - z0 < 65535 ? batches - z0 : 65535;
            GemmExtras ex;
            if (extras) {
                ex = *extras;
                if (ex.gate) ex.gate += z0 * c_chunk;
            }
            if (int rc = gemm_dispatch(ctx, name, nba == 1 ? A : A + z0 * a_chunk, nbb == 1 ? B : B + z0 * b_chunk,
                                       C + z0 * c_chunk, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, run,
                                       nba == 1 ? 1 : run, nbb == 1 ? 1 : run, a_chunk, b_chunk, c_chunk, depth,
                                       extras ? &ex : nullptr))
                return rc;
        }
        return ZG_HIP_OK;
    }
    if (k == 0 || alpha == 0.f) {
        if (beta == 1.f) return ZG_HIP_OK;
        size_t blocks = ceil_div_sz(m * n, 256);
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(scale_c_kernel, dim3((unsigned)blocks, 1, (unsigned)batches), dim3(256), 0, ctx->stream, C, m,
                           n, ldc, beta, c_chunk);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    GemmArgs g = gemm_args(A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, nba, nbb, a_chunk, b_chunk,
                           c_chunk, extras);
    const bool a_kmajor = !trans_a, b_kmajor = trans_b != 0;

    // Kernel mode per tile shape: fast (whole tiles in m and n, C fit for vector stores), edge (everything else) or
    // checked (leading dimensions too large for 32-bit byte offsets), see gemm_kernel.
    const bool c_vec = aligned16(C) && ldc % 4 == 0 && c_chunk % 4 == 0 && n % 4 == 0;
    const bool small_ld = lda < ((size_t)1 << 21) && ldb < ((size_t)1 << 21);
    // A and B go through 16-byte buffer loads, which the memory system serves at any 4-byte alignment (measured: an
    // odd leading dimension costs a few percent); the fast kernels store C in vectors, the edge kernels also in scalars
    g.c_vec = c_vec;
    g.bounded_tail = (!a_kmajor && m % 4 != 0) || (!b_kmajor && n % 4 != 0);
    auto tiles = [&](size_t bm, size_t bn) { return ceil_div_sz(m, bm) * ceil_div_sz(n, bn) * batches; };
    auto mode = [&](size_t bm, size_t bn) {
        if (!small_ld) return 2;
        return (m % bm == 0 && n % bn == 0 && c_vec) ? 0 : 1;  // any k: the last tiles are masked on their way into LDS
    };
    const size_t n_cu = (size_t)ctx->n_cu;
    const size_t kt_total = ceil_div_sz(k, kBK);
    g.split_tiles = kt_total;
    g.split_stride = 0;

    // leading dimensions of 2^21 values and more (a few rows of millions of columns): 64 x 64 tiles with 64-bit row
    // offsets, whole, or with k in ranges where the plan for 64 x 64 tiles cuts it (32 x 32 over 2097152 values of k on
    // one workgroup: 78 ms)
    const GemmPlan far_plan = small_ld ? GemmPlan() : gemm_plan_single(m, n, k, batches, n_cu);
    if (!small_ld && !(far_plan.kind == GemmPlan::kSplit && far_plan.tile == 2))
        return launch_gemm<64, 64>(ctx, g, a_kmajor, b_kmajor, 2, batches);
    if (small_ld && gemm_is_micro(m, n, k, batches, g)) return launch_gemm_micro(ctx, g, a_kmajor, b_kmajor, batches);
    const bool deep = small_ld && gemm_is_deep(m, n, k, batches, a_kmajor, b_kmajor, n_cu);
    if (!deep && gemm_is_tiny(m, n, k, batches, lda, ldb, n_cu)) return launch_gemm_tiny(ctx, g, a_kmajor, b_kmajor, batches);
    if (deep) {
        g.tiles_m = (unsigned)ceil_div_sz(m, 16);
        g.tiles_n = (unsigned)ceil_div_sz(n, 16);
        hipLaunchKernelGGL(gemm_deep_kernel, dim3(g.tiles_m * g.tiles_n), dim3(256), 0, ctx->stream, g);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    // Skinny weight-gradient products with a long k (one side of C at most 32 wide, both operands stored k-strided:
    // the 16-wide layer of the GCN, 16 x 1433 over 2708 nodes): 64-wide tiles would compute mostly padding, so the
    // unstaged kernel takes ranges of k (one round of 256 per workgroup, at most 32 ranges) and the split-k reduction
    // adds the partial blocks: 11.9 us against 15.3 us.  With a k-contiguous operand the unstaged kernel's loads are
    // 16 bytes per row and lane, which costs more than the padding (2708 x 16 x 1433: 17.8 us against 14.1 us).
    if (small_ld && !a_kmajor && !b_kmajor && (m <= 32 || n <= 32) && k > 512 && tiles(32, 32) <= n_cu) {
        size_t per = 0;
        const size_t splits = gemm_skinny_splits(m, n, k, n_cu, &per);
        float* part = (float*)workspace(ctx, batches * splits * m * n * sizeof(float));
        if (!part) return ZG_HIP_EOOM;
        GemmArgs gs = g;
        gs.C = part;
        gs.ldc = n;
        gs.c_chunk = splits * m * n;
        gs.split_tiles = per;
        gs.split_stride = m * n;
        gs.alpha = 1.f;
        gs.beta = 0.f;
        gs.bias = nullptr;  // the extras belong to the sum of the partial products: the reduce kernel applies them
        gs.gate = nullptr;
        gs.relu = 0;
        if (int rc = launch_gemm_tiny(ctx, gs, a_kmajor, b_kmajor, batches, splits)) return rc;
        if (splits > 16) {
            hipLaunchKernelGGL(splitk_reduce_many_kernel, dim3((unsigned)ceil_div_sz(m * n, 64), 1, (unsigned)batches), dim3(256), 0,
                               ctx->stream, part, C, m, n, ldc, (int)splits, alpha, beta, c_chunk, g.bias, g.gate, g.relu);
            ZG_LAUNCH_CHECK();
            return ZG_HIP_OK;
        }
        size_t blocks = ceil_div_sz(m * n, 256);
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks, 1, (unsigned)batches), dim3(256), 0, ctx->stream,
                           part, C, m, n, ldc, (int)splits, alpha, beta, c_chunk, g.bias, g.gate, g.relu);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }

    // ---- plan: which tile, whether k is cut, whether C is cut into a block of whole rounds plus strips ----
    const GemmPlan plan = small_ld ? gemm_plan(ctx, m, n, k, batches, a_kmajor, b_kmajor, depth) : far_plan;
    if (plan.kind == GemmPlan::kParts) {
        // C = [ main | right ] over [ bottom ]: main is rm x rn whole large tiles (a whole number of rounds, or nearly),
        // the strips are products of their own and go through this function again (they may cut k, not C).
        const size_t m1 = plan.rm * 256, n1 = plan.rn * 128;
        struct Part {
            size_t r0, c0, mm, nn;
        } parts[3] = {{0, 0, m1, n1}, {0, n1, m1, n - n1}, {m1, 0, m - m1, n}};
        for (const Part& pt : parts) {
            if (pt.mm == 0 || pt.nn == 0) continue;
            const float* As = trans_a ? A + pt.r0 : A + pt.r0 * lda;
            const float* Bs = trans_b ? B + pt.c0 * ldb : B + pt.c0;
            float* Cs = C + pt.r0 * ldc + pt.c0;
            GemmExtras ex;
            if (extras) {
                ex.bias = extras->bias ? extras->bias + pt.c0 : nullptr;
                ex.gate = extras->gate ? extras->gate + (pt.r0 * ldc + pt.c0) : nullptr;
                ex.relu = extras->relu;
            }
            if (int rc = gemm_dispatch(ctx, name, As, Bs, Cs, pt.mm, pt.nn, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta,
                                       1, 1, 1, 0, 0, 0, depth + 1, extras ? &ex : nullptr))
                return rc;
        }
        return ZG_HIP_OK;
    }
    const int tile = plan.tile;  // 0: 256 x 128, 1: 128 x 128, 2: 64 x 64
    const size_t bm = kGemmTiles[tile].bm, bn = kGemmTiles[tile].bn;
    if (plan.kind == GemmPlan::kSplit) {
        // k is cut over several workgroups per tile (an even number of k-tiles each); each writes its partial tile to the
        // workspace and a second kernel adds the partials in split order: the order is fixed, so the result does not
        // depend on scheduling.
        const size_t splits = plan.splits, per = plan.per;
        float* part = (float*)workspace(ctx, batches * splits * m * n * sizeof(float));
        if (!part) return ZG_HIP_EOOM;
        GemmArgs gs = g;
        gs.C = part;
        gs.ldc = n;
        gs.c_chunk = splits * m * n;
        gs.split_tiles = per;
        gs.split_stride = m * n;
        gs.alpha = 1.f;
        gs.beta = 0.f;
        gs.bias = nullptr;  // the extras belong to the sum of the partial products: the reduce kernel applies them
        gs.gate = nullptr;
        gs.relu = 0;
        gs.c_vec = n % 4 == 0 && (m * n) % 4 == 0;  // the partial-product buffer is 256-byte aligned and dense
        const int split_mode = !small_ld ? 2 : ((m % bm == 0 && n % bn == 0 && gs.c_vec) ? 0 : 1);
        int rc = tile == 0   ? launch_gemm<256, 128>(ctx, gs, a_kmajor, b_kmajor, split_mode, batches)
                 : tile == 1 ? launch_gemm<128, 128>(ctx, gs, a_kmajor, b_kmajor, split_mode, batches)
                             : launch_gemm<64, 64>(ctx, gs, a_kmajor, b_kmajor, split_mode, batches);
        if (rc) return rc;
        if (splits > 16) {
            hipLaunchKernelGGL(splitk_reduce_many_kernel, dim3((unsigned)ceil_div_sz(m * n, 64), 1, (unsigned)batches), dim3(256), 0,
                               ctx->stream, part, C, m, n, ldc, (int)splits, alpha, beta, c_chunk, g.bias, g.gate, g.relu);
            ZG_LAUNCH_CHECK();
            return ZG_HIP_OK;
        }
        const bool vec4 = gs.c_vec && c_vec && !g.gate;
        size_t blocks = ceil_div_sz(vec4 ? m * n / 4 : m * n, 256);
        if (blocks > 4096) blocks = 4096;
        if (vec4)
            hipLaunchKernelGGL(splitk_reduce_vec4_kernel, dim3((unsigned)blocks, 1, (unsigned)batches), dim3(256), 0,
                               ctx->stream, part, C, m, n, ldc, (int)splits, alpha, beta, c_chunk, g.bias, g.relu);
        else
            hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks, 1, (unsigned)batches), dim3(256), 0,
                               ctx->stream, part, C, m, n, ldc, (int)splits, alpha, beta, c_chunk, g.bias, g.gate, g.relu);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (plan.kind == GemmPlan::kTail) {
        // whole tiles for a whole number of rounds, the remaining tiles in pieces along k, one more kernel for their sums
        const size_t tail_tiles = tiles(bm, bn) - plan.whole;
        float* part = (float*)workspace(ctx, tail_tiles * plan.splits * bm * bn * sizeof(float));
        if (!part) return ZG_HIP_EOOM;
        g.tail_first = (unsigned)plan.whole;
        g.tail_splits = (unsigned)plan.splits;
        g.tail_part = part;
        g.split_tiles = plan.per;
        const int md = mode(bm, bn);
        int rc = tile == 1 ? launch_gemm<128, 128>(ctx, g, a_kmajor, b_kmajor, md, 1)
                           : launch_gemm<64, 64>(ctx, g, a_kmajor, b_kmajor, md, 1);
        if (rc) return rc;
        const unsigned blocks = (unsigned)(tail_tiles * (bm * bn / 1024));
        if (tile == 1) hipLaunchKernelGGL((gemm_tail_reduce_kernel<128, 128>), dim3(blocks), dim3(256), 0, ctx->stream, g);
        else hipLaunchKernelGGL((gemm_tail_reduce_kernel<64, 64>), dim3(blocks), dim3(256), 0, ctx->stream, g);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    if (tile == 0) return launch_gemm<256, 128>(ctx, g, a_kmajor, b_kmajor, mode(256, 128), batches);
    if (tile == 1) return launch_gemm<128, 128>(ctx, g, a_kmajor, b_kmajor, mode(128, 128), batches);
    return launch_gemm<64, 64>(ctx, g, a_kmajor, b_kmajor, mode(64, 64), batches);
}

// The workspace a single product of this shape asks for when it is dispatched (the partial tiles of a k that is cut),
// following gemm_dispatch_body's choices.  A product that waits reserves it when it is queued, so that the call
// which later launches it, whichever that is, allocates nothing.
static size_t gemm_workspace_need(zg_hip_ctx* ctx, size_t m, size_t n, size_t k, int trans_a, int trans_b, size_t lda,
                                  size_t ldb, int depth) {
    if (m == 0 || n == 0 || k == 0) return 0;
    const bool a_kmajor = !trans_a, b_kmajor = trans_b != 0;
    const size_t n_cu = (size_t)ctx->n_cu;
    const bool small_ld = lda < ((size_t)1 << 21) && ldb < ((size_t)1 << 21);
    if (!small_ld) {
        const GemmPlan far_plan = gemm_plan_single(m, n, k, 1, n_cu);
        return (far_plan.kind == GemmPlan::kSplit && far_plan.tile == 2) ? far_plan.splits * m * n * sizeof(float) : 0;
    }
    if (gemm_is_tiny(m, n, k, 1, lda, ldb, n_cu)) return 0;
    if (gemm_is_deep(m, n, k, 1, a_kmajor, b_kmajor, n_cu)) return 0;
    if (!a_kmajor && !b_kmajor && (m <= 32 || n <= 32) && k > 512 && ceil_div_sz(m, 32) * ceil_div_sz(n, 32) <= n_cu) {
        size_t per = 0;
        return gemm_skinny_splits(m, n, k, n_cu, &per) * m * n * sizeof(float);
    }
    const GemmPlan plan = gemm_plan(ctx, m, n, k, 1, a_kmajor, b_kmajor, depth);
    if (plan.kind == GemmPlan::kTail) {
        const size_t bm = kGemmTiles[plan.tile].bm, bn = kGemmTiles[plan.tile].bn;
        return (ceil_div_sz(m, bm) * ceil_div_sz(n, bn) - plan.whole) * plan.splits * bm * bn * sizeof(float);
    }
    if (plan.kind == GemmPlan::kParts) {
        const size_t m1 = plan.rm * 256, n1 = plan.rn * 128;
        const size_t shapes[3][2] = {{m1, n1}, {m1, n - n1}, {m - m1, n}};
        size_t need = 0;
        for (const auto& sh : shapes) {
            if (sh[0] == 0 || sh[1] == 0) continue;
            const size_t part = gemm_workspace_need(ctx, sh[0], sh[1], k, trans_a, trans_b, lda, ldb, depth + 1);
            need = part > need ? part : need;
        }
        return need;
    }
    if (plan.kind == GemmPlan::kSplit) return plan.splits * m * n * sizeof(float);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// matvec / outer / transpose
// ------------------------------------------------------------------------------------------------

// y = alpha * A x + beta * y, A is [m, n] row-major (cblas_sgemv, src/device/host_device.zig:232-240).  TPR threads per row
// (4, 16 or 64 lanes of a wave, or a whole workgroup), 256 / TPR rows per workgroup; a thread has four 16-byte loads of
// its row in flight (and the matching pieces of x, which stay in the caches), the partial sums of the four are added
// in a fixed order and the threads of a row combine by shuffles (through LDS for a workgroup).  Long rows on few
// workgroups are cut into segments of `seg` columns (blockIdx.y): the segment sums go to part [segments][m] and
// vec_final_kernel adds them in segment order.  VEC false: any alignment, any n, value by value.
template <int TPR, bool VEC>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const float* A, const float* x, float* y, float* part, size_t m,
                                                         size_t n, size_t seg, float alpha, float beta) {
    __shared__ float smem[256 / kWave];
    const int lane = threadIdx.x % TPR;
    const size_t row = (size_t)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
    const bool live = row < m;
    const size_t c0 = (size_t)blockIdx.y * seg, c1 = c0 + seg < n ? c0 + seg : n;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (live) {
        const float* a = A + row * n;
        if (VEC) {
            const float4* a4 = reinterpret_cast<const float4*>(a);
            const float4* x4 = reinterpret_cast<const float4*>(x);
            const size_t j1 = c1 >> 2;
            auto dot4 = [](float4 u, float4 v) { return ((u.x * v.x + u.y * v.y) + u.z * v.z) + u.w * v.w; };
            size_t j0 = c0 >> 2;
            for (; j0 + 4 * TPR <= j1; j0 += 4 * TPR) {
                const size_t j = j0 + lane;
                const float4 u0 = a4[j], u1 = a4[j + TPR], u2 = a4[j + 2 * TPR], u3 = a4[j + 3 * TPR];
                s0 += dot4(u0, x4[j]);
                s1 += dot4(u1, x4[j + TPR]);
                s2 += dot4(u2, x4[j + 2 * TPR]);
                s3 += dot4(u3, x4[j + 3 * TPR]);
            }
            if (j0 < j1) {  // the last, partial trip: its loads in flight together, the ones past the end left out
                const size_t j = j0 + lane;
                float4 u[4];
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (j + (size_t)k * TPR < j1) u[k] = a4[j + (size_t)k * TPR];
                if (j < j1) s0 += dot4(u[0], x4[j]);
                if (j + TPR < j1) s1 += dot4(u[1], x4[j + TPR]);
                if (j + 2 * TPR < j1) s2 += dot4(u[2], x4[j + 2 * TPR]);
                if (j + 3 * TPR < j1) s3 += dot4(u[3], x4[j + 3 * TPR]);
            }
        } else {
            size_t j = c0 + lane;
            for (; j + 3 * TPR < c1; j += 4 * TPR) {
                const float u0 = a[j], u1 = a[j + TPR], u2 = a[j + 2 * TPR], u3 = a[j + 3 * TPR];
                s0 += u0 * x[j];
                s1 += u1 * x[j + TPR];
                s2 += u2 * x[j + 2 * TPR];
                s3 += u3 * x[j + 3 * TPR];
            }
            for (; j < c1; j += TPR) s0 += a[j] * x[j];
        }
    }
    float s = (s0 + s1) + (s2 + s3);
    if (TPR <= kWave) {
        s = group_reduce<SumAcc, (TPR <= kWave ? TPR : kWave)>(s);
    } else {
        s = block_reduce<SumAcc>(s, smem);
    }
    if (live && lane == 0) {
        if (part) part[(size_t)blockIdx.y * m + row] = s;
        else y[row] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[row];
    }
}

// y[o] = alpha * (part[0][o] + part[1][o] + ...) + beta * y[o] for partial results [chunks][n_out]: a workgroup owns 64
// adjacent outputs, wave w adds chunks w, w + 4, ... with sixteen loads in flight, and the four wave sums are added in
// wave order.
__global__ __launch_bounds__(256) void vec_final_kernel(const float* part, float* y, size_t n_out, size_t chunks, float alpha,
                                                         float beta) {
    __shared__ float smem[4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const size_t o = (size_t)blockIdx.x * 64 + lane;
    float s = 0.f;
    if (o < n_out) {
        for (size_t base = 0; base < chunks; base += 64) {
            float t[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const size_t k = base + (size_t)w + 4 * (size_t)u;
                t[u] = k < chunks ? part[k * n_out + o] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 16; u++) s += t[u];
        }
    }
    smem[w][lane] = s;
    __syncthreads();
    if (w == 0 && o < n_out) {
        s = ((smem[0][lane] + smem[1][lane]) + smem[2][lane]) + smem[3][lane];
        y[o] = (beta == 0.f) ? alpha * s : alpha * s + beta * y[o];
    }
}

// y = alpha * A^T x + beta * y, A is [m, n] row-major, y has n entries.  A workgroup is cx column-threads by ry = 256 / cx
// row-threads and owns cx * V adjacent columns and one chunk of rows: a thread walks rows ty, ty + ry, ... of the chunk
// with eight loads of V columns in flight (V = 4: 16 bytes), multiplies by x[row] and adds in row order; the row-threads
// of a column combine in ty order through LDS.  One chunk: the result is written here; several: the chunk sums go to
// part [chunks][n] and vec_final_kernel adds them in chunk order.
template <int V>
__global__ __launch_bounds__(256) void gemv_t_kernel(const float* A, const float* x, float* y, float* part, size_t m,
                                                      size_t n, int log2_cx, size_t rows_per_chunk, float alpha, float beta) {
    __shared__ float smem[256 * V];
    const int cx = 1 << log2_cx, ry = 256 >> log2_cx;
    const int tx = threadIdx.x & (cx - 1), ty = threadIdx.x >> log2_cx;
    const size_t col0 = ((size_t)blockIdx.x * cx + tx) * V;
    const size_t r0 = (size_t)blockIdx.y * rows_per_chunk;
    const size_t r1 = r0 + rows_per_chunk < m ? r0 + rows_per_chunk : m;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = 0.f;
    const bool active = col0 < n;
    if (active) {
        const float* ab = A + col0;
        size_t r = r0 + ty;
        if constexpr (V == 4) {
            for (; r + 7 * (size_t)ry < r1; r += 8 * (size_t)ry) {
                float4 u[8];
                float xs[8];
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    u[k] = *reinterpret_cast<const float4*>(ab + (r + (size_t)k * ry) * n);
                    xs[k] = x[r + (size_t)k * ry];
                }
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    acc[0] += u[k].x * xs[k];
                    acc[1 % V] += u[k].y * xs[k];
                    acc[2 % V] += u[k].z * xs[k];
                    acc[3 % V] += u[k].w * xs[k];
                }
            }
            for (; r < r1; r += ry) {
                const float4 u = *reinterpret_cast<const float4*>(ab + r * n);
                const float xv = x[r];
                acc[0] += u.x * xv;
                acc[1 % V] += u.y * xv;
                acc[2 % V] += u.z * xv;
                acc[3 % V] += u.w * xv;
            }
        } else {
            // single columns (a row length that is no multiple of four): sixteen rows in flight, then eight
            for (; r + 15 * (size_t)ry < r1; r += 16 * (size_t)ry) {
                float u[16], xs[16];
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    u[k] = ab[(r + (size_t)k * ry) * n];
                    xs[k] = x[r + (size_t)k * ry];
                }
#pragma unroll
                for (int k = 0; k < 16; k++) acc[0] += u[k] * xs[k];
            }
            for (; r + 7 * (size_t)ry < r1; r += 8 * (size_t)ry) {
                float u[8], xs[8];
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    u[k] = ab[(r + (size_t)k * ry) * n];
                    xs[k] = x[r + (size_t)k * ry];
                }
#pragma unroll
                for (int k = 0; k < 8; k++) acc[0] += u[k] * xs[k];
            }
            for (; r < r1; r += ry) acc[0] += ab[r * n] * x[r];
        }
    }
#pragma unroll
    for (int v = 0; v < V; v++) smem[threadIdx.x * V + v] = acc[v];
    __syncthreads();
    if (ty == 0 && active) {
        for (int t = 1; t < ry; t++) {
#pragma unroll
            for (int v = 0; v < V; v++) acc[v] += smem[((t << log2_cx) + tx) * V + v];
        }
#pragma unroll
        for (int v = 0; v < V; v++) {
            const size_t c = col0 + v;
            if (c < n) {
                if (part) part[(size_t)blockIdx.y * n + c] = acc[v];
                else y[c] = (beta == 0.f) ? alpha * acc[v] : alpha * acc[v] + beta * y[c];
            }
        }
    }
}

// A += alpha * x y^T   (cblas_sger, src/device/host_device.zig:252-258).  VEC: 16-byte pieces of a row of A (rows that start
// on 16-byte boundaries), four per thread in flight.
template <bool VEC>
__global__ __launch_bounds__(256) void ger_kernel(const float* x, size_t xl, const float* y, size_t yl, float* A,
                                                   float alpha) {
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, nt = (size_t)gridDim.x * 256;
    if (VEC) {
        const size_t yl4 = yl >> 2, n4 = xl * yl4;
        float4* a4 = reinterpret_cast<float4*>(A);
        const float4* y4 = reinterpret_cast<const float4*>(y);
        auto piece = [&](size_t i, float4 a) {
            const size_t r = i / yl4, c = i % yl4;
            const float ax = __fmul_rn(alpha, x[r]);
            const float4 yv = y4[c];
            a.x = __fadd_rn(a.x, __fmul_rn(ax, yv.x));
            a.y = __fadd_rn(a.y, __fmul_rn(ax, yv.y));
            a.z = __fadd_rn(a.z, __fmul_rn(ax, yv.z));
            a.w = __fadd_rn(a.w, __fmul_rn(ax, yv.w));
            return a;
        };
        size_t i = tid;
        for (; i + 3 * nt < n4; i += 4 * nt) {
            const float4 u0 = nt_load(a4 + i), u1 = nt_load(a4 + i + nt), u2 = nt_load(a4 + i + 2 * nt), u3 = nt_load(a4 + i + 3 * nt);
            nt_store(piece(i, u0), a4 + i);
            nt_store(piece(i + nt, u1), a4 + i + nt);
            nt_store(piece(i + 2 * nt, u2), a4 + i + 2 * nt);
            nt_store(piece(i + 3 * nt, u3), a4 + i + 3 * nt);
        }
        for (; i < n4; i += nt) a4[i] = piece(i, a4[i]);
    } else {
        for (size_t i = tid; i < xl * yl; i += nt) {
            const size_t r = i / yl, c = i % yl;
            A[i] = __fadd_rn(A[i], __fmul_rn(__fmul_rn(alpha, x[r]), y[c]));
        }
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

// The same through a 64 x 64 tile with 16-byte accesses on both sides (m and n multiples of 4, A and B on 16-byte
// boundaries): thread (tx, ty) of 16 x 16 reads pieces tx of rows ty, ty + 16, ... of the tile of A, and writes pieces
// tx of rows ty, ty + 16, ... of the tile of B, whose four values come from four rows of the LDS tile.
// Tiles are numbered along the rows of A; `diagonal` numbers them down the diagonals instead (tile row = id mod gy, tile
// column = id / gy + tile row), so that the tiles in flight differ in both their column of A and their column of B: with
// both row lengths multiples of 4 KiB, tiles of one row of A write to addresses a multiple of 4 KiB apart, which land on
// few memory channels (4096 x 4096: 23.4 -> 20.5 us, 8192 x 8192: 123 -> 103 us).
__global__ __launch_bounds__(256) void transpose_vec_kernel(const float* A, float* B, size_t m, size_t n, float alpha,
                                                            bool diagonal, unsigned gx, unsigned gy) {
    __shared__ float tile[64][65];
    unsigned bx, by;
    if (diagonal) {
        by = blockIdx.x % gy;
        bx = (blockIdx.x / gy + by) % gx;
    } else {
        bx = blockIdx.x % gx;
        by = blockIdx.x / gx;
    }
    const size_t bi = (size_t)by * 64, bj = (size_t)bx * 64;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    float4 u[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const size_t i = bi + ty + 16 * k, j = bj + 4 * tx;
        if (i < m && j < n) u[k] = *reinterpret_cast<const float4*>(A + i * n + j);
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const size_t i = bi + ty + 16 * k, j = bj + 4 * tx;
        if (i < m && j < n) {
            float* t = &tile[ty + 16 * k][4 * tx];
            t[0] = u[k].x;
            t[1] = u[k].y;
            t[2] = u[k].z;
            t[3] = u[k].w;
        }
    }
    __syncthreads();
    float4 old[4];
    if (alpha != 0.f) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const size_t j = bj + ty + 16 * k, i = bi + 4 * tx;  // B[j, i .. i + 3]
            if (j < n && i < m) old[k] = *reinterpret_cast<const float4*>(B + j * m + i);
        }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int r = ty + 16 * k;
        const size_t j = bj + r, i = bi + 4 * tx;
        if (j < n && i < m) {
            float4 v = make_float4(tile[4 * tx][r], tile[4 * tx + 1][r], tile[4 * tx + 2][r], tile[4 * tx + 3][r]);
            if (alpha != 0.f) {
                v.x = __fadd_rn(v.x, __fmul_rn(alpha, old[k].x));
                v.y = __fadd_rn(v.y, __fmul_rn(alpha, old[k].y));
                v.z = __fadd_rn(v.z, __fmul_rn(alpha, old[k].z));
                v.w = __fadd_rn(v.w, __fmul_rn(alpha, old[k].w));
            }
            *reinterpret_cast<float4*>(B + j * m + i) = v;
        }
    }
}

}  // namespace zg

using namespace zg;

ZG_API int zg_hip_gemm_timing(zg_hip_ctx* ctx, int enable) {
    ZG_CTX(ctx);
    if (!ctx->gemm_plans) ctx->gemm_plans = new GemmPlanCache();
    if (enable) ctx->gemm_plans->used = 0;
    ctx->gemm_plans->timing = enable != 0;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_gemm_timing_read(zg_hip_ctx* ctx, double* total_ms, uint64_t* products) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "gemm_timing_read");
    ZG_REQUIRE(total_ms && products, "gemm_timing_read: null output");
    *total_ms = 0.0;
    *products = 0;
    if (!ctx->gemm_plans) return ZG_HIP_OK;
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));
    for (size_t i = 0; i < ctx->gemm_plans->used; i++) {
        float ms = 0.f;
        ZG_HIP_TRY(hipEventElapsedTime(&ms, ctx->gemm_plans->pairs[i].first, ctx->gemm_plans->pairs[i].second));
        *total_ms += (double)ms;
    }
    *products = ctx->gemm_plans->used;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_gemm_plan(zg_hip_ctx* ctx, size_t m, size_t n, size_t k, size_t batches, int64_t* out) {
    ZG_REQUIRE(out != nullptr, "gemm_plan: null output");
    ZG_REQUIRE(m > 0 && n > 0 && k > 0 && batches > 0, "gemm_plan: empty product");
    const GemmPlan p = gemm_plan_compute(ctx ? (size_t)ctx->n_cu : 256, m, n, k, batches, 0);
    out[0] = (int64_t)p.kind;
    out[1] = p.tile;
    out[2] = (int64_t)p.splits;
    out[3] = (int64_t)p.per;
    out[4] = (int64_t)(p.kind == GemmPlan::kTail ? p.whole : p.rm);
    out[5] = (int64_t)p.rn;
    out[6] = (int64_t)(p.us + 0.5);
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Products that wait for what follows them (see zg_hip_ctx::deferred)
// ------------------------------------------------------------------------------------------------
namespace zg {

struct ByteRange {
    const char* lo;
    const char* hi;
};
static ByteRange operand_range(const float* p, size_t rows, size_t cols, size_t ld) {
    const char* lo = reinterpret_cast<const char*>(p);
    return ByteRange{lo, lo + ((rows - 1) * ld + cols) * sizeof(float)};
}
static bool ranges_meet(ByteRange a, ByteRange b) {
    return a.lo < b.hi && b.lo < a.hi;
}

static ByteRange product_a_range(const zg_deferred_gemm& d) {
    return operand_range(d.A, d.trans_a ? d.k : d.m, d.trans_a ? d.m : d.k, d.lda);
}
static ByteRange product_b_range(const zg_deferred_gemm& d) {
    return operand_range(d.B, d.trans_b ? d.n : d.k, d.trans_b ? d.k : d.n, d.ldb);
}
static ByteRange product_c_range(const zg_deferred_gemm& d) {
    return operand_range(d.C, d.m, d.n, d.ldc);
}

bool gemm_group_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi) {
    const ByteRange r{lo, hi};
    auto product = [&](const zg_deferred_gemm& d) {
        return d.active && (ranges_meet(r, product_a_range(d)) || ranges_meet(r, product_b_range(d)) ||
                            ranges_meet(r, product_c_range(d)));
    };
    const zg_waiting_bias& b = ctx->bias_wait;
    return product(ctx->deferred) || product(ctx->deferred_w) ||
           (b.active && (ranges_meet(r, operand_range(b.gy, b.R, b.inner, b.inner)) ||
                         ranges_meet(r, operand_range(b.gb, 1, b.inner, b.inner))));
}

// Whatever waits of a layer's backward pass goes out: in one launch when the weight-gradient product was recorded (it
// is only recorded when every waiting member fits linear_bwd_small_kernel), else the bias gradient's column sum and
// the product with what was attached to it.
int flush_deferred_gemm(zg_hip_ctx* ctx) {
    const zg_deferred_gemm d = ctx->deferred, w = ctx->deferred_w;
    const zg_waiting_bias b = ctx->bias_wait;
    if (!d.active && !w.active && !b.active) return ZG_HIP_OK;
    ctx->deferred.active = false;
    ctx->deferred_w.active = false;
    ctx->bias_wait.active = false;
    int rc = ZG_HIP_OK;
    if (w.active) {
        rc = launch_linear_bwd_small(ctx, w.A, w.B, w.ldb, d.active ? d.B : nullptr, d.active ? d.ldb : 0,
                                     d.active ? d.gate : nullptr, w.C, w.zeroed ? 0.f : 1.f, b.active ? b.gb : nullptr,
                                     b.active && b.fresh ? 0.f : 1.f, d.active ? d.C : nullptr, w.k, w.n, w.m);
    } else {
        if (b.active) rc = launch_bias_col_sum(ctx, b.gy, b.gb, b.R, b.inner, b.fresh);
        if (!rc && d.active) {
            GemmExtras ex{d.bias, d.gate, d.relu};
            const bool any = d.bias || d.gate || d.relu;
            rc = gemm_dispatch(ctx, d.name, d.A, d.B, d.C, d.m, d.n, d.k, d.trans_a, d.trans_b, d.lda, d.ldb, d.ldc, d.alpha,
                               0.f, 1, 1, 1, 0, 0, 0, 0, any ? &ex : nullptr);
        }
    }
    if (rc) {  // a product failed: the zeros its output was owed are still owed
        if (d.active && d.zeroed) (void)zg_hip_mem_fill(ctx, d.C, d.m * d.n, 0.f);
        if (w.active && w.zeroed) (void)zg_hip_mem_fill(ctx, w.C, w.m * w.n, 0.f);
        if (b.active && b.fresh) (void)zg_hip_mem_fill(ctx, b.gb, b.inner, 0.f);
    }
    run_deferred_frees(ctx);  // blocks that hold operands and were given back while the work waited
    return rc;
}

// An operand that joins waiting work after the fact (a bias row, a mask): the waiting fills meet none of the operands the
// work already has, but one may meet this one; then the fills go out first.  False: they could not be launched.
static bool fills_clear_of(zg_hip_ctx* ctx, const float* p, size_t n) {
    const void* ptrs[1] = {p};
    const size_t bytes[1] = {n * sizeof(float)};
    if (!ctx->n_pending_fills || !fills_touch(ctx, ptrs, bytes, 1)) return true;
    return flush_fills(ctx) == ZG_HIP_OK;
}

// bias.add_(y): z = x + y over the product's output, one operand the output itself, the other a row of n values
bool deferred_take_add(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, const float* z, size_t zl) {
    zg_deferred_gemm& d = ctx->deferred;
    if (!d.active || d.kind != 1 || d.bias || d.relu || z != d.C || zl != d.m * d.n || d.n == zl) return false;
    const float* row = nullptr;
    if (y == d.C && yl == zl && xl == d.n) row = x;
    else if (x == d.C && xl == zl && yl == d.n) row = y;
    if (!row) return false;
    if (ranges_meet(operand_range(row, 1, d.n, d.n), operand_range(d.C, d.m, d.n, d.ldc))) return false;
    if (!fills_clear_of(ctx, row, d.n)) return false;
    d.bias = row;
    return true;
}

// relu_(y) in place on the product's output: the last thing a layer's forward pass does, so the product goes out
bool deferred_take_relu(zg_hip_ctx* ctx, const float* x, const float* y, size_t n, int* rc) {
    zg_deferred_gemm& d = ctx->deferred;
    if (!d.active || d.kind != 1 || d.relu || x != d.C || y != d.C || n != d.m * d.n) return false;
    d.relu = 1;
    *rc = flush_deferred_gemm(ctx);
    return true;
}

// relu_inplace_bwd(x, x_g) on the product's output x_g: x_g = 0 where x <= 0, x laid out like the output
bool deferred_take_relu_mask(zg_hip_ctx* ctx, const float* x, const float* x_g, size_t n, int* rc) {
    zg_deferred_gemm& d = ctx->deferred;
    if (!d.active || d.kind != 2 || d.gate || x_g != d.C || n != d.m * d.n || !x) return false;
    const ByteRange xr = operand_range(x, d.m, d.n, d.n);
    if (ranges_meet(xr, operand_range(d.C, d.m, d.n, d.ldc))) return false;
    // a mask that lies in what the weight-gradient product or the bias gradient of the same launch write must be
    // read after they ran: then the mask is not taken over and the call sends everything out first
    if (ctx->deferred_w.active && ranges_meet(xr, product_c_range(ctx->deferred_w))) return false;
    if (ctx->bias_wait.active &&
        ranges_meet(xr, operand_range(ctx->bias_wait.gb, 1, ctx->bias_wait.inner, ctx->bias_wait.inner)))
        return false;
    if (!fills_clear_of(ctx, x, n)) return false;
    d.gate = x;
    *rc = flush_deferred_gemm(ctx);
    return true;
}

// matmul and bmm_acc.  In order: a waiting zero fill of exactly C turns C += ... into C = ...; the other fills go out;
// a product that is already waiting either lets this one pass (it waits for its mask and this one touches none of
// its operands: the weight-gradient product after the input-gradient product) or goes out first; then this product
// waits itself if it is a layer's forward product or an input-gradient product, or is launched.
static int gemm_entry(zg_hip_ctx* ctx, const char* name, const float* A, const float* B, float* C, size_t m, size_t n,
                      size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta,
                      size_t batches, size_t nba, size_t nbb, size_t a_chunk, size_t b_chunk, size_t c_chunk) {
    const bool plain = batches == 1 && m > 0 && n > 0 && k > 0 && alpha != 0.f && A && B && C && ldc == n;
    const bool zeroed = beta == 1.f && C && ldc == n && k > 0 && alpha != 0.f && m > 0 && n > 0 && batches > 0 &&
                        absorb_zero_fill(ctx, C, batches * m * n);
    const float beta_eff = zeroed ? 0.f : beta;
    // the other waiting fills go out if one meets an operand; the rest stay (the zero_grad() fills of the layers whose
    // backward pass comes later, each taken over by the op that accumulates into it)
    if (ctx->n_pending_fills) {
        bool touched = !plain;
        if (plain) {
            const ByteRange rs[3] = {operand_range(A, trans_a ? k : m, trans_a ? m : k, lda),
                                     operand_range(B, trans_b ? n : k, trans_b ? k : n, ldb), operand_range(C, m, n, ldc)};
            const void* ptrs[3] = {rs[0].lo, rs[1].lo, rs[2].lo};
            const size_t bytes[3] = {(size_t)(rs[0].hi - rs[0].lo), (size_t)(rs[1].hi - rs[1].lo),
                                     (size_t)(rs[2].hi - rs[2].lo)};
            touched = fills_touch(ctx, ptrs, bytes, 3);
        }
        if (touched)
            if (int rc = flush_fills(ctx)) return rc;
    }
    if (ctx->steps.count)
        if (int rc = flush_steps(ctx)) return rc;
    auto launch_now = [&]() {
        const int rc = gemm_dispatch(ctx, name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta_eff, batches, nba,
                                     nbb, a_chunk, b_chunk, c_chunk);
        if (rc && zeroed) (void)zg_hip_mem_fill(ctx, C, batches * m * n, 0.f);  // refused: the zeros are still owed
        return rc;
    };
    const size_t n_cu = (size_t)ctx->n_cu;
    const ByteRange tC = (plain && C) ? operand_range(C, m, n, ldc) : ByteRange{nullptr, nullptr};
    // a weight-gradient product the one-launch layer backward can take: gw (+)= gy^T x, gy dense
    const bool w_shape = plain && trans_a && !trans_b && alpha == 1.f && (beta_eff == 0.f || beta_eff == 1.f) && lda == m &&
                         gemm_is_tiny(m, n, k, 1, lda, ldb, n_cu) &&
                         gemm_validate(name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc) == ZG_HIP_OK;
    auto record_w = [&]() {
        zg_deferred_gemm& w = ctx->deferred_w;
        w = zg_deferred_gemm{};
        w.active = true;
        w.zeroed = beta_eff == 0.f;
        w.A = A;
        w.B = B;
        w.C = C;
        w.m = m;
        w.n = n;
        w.k = k;
        w.lda = lda;
        w.ldb = ldb;
        w.ldc = ldc;
        w.trans_a = 1;
        w.trans_b = 0;
        w.name = name;
    };
    const zg_waiting_bias& bw = ctx->bias_wait;
    const bool clear_of_bias =
        !bw.active || !plain ||
        (!ranges_meet(tC, operand_range(bw.gy, bw.R, bw.inner, bw.inner)) &&
         !ranges_meet(tC, operand_range(bw.gb, 1, bw.inner, bw.inner)) &&
         !ranges_meet(operand_range(bw.gb, 1, bw.inner, bw.inner), operand_range(A, trans_a ? k : m, trans_a ? m : k, lda)) &&
         !ranges_meet(operand_range(bw.gb, 1, bw.inner, bw.inner), operand_range(B, trans_b ? n : k, trans_b ? k : n, ldb)));
    if (ctx->deferred.active) {
        const zg_deferred_gemm& d = ctx->deferred;
        bool pass = false;
        if (d.kind == 2 && plain && !ctx->deferred_w.active && clear_of_bias &&
            gemm_validate(name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc) == ZG_HIP_OK) {
            const ByteRange dA = product_a_range(d), dB = product_b_range(d), dC = product_c_range(d);
            const ByteRange tA = operand_range(A, trans_a ? k : m, trans_a ? m : k, lda);
            const ByteRange tB = operand_range(B, trans_b ? n : k, trans_b ? k : n, ldb);
            pass = !ranges_meet(tC, dA) && !ranges_meet(tC, dB) && !ranges_meet(tC, dC) && !ranges_meet(dC, tA) &&
                   !ranges_meet(dC, tB);
        }
        if (pass) {
            // the layer's weight-gradient product after its input-gradient product: both small and fed by the same
            // dense gy, it waits too and the layer's backward leaves in one launch; else it goes out now
            if (w_shape && A == d.A && d.alpha == 1.f && d.lda == d.k && m == d.k && k == d.m && n == d.n &&
                gemm_is_tiny(d.m, d.n, d.k, 1, d.lda, d.ldb, n_cu)) {
                record_w();
                return ZG_HIP_OK;
            }
            return launch_now();
        }
        if (int rc = flush_deferred_gemm(ctx)) return rc;
    } else if (bw.active) {
        // only a bias gradient waits: the layer's input-gradient product may join it (below), its weight-gradient
        // product takes it along now (a first layer has no input gradient); anything else sends it out first
        const bool same_gy = plain && A == bw.gy && clear_of_bias;
        if (same_gy && w_shape && m == bw.inner && k == bw.R) {
            record_w();
            return flush_deferred_gemm(ctx);
        }
        const bool joins = same_gy && !trans_a && !trans_b && zeroed && beta_eff == 0.f && m == bw.R && k == bw.inner &&
                           lda == k;
        if (!joins)
            if (int rc = flush_deferred_gemm(ctx)) return rc;
    }
    const int kind = (!trans_a && trans_b) ? 1 : ((!trans_a && !trans_b && zeroed) ? 2 : 0);
    if (plain && beta_eff == 0.f && kind != 0) {
        if (int rc = gemm_validate(name, A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc)) {
            if (zeroed) (void)zg_hip_mem_fill(ctx, C, m * n, 0.f);
            return rc;
        }
        // whichever call launches the product later must not have to grow the workspace for it
        if (const size_t need = gemm_workspace_need(ctx, m, n, k, trans_a, trans_b, lda, ldb, 0))
            if (!workspace(ctx, need)) {
                if (zeroed) (void)zg_hip_mem_fill(ctx, C, m * n, 0.f);
                return ZG_HIP_EOOM;
            }
        zg_deferred_gemm& d = ctx->deferred;
        d = zg_deferred_gemm{};
        d.active = true;
        d.kind = kind;
        d.zeroed = zeroed;
        d.A = A;
        d.B = B;
        d.C = C;
        d.m = m;
        d.n = n;
        d.k = k;
        d.lda = lda;
        d.ldb = ldb;
        d.ldc = ldc;
        d.trans_a = trans_a;
        d.trans_b = trans_b;
        d.alpha = alpha;
        d.name = name;
        return ZG_HIP_OK;
    }
    return launch_now();
}

}  // namespace zg

ZG_API int zg_hip_matmul(zg_hip_ctx* ctx, const float* A, const float* B, float* C, size_t m, size_t n, size_t k,
                         int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    return gemm_entry(ctx, "matmul", A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, 1, 1, 1, 0, 0, 0);
}

ZG_API int zg_hip_linear_fwd(zg_hip_ctx* ctx, const float* x, const float* w, const float* bias, float* y, size_t batch,
                             size_t fan_in, size_t fan_out, int relu) {
    ZG_CTX(ctx);
    ZG_REQUIRE(fan_in >= 1, "linear_fwd: fan_in is 0");
    if (batch == 0 || fan_out == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && w && y, "linear_fwd: null pointer");
    const GemmExtras ex = {bias, nullptr, relu};
    return gemm_dispatch(ctx, "linear_fwd", x, w, y, batch, fan_out, fan_in, 0, 1, fan_in, fan_in, fan_out, 1.f, 0.f, 1, 1,
                         1, 0, 0, 0, 0, &ex);
}

// gx = (accumulate ? gx : 0) + gy . w, then gx = 0 where act_in <= 0 (act_in: the ReLU output that fed this layer,
// null for none): the input gradient of a Linear layer with the ReLU backward of the layer before it.
ZG_API int zg_hip_linear_bwd_input(zg_hip_ctx* ctx, const float* gy, const float* w, const float* act_in, float* gx,
                                   size_t batch, size_t fan_in, size_t fan_out, int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(fan_out >= 1, "linear_bwd_input: fan_out is 0");
    if (batch == 0 || fan_in == 0) return ZG_HIP_OK;
    ZG_REQUIRE(gy && w && gx, "linear_bwd_input: null pointer");
    if (accumulate) {  // the mask shares the epilogue registers with the old values of gx: two launches here
        if (int rc = gemm_dispatch(ctx, "linear_bwd_input", gy, w, gx, batch, fan_in, fan_out, 0, 0, fan_out, fan_in, fan_in,
                                   1.f, 1.f, 1, 1, 1, 0, 0, 0))
            return rc;
        return act_in ? zg_hip_relu_inplace_bwd(ctx, act_in, gx, batch * fan_in) : ZG_HIP_OK;
    }
    const GemmExtras ex = {nullptr, act_in, 0};
    return gemm_dispatch(ctx, "linear_bwd_input", gy, w, gx, batch, fan_in, fan_out, 0, 0, fan_out, fan_in, fan_in, 1.f, 0.f,
                         1, 1, 1, 0, 0, 0, 0, act_in ? &ex : nullptr);
}

// The backward of a Linear layer y = x . w^T + b whose output gradient gy is final (src/ndtensor.zig:1092-1136 for the
// two products, the bias's unbroadcast, and the ReLU backward of the layer before):
//   gw += gy^T . x;   gb += column sums of gy (gb may be null);   gx = gy . w, zeroed where act_in <= 0 (gx may be
//   null: no input gradient; act_in may be null: no mask).
// A layer small enough for the unstaged product kernel and the one-chunk column sum takes one launch; any other
// layer takes the separate ops.  Same values either way.
ZG_API int zg_hip_linear_bwd(zg_hip_ctx* ctx, const float* gy, const float* x, const float* w, const float* act_in,
                             float* gw, float* gb, float* gx, size_t batch, size_t fan_in, size_t fan_out) {
    ZG_CTX(ctx);
    if (batch == 0 || fan_in == 0 || fan_out == 0) return ZG_HIP_OK;
    ZG_REQUIRE(gy && x && gw, "linear_bwd: null pointer");
    ZG_REQUIRE(!gx || w, "linear_bwd: an input gradient needs the weights");
    const size_t n_cu = (size_t)ctx->n_cu;
    const bool small = gemm_is_tiny(fan_out, fan_in, batch, 1, fan_out, fan_in, n_cu) &&
                       (!gx || gemm_is_tiny(batch, fan_in, fan_out, 1, fan_out, fan_in, n_cu)) &&
                       // a single column or a single row takes other kernels in the separate op (row sums, a copy)
                       (!gb || (batch > 1 && fan_out > 1 && batch * fan_out <= kColSingleChunkMax));
    if (!small) {
        if (gb) {
            const uint64_t gy_shape[2] = {batch, fan_out}, gb_shape[1] = {fan_out};
            if (int rc = zg_hip_unbroadcast(ctx, gy, gy_shape, 2, gb, gb_shape, 1, nullptr, 0, 1.f, 1.f)) return rc;
        }
        if (gx)
            if (int rc = zg_hip_linear_bwd_input(ctx, gy, w, act_in, gx, batch, fan_in, fan_out, 0)) return rc;
        return gemm_dispatch(ctx, "linear_bwd", gy, x, gw, fan_out, fan_in, batch, 1, 0, fan_out, fan_in, fan_in, 1.f, 1.f,
                             1, 1, 1, 0, 0, 0);
    }
    return launch_linear_bwd_small(ctx, gy, x, fan_in, w, fan_in, act_in, gw, 1.f, gb, 1.f, gx, batch, fan_in, fan_out);
}

ZG_API int zg_hip_bmm_acc(zg_hip_ctx* ctx, const float* A, const uint64_t* A_shape, const float* B,
                          const uint64_t* B_shape, float* C, const uint64_t* C_shape, int trans_a, int trans_b,
                          size_t lda, size_t ldb, size_t ldc, float alpha, float beta) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    ZG_REQUIRE(A_shape && B_shape && C_shape, "bmm_acc: null shape");
    const size_t nba = A_shape[0], nbb = B_shape[0], nbc = C_shape[0];
    const size_t m = C_shape[1], n = C_shape[2], k = A_shape[2];
    ZG_REQUIRE(A_shape[1] == m, "bmm_acc: A rows %llu != C rows %zu", (unsigned long long)A_shape[1], m);
    ZG_REQUIRE(B_shape[1] == k && B_shape[2] == n, "bmm_acc: B shape does not match [%zu, %zu]", k, n);
    if (nbc > 0) ZG_REQUIRE(nba >= 1 && nbb >= 1, "bmm_acc: zero operand batches");
    return gemm_entry(ctx, "bmm_acc", A, B, C, m, n, k, trans_a, trans_b, lda, ldb, ldc, alpha, beta, nbc, nba ? nba : 1,
                      nbb ? nbb : 1, A_shape[1] * A_shape[2], B_shape[1] * B_shape[2], C_shape[1] * C_shape[2]);
}

ZG_API int zg_hip_matvec(zg_hip_ctx* ctx, const float* A, const float* x, float* y, size_t m, size_t n, int trans_a,
                         float alpha, float beta) {
    ZG_CTX(ctx);
    if (m == 0 || n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(A && x && y, "matvec: null pointer");
    const size_t n_cu = (size_t)ctx->n_cu;
    if (!trans_a) {
        const bool vec = aligned16(A) && aligned16(x) && n % 4 == 0;
        // lanes per row by row length; a whole workgroup for rows of more than 4096 columns
        // (one lane per row below 16 columns, two below 32: four lanes on a row of 4 values left three of them idle)
        const int tpr = n < 16 ? 1 : n < 32 ? 2 : n <= 64 ? 4 : n <= 256 ? 16 : n <= 4096 ? 64 : 256;
        const size_t wgs = ceil_div_sz(m, (size_t)(256 / tpr));
        ZG_REQUIRE(wgs <= 0x7fffffffull, "matvec: too many rows");
        // few long rows: segments of at least 4096 columns, about eight workgroups per compute unit
        size_t seg = n, n_seg = 1;
        if (tpr == 256 && m < 2 * n_cu && n >= 16384) {
            seg = ceil_div_sz(ceil_div_sz(n, ceil_div_sz(8 * n_cu, m)), 1024) * 1024;
            if (seg < 4096) seg = 4096;
            n_seg = ceil_div_sz(n, seg);
            if (n_seg > 65535) {
                n_seg = 65535;
                seg = ceil_div_sz(ceil_div_sz(n, n_seg), 1024) * 1024;
                n_seg = ceil_div_sz(n, seg);
            }
        }
        float* part = nullptr;
        if (n_seg > 1) {
            part = (float*)workspace(ctx, n_seg * m * sizeof(float));
            if (!part) return ZG_HIP_EOOM;
        }
        const dim3 grid((unsigned)wgs, (unsigned)n_seg);
#define ZG_GEMV(T)                                                                                                     \
    do {                                                                                                               \
        if (vec) hipLaunchKernelGGL((gemv_rows_kernel<T, true>), grid, dim3(256), 0, ctx->stream, A, x, y, part, m, n, seg, \
                                    alpha, beta);                                                                      \
        else hipLaunchKernelGGL((gemv_rows_kernel<T, false>), grid, dim3(256), 0, ctx->stream, A, x, y, part, m, n, seg, \
                                alpha, beta);                                                                          \
    } while (0)
        if (tpr == 1) ZG_GEMV(1);
        else if (tpr == 2) ZG_GEMV(2);
        else if (tpr == 4) ZG_GEMV(4);
        else if (tpr == 16) ZG_GEMV(16);
        else if (tpr == 64) ZG_GEMV(64);
        else ZG_GEMV(256);
#undef ZG_GEMV
        ZG_LAUNCH_CHECK();
        if (n_seg > 1)
            hipLaunchKernelGGL(vec_final_kernel, dim3((unsigned)ceil_div_sz(m, 64)), dim3(256), 0, ctx->stream, part, y, m,
                               n_seg, alpha, beta);
    } else {
        // column-threads as the column reductions have them: 4 columns per thread where rows start on 16-byte
        // boundaries, at most 64 column-threads (1 KiB of a row) per workgroup
        const int V = (n % 4 == 0 && aligned16(A)) ? 4 : 1;
        const size_t colv = n / V;
        int log2_cx = 0;
        // 16 row-threads (and 16 column-threads) where a row-thread gets four rows or more, fewer for shorter matrices
        // (7 x 1048576: 11.5 us with 16 row-threads, 5.7 us with 4; 64 x 1048576: 50.5 us with 4, 39.1 us with 16)
        // single columns (V = 1): 64 column-threads, so that a wave still reads 256 adjacent bytes of a row (16 of them,
        // 64 bytes: [8192, 32001] at 33 % of 8 TB/s)
        const int cx_max = V == 1 ? 6 : m >= 64 ? 4 : m >= 32 ? 5 : 6;
        while (((size_t)1 << log2_cx) < colv && log2_cx < cx_max) log2_cx++;
        // narrower column groups (down to 16 column-threads) while they are fewer than two per compute unit: a wide matrix
        // of few rows then needs no row chunks at all
        while (V == 4 && log2_cx > 4 && ceil_div_sz(colv, (size_t)1 << log2_cx) < 2 * n_cu) log2_cx--;
        const size_t gx = ceil_div_sz(colv, (size_t)1 << log2_cx);
        const size_t ry = (size_t)256 >> log2_cx;
        // row chunks: about two workgroups per compute unit, at least 64 rows and eight trips of ry rows each, at most 1024
        size_t chunks = ceil_div_sz(2 * n_cu, gx);
        size_t max_chunks = ceil_div_sz(m, ry * 8);
        if (max_chunks > m / 64) max_chunks = m / 64;
        if (chunks > max_chunks) chunks = max_chunks;
        if (chunks > 1024) chunks = 1024;
        if (m * n <= kColSingleChunkMax || chunks < 1) chunks = 1;
        const size_t rows_per_chunk = ceil_div_sz(m, chunks);
        chunks = ceil_div_sz(m, rows_per_chunk);
        float* part = nullptr;
        if (chunks > 1) {
            part = (float*)workspace(ctx, chunks * n * sizeof(float));
            if (!part) return ZG_HIP_EOOM;
        }
        ZG_REQUIRE(gx <= 0x7fffffffull, "matvec: too many columns");
        const dim3 grid((unsigned)gx, (unsigned)chunks);
        if (V == 4)
            hipLaunchKernelGGL(gemv_t_kernel<4>, grid, dim3(256), 0, ctx->stream, A, x, y, part, m, n, log2_cx, rows_per_chunk,
                               alpha, beta);
        else
            hipLaunchKernelGGL(gemv_t_kernel<1>, grid, dim3(256), 0, ctx->stream, A, x, y, part, m, n, log2_cx, rows_per_chunk,
                               alpha, beta);
        ZG_LAUNCH_CHECK();
        if (chunks > 1)
            hipLaunchKernelGGL(vec_final_kernel, dim3((unsigned)ceil_div_sz(n, 64)), dim3(256), 0, ctx->stream, part, y, n,
                               chunks, alpha, beta);
    }
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_outer(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, float* A, float alpha) {
    ZG_CTX(ctx);
    if (xl == 0 || yl == 0) return ZG_HIP_OK;
    ZG_REQUIRE(x && y && A, "outer: null pointer");
    const bool vec = aligned16(A) && aligned16(y) && yl % 4 == 0;
    size_t blocks = ceil_div_sz(xl * yl, vec ? 256 * 16 : 256);
    // a workgroup per 16 KiB of A at any size (16384 x 16384: 446 -> 363 us against a grid capped at 16 per compute unit);
    // the value-by-value form keeps the cap, its threads walking the rest (1048576 x 7: 12.2 us capped, 16.8 us not)
    const size_t cap = vec ? 0x7fffffffull : (size_t)ctx->n_cu * 16;
    if (blocks > cap) blocks = cap;
    if (vec) hipLaunchKernelGGL(ger_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, x, xl, y, yl, A, alpha);
    else hipLaunchKernelGGL(ger_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, x, xl, y, yl, A, alpha);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_transpose(zg_hip_ctx* ctx, const float* A, float* B, size_t m, size_t n, float alpha) {
    ZG_CTX(ctx);
    if (m == 0 || n == 0) return ZG_HIP_OK;
    ZG_REQUIRE(A && B, "transpose: null pointer");
    ZG_REQUIRE(A != B, "transpose: in-place transpose is not supported");
    if (aligned16(A) && aligned16(B) && m % 4 == 0 && n % 4 == 0 && ceil_div_sz(m, 64) * ceil_div_sz(n, 64) <= 0x7fffffffull) {
        const unsigned gx = (unsigned)ceil_div_sz(n, 64), gy = (unsigned)ceil_div_sz(m, 64);
        // wide matrices only: on 65536 x 4096 and on row lengths that are no multiple of 4 KiB the order along the rows
        // is 3 to 8 % faster
        const bool diagonal = n % 1024 == 0 && m % 1024 == 0 && n >= m;
        dim3 grid((unsigned)((size_t)gx * gy));
        hipLaunchKernelGGL(transpose_vec_kernel, grid, dim3(256), 0, ctx->stream, A, B, m, n, alpha, diagonal, gx, gy);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    dim3 grid((unsigned)ceil_div_sz(n, 32), (unsigned)ceil_div_sz(m, 32));
    ZG_REQUIRE(grid.y <= 65535, "transpose: too many rows");
    hipLaunchKernelGGL(transpose_kernel, grid, dim3(256), 0, ctx->stream, A, B, m, n, alpha);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}
