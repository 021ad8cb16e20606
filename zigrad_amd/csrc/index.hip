// Indexing ops: gather offsets, scatter_add, index_select fwd/bwd and the GCN degree-scaled
// message-passing scatter with its backward.
//
// Every accumulating op here is a destination-sorted segmented reduction: the input indices are
// bucketed by destination (integer histogram + scan + placement), each bucket is put back into input
// order, and one thread group then adds a destination's contributions one after the other in that
// order.  That is the order of the sequential host loops (src/device/host_device.zig:1039-1087,
// :1356-1403), so results are deterministic and round like the host's; there are no floating-point
// atomics.  The work is latency/HBM bound: indices and rows are read once, destinations written once.
#include "common.h"

namespace zg {

// ------------------------------------------------------------------------------------------------
// segment plan: row_ptr[nb + 1], perm[n] (input positions grouped by bucket, ascending inside a bucket)
// ------------------------------------------------------------------------------------------------
struct Plan {
    uint32_t* row_ptr;   // nb + 1
    uint32_t* cursor;    // nb
    uint32_t* perm_tmp;  // n
    uint32_t* perm;      // n
    uint32_t* peer;      // n: optional payload (the other endpoint of an edge) in the order of perm
    uint32_t* peer_tmp;  // n: the payload in the order of perm_tmp
    uint32_t* tile_sums; // scan scratch
    uint32_t* long_list; // [0] = number of long buckets, then their ids (at most n / kLongBucket of them)
    // scratch of the radix build (n >= kRadixMinEntries): two key arrays, the payload as 32-bit values in input order,
    // per-tile digit counts; null for shorter inputs
    uint32_t* rx_keys[2];
    uint32_t* rx_in0;  // the 32-bit keys in input order (what the first pass reads): rx_keys[0], or a buffer that outlives the build
    uint32_t* rx_peer0;
    uint32_t* rx_counts;
    size_t n, nb;
    long n_long;         // host copy of long_list[0] where the host has read it back (kept plans), else -1
};

// A bucket with more entries than this is "long": its entries are added by a whole wave (loads in parallel, additions
// still one after the other in input order) instead of by one thread.
constexpr uint32_t kLongBucket = 256;
// Up to this length a bucket is put back into input order by ranking every entry against every other (len^2 / 64
// loads per lane); beyond it the bucket is rebuilt in order by one pass over the input.
constexpr uint32_t kRankMax = 1024;

constexpr int kScanTile = 2048;  // elements per workgroup of the scan (256 threads x 8)

static size_t align_up(size_t v, size_t a) {
    return (v + a - 1) / a * a;
}

// Inputs of at least this many entries are ordered by the radix build (build_plan_radix), shorter ones by the
// histogram / place / rank build (build_plan).  A global atomic costs about 40 ns on this chip (the eight L2s are not
// coherent with each other, so device-scope atomics are served by the memory side) and the short build spends two per
// entry; the radix build spends none but takes ten launches of at least 4 to 5 us each.  Measured, ordering only: one
// million entries into 100 k buckets 145 us (atomics) against 112 us (radix), eight million into a million about
// 1100 us against 510 us; at a quarter of a million entries the two take the same time, and below that the short
// build is the faster one on keys that do not repeat much (13264 entries into 2708 buckets: 24 us against 47 us).
constexpr size_t kRadixMinEntries = (size_t)1 << 18;
constexpr int kRxThreads = 256, kRxPerThread = 16, kRxTile = kRxThreads * kRxPerThread;  // entries per workgroup
// digit width: 8 bits a pass, or 9 where that saves a pass (17, 18 and 25 to 27 bits of bucket number: two passes instead
// of three for 65 K to 262 K buckets); the kernels take it as a template argument
constexpr int kRxMaxBins = 512;
static bool radix_build_applies(size_t n, size_t nb) {
    // few destinations for many entries (64 and more each on average): the short build's atomics all land on the same
    // few addresses and its buckets are long to rank (13264 entries into 17 buckets: 217 us against 35 us; into 1000
    // buckets: 24 us against 48 us)
    const bool crowded = n >= 512 && n / 64 >= nb;
    return (n >= kRadixMinEntries || crowded) && nb < ((size_t)1 << 31);
}

static size_t plan_bytes(size_t n, size_t nb) {
    size_t tiles = ceil_div_sz(nb + 1, kScanTile);
    size_t bytes = align_up((nb + 1) * 4, 256) + align_up(nb * 4, 256) + 4 * align_up(n * 4, 256) +
                   align_up((tiles + 1) * 4, 256) + align_up((n / kLongBucket + 2) * 4, 256);
    if (radix_build_applies(n, nb))
        bytes += 3 * align_up(n * 4, 256) + align_up(ceil_div_sz(n, kRxTile) * kRxMaxBins * 4, 256);
    return bytes;
}

static Plan carve_plan(void* mem, size_t n, size_t nb) {
    char* p = (char*)mem;
    Plan pl;
    pl.n = n;
    pl.nb = nb;
    pl.n_long = -1;
    pl.row_ptr = (uint32_t*)p;
    p += align_up((nb + 1) * 4, 256);
    pl.cursor = (uint32_t*)p;
    p += align_up(nb * 4, 256);
    pl.perm_tmp = (uint32_t*)p;
    p += align_up(n * 4, 256);
    pl.perm = (uint32_t*)p;
    p += align_up(n * 4, 256);
    pl.peer = (uint32_t*)p;
    p += align_up(n * 4, 256);
    pl.peer_tmp = (uint32_t*)p;
    p += align_up(n * 4, 256);
    pl.tile_sums = (uint32_t*)p;
    p += align_up((ceil_div_sz(nb + 1, kScanTile) + 1) * 4, 256);
    pl.long_list = (uint32_t*)p;
    p += align_up((n / kLongBucket + 2) * 4, 256);
    pl.rx_keys[0] = pl.rx_keys[1] = pl.rx_in0 = pl.rx_peer0 = pl.rx_counts = nullptr;
    if (radix_build_applies(n, nb)) {
        pl.rx_keys[0] = pl.rx_in0 = (uint32_t*)p;
        p += align_up(n * 4, 256);
        pl.rx_keys[1] = (uint32_t*)p;
        p += align_up(n * 4, 256);
        pl.rx_peer0 = (uint32_t*)p;
        p += align_up(n * 4, 256);
        pl.rx_counts = (uint32_t*)p;
    }
    return pl;
}

__global__ void zero_u32_kernel(uint32_t* a, size_t na, uint32_t* b, size_t nb, uint32_t* one = nullptr,
                                uint32_t* other = nullptr) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < na; k += nt) a[k] = 0;
    for (size_t k = i; k < nb; k += nt) b[k] = 0;
    if (i == 0 && one) one[0] = 0;
    if (i == 0 && other) other[0] = 0;
}

// key = idx[e] / divisor (divisor 1 for plain indices)
__global__ void histogram_kernel(const uint64_t* keys, size_t n, size_t nb, uint32_t* counts) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; e < n; e += nt) {
        uint64_t k = keys[e];
        if (k < nb) atomicAdd(&counts[k], 1u);
    }
}

// exclusive scan, three launches: per-tile scan + tile sums, scan of tile sums (scan_single_kernel), add back
__global__ __launch_bounds__(256) void scan_tiles_kernel(uint32_t* data, size_t n, uint32_t* tile_sums) {
    __shared__ uint32_t wave_tot[4];
    const size_t base = (size_t)blockIdx.x * kScanTile + (size_t)threadIdx.x * 8;
    uint32_t v[8], s = 0;
    // a thread's eight values as two 16-byte pieces where they are all there (value by value, a load touched 64 lanes x 4
    // bytes spread over 2 KiB: 16.7 M buckets took 68 us)
    const bool whole = base + 8 <= n && (reinterpret_cast<uintptr_t>(data) & 15u) == 0;
    if (whole) {
        const uint4 a = *reinterpret_cast<const uint4*>(data + base), b = *reinterpret_cast<const uint4*>(data + base + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
#pragma unroll
        for (int k = 0; k < 8; k++) s += v[k];
    } else {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[k] = (base + k < n) ? data[base + k] : 0;
            s += v[k];
        }
    }
    // inclusive scan of s across the workgroup
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t inc = s;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        uint32_t t = __shfl_up(inc, d, 64);
        if (lane >= d) inc += t;
    }
    if (lane == 63) wave_tot[wave] = inc;
    __syncthreads();
    uint32_t wave_off = 0;
    for (int w = 0; w < wave; w++) wave_off += wave_tot[w];
    uint32_t run = wave_off + inc - s;  // exclusive prefix of this thread's first element
    if (whole) {
        uint32_t o[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            o[k] = run;
            run += v[k];
        }
        *reinterpret_cast<uint4*>(data + base) = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4*>(data + base + 4) = make_uint4(o[4], o[5], o[6], o[7]);
    } else {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            if (base + k < n) data[base + k] = run;
            run += v[k];
        }
    }
    if (threadIdx.x == 255) tile_sums[blockIdx.x] = wave_off + inc;
}

// exclusive scan of a short array by one workgroup, 2048 elements per round with a running carry
__global__ __launch_bounds__(256) void scan_single_kernel(uint32_t* data, size_t n) {
    __shared__ uint32_t wave_tot[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t carry = 0;
    for (size_t c = 0; c < n; c += kScanTile) {
        const size_t base = c + (size_t)threadIdx.x * 8;
        uint32_t v[8], s = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[k] = (base + k < n) ? data[base + k] : 0;
            s += v[k];
        }
        uint32_t inc = s;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            uint32_t t = __shfl_up(inc, d, 64);
            if (lane >= d) inc += t;
        }
        __syncthreads();  // wave_tot of the previous round has been read by everyone
        if (lane == 63) wave_tot[wave] = inc;
        __syncthreads();
        uint32_t wave_off = carry;
        for (int w = 0; w < wave; w++) wave_off += wave_tot[w];
        uint32_t run = wave_off + inc - s;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            if (base + k < n) data[base + k] = run;
            run += v[k];
        }
        carry += wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
    }
}

__global__ __launch_bounds__(256) void scan_add_kernel(uint32_t* data, size_t n, const uint32_t* tile_sums) {
    const uint32_t off = tile_sums[blockIdx.x];
    const size_t base = (size_t)blockIdx.x * kScanTile;
    for (int k = threadIdx.x; k < kScanTile; k += 256)
        if (base + k < n) data[base + k] += off;
}

// `payload` (the other index array of an edge list, possibly in host memory) is read here, in input order and
// coalesced, and travels with its entry from then on in device memory.
__global__ void place_kernel(const uint64_t* keys, size_t n, size_t nb, const uint32_t* row_ptr, uint32_t* cursor,
                             uint32_t* perm_tmp, const uint64_t* payload, uint32_t* peer_tmp) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    for (; e < n; e += nt) {
        uint64_t k = keys[e];
        if (k < nb) {
            uint32_t pos = row_ptr[k] + atomicAdd(&cursor[k], 1u);
            perm_tmp[pos] = (uint32_t)e;
            if (payload) {
                const uint64_t v = payload[e];
                peer_tmp[pos] = v < 0xffffffffull ? (uint32_t)v : 0xffffffffu;
            }
        }
    }
}

// Put each bucket back into ascending input position: rank of an entry = number of smaller entries
// in its bucket.  One wave per bucket; the bucket's positions are first copied to LDS, from where every lane reads
// them four at a time (all lanes the same address), so that a bucket of a thousand entries costs a thousand LDS reads
// per lane and not a thousand trips to the L1 each (1000 entries in one bucket: 1.2 ms that way).
// With `peer_tmp` the payload is laid out in the same order, so that the apply kernels read it next to perm.
// Buckets of more than kLongBucket entries are listed in `long_list`; those of more than kRankMax entries are left
// to order_long_segments_kernel.
// With `list` (and its length at list_count[0]) the waves take the buckets listed there instead of all buckets, and
// the long ones among them have been listed already (order_sparse_kernel).
__global__ __launch_bounds__(256) void order_segments_kernel(const uint32_t* row_ptr, size_t nb, const uint32_t* perm_tmp,
                                                              uint32_t* perm, const uint32_t* peer_tmp, uint32_t* peer,
                                                              uint32_t* long_list, const uint32_t* list = nullptr,
                                                              const uint32_t* list_count = nullptr) {
    __shared__ __align__(16) uint32_t ids[4][kRankMax];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    size_t b = (size_t)blockIdx.x * 4 + wave;
    if (list) b = b < list_count[0] ? list[b] : nb;
    uint32_t s = 0, len = 0;
    if (b < nb) {
        s = row_ptr[b];
        len = row_ptr[b + 1] - s;
        if (!list && len > kLongBucket && lane == 0) long_list[1 + atomicAdd(&long_list[0], 1u)] = (uint32_t)b;
    }
    const bool here = b < nb && len <= kRankMax;
    const uint32_t len4 = (len + 3) & ~3u;
    if (here)
        for (uint32_t i = lane; i < len4; i += 64) ids[wave][i] = i < len ? perm_tmp[s + i] : 0xffffffffu;  // no position is above the padding
    __syncthreads();
    if (!here) return;
    for (uint32_t i = lane; i < len; i += 64) {
        const uint32_t id = ids[wave][i];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < len4; j += 4) {
            const uint4 q = *reinterpret_cast<const uint4*>(&ids[wave][j]);
            rank += (q.x < id ? 1u : 0u) + (q.y < id ? 1u : 0u) + (q.z < id ? 1u : 0u) + (q.w < id ? 1u : 0u);
        }
        perm[s + rank] = id;
        if (peer_tmp) peer[s + rank] = peer_tmp[s + i];
    }
}

// Many destinations for few entries (four destinations per entry and more): a wave per bucket would spend its launch
// on empty buckets (65536 entries into 16.7 M destinations: 1.07 ms).  Here a thread looks at one bucket: nothing to do
// for an empty one, a copy for a single entry, a rank by counting for up to kSparseSerial entries; longer buckets go to
// `mid_list` (count at mid_count[0]) for order_segments_kernel, a wave each, and those of more than kLongBucket entries
// to `long_list` as order_segments_kernel lists them.
constexpr uint32_t kSparseSerial = 16;
__global__ __launch_bounds__(256) void order_sparse_kernel(const uint32_t* row_ptr, size_t nb, const uint32_t* perm_tmp,
                                                            uint32_t* perm, const uint32_t* peer_tmp, uint32_t* peer,
                                                            uint32_t* long_list, uint32_t* mid_count, uint32_t* mid_list) {
    const size_t b = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nb) return;
    const uint32_t s = row_ptr[b], len = row_ptr[b + 1] - s;
    if (len == 0) return;
    if (len > kLongBucket) long_list[1 + atomicAdd(&long_list[0], 1u)] = (uint32_t)b;
    if (len == 1) {
        perm[s] = perm_tmp[s];
        if (peer_tmp) peer[s] = peer_tmp[s];
    } else if (len <= kSparseSerial) {
        uint32_t ids[kSparseSerial];
#pragma unroll
        for (uint32_t i = 0; i < kSparseSerial; i++) ids[i] = i < len ? perm_tmp[s + i] : 0xffffffffu;
#pragma unroll
        for (uint32_t i = 0; i < kSparseSerial; i++) {
            if (i < len) {
                uint32_t rank = 0;
#pragma unroll
                for (uint32_t j = 0; j < kSparseSerial; j++) rank += ids[j] < ids[i] ? 1u : 0u;
                perm[s + rank] = ids[i];
                if (peer_tmp) peer[s + rank] = peer_tmp[s + i];
            }
        }
    } else if (len <= kRankMax) {
        mid_list[atomicAdd(mid_count, 1u)] = (uint32_t)b;
    }
}

// The buckets of more than kRankMax entries, rebuilt in input order: one workgroup per such bucket walks the whole
// key array, 4096 entries a round, and writes the positions whose key is the bucket's, in order (a workgroup-wide
// prefix sum of the per-thread match counts gives each thread its place).  Cost: one read of the key array per very
// long bucket, and there are at most n / kRankMax of them.
constexpr int kOrderLongThreads = 1024;
__global__ __launch_bounds__(kOrderLongThreads) void order_long_segments_kernel(const uint64_t* keys, size_t n,
                                                                                const uint32_t* row_ptr,
                                                                                const uint32_t* long_list, uint32_t* perm,
                                                                                const uint64_t* payload, uint32_t* peer) {
    __shared__ uint32_t wave_tot[kOrderLongThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t n_long = long_list[0];
    for (uint32_t li = blockIdx.x; li < n_long; li += gridDim.x) {
        const uint32_t b = long_list[1 + li];
        const uint32_t s = row_ptr[b], len = row_ptr[b + 1] - s;
        if (len <= kRankMax) continue;  // ordered by order_segments_kernel already (uniform over the workgroup)
        uint32_t written = 0;
        for (size_t e0 = 0; e0 < n; e0 += (size_t)kOrderLongThreads * 4) {
            const size_t mine = e0 + (size_t)threadIdx.x * 4;
            bool hit[4];
            uint32_t cnt = 0;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                hit[u] = (mine + u < n) && keys[mine + u] == (uint64_t)b;
                cnt += hit[u] ? 1u : 0u;
            }
            uint32_t inc = cnt;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t t = __shfl_up(inc, d, 64);
                if (lane >= d) inc += t;
            }
            __syncthreads();  // wave_tot of the previous round has been read by everyone
            if (lane == 63) wave_tot[wave] = inc;
            __syncthreads();
            uint32_t before = 0, total = 0;
            for (int w = 0; w < kOrderLongThreads / 64; w++) {
                const uint32_t t = wave_tot[w];
                before += (w < wave) ? t : 0u;
                total += t;
            }
            uint32_t pos = s + written + before + inc - cnt;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (hit[u]) {
                    if (pos < s + len) {  // cannot fail: the histogram counted the same matches
                        perm[pos] = (uint32_t)(mine + u);
                        if (payload) {
                            const uint64_t v = payload[mine + u];
                            peer[pos] = v < 0xffffffffull ? (uint32_t)v : 0xffffffffu;
                        }
                    }
                    pos++;
                }
            }
            written += total;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The radix build: a stable least-significant-digit sort of (bucket, input position) by bucket, 8 bits a pass, so the
// entries of a bucket end up in input order by construction (no ranking pass) and no global atomic is needed.
// A pass is three launches.  count: every workgroup counts the digits of its tile of 4096 entries in LDS.  scan: one
// workgroup turns the counts [tile][digit] into starting positions, digit-major.  scatter: every workgroup ranks its
// entries among those of the same digit in its tile, in input order, and writes key and position to their places.
// Nothing waits for another workgroup inside a kernel.  A key outside [0, nb) becomes nb and sorts behind all buckets.
// ------------------------------------------------------------------------------------------------
// A kept plan is rebuilt only when the arrays it was built from have changed.  `gate` (null: build unconditionally) is
// two words in device memory.  The first kernel of a build compares the arrays with the 32-bit copies the plan keeps
// (keys32, peer0), brings the copies up to date and sets gate[0] where it finds a difference; the first scan copies
// gate[0] to gate[1]; every later kernel returns at once when gate[1] is zero, and the first scatter pass, which reads
// gate[1] only, clears gate[0] for the next build.  No kernel reads a word that another workgroup of the same launch
// writes.
struct RxGate {
    const uint32_t* in = nullptr;  // the kernel runs when this is null or points at a non-zero word
    uint32_t* move_to = nullptr;   // first scan only: receives *in
    uint32_t* tally = nullptr;     // first scan only: [0] builds skipped, [1] builds done, in device memory ...
    uint32_t* tally_host = nullptr;  // ... and mirrored into pinned host memory, where the host reads it without waiting
};

template <int BITS>
__global__ __launch_bounds__(kRxThreads) void rx_count_first_kernel(const uint64_t* keys, const uint64_t* payload, size_t n,
                                                                    uint32_t nb, uint32_t* keys32, uint32_t* peer0,
                                                                    uint32_t* counts, uint32_t* gate) {
    constexpr int kRxBins = 1 << BITS;
    __shared__ uint32_t hist[kRxBins];
    for (int i = threadIdx.x; i < kRxBins; i += kRxThreads) hist[i] = 0;
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * kRxTile;
    bool changed = false;
#pragma unroll 4
    for (int r = 0; r < kRxPerThread; r++) {
        const size_t e = base + (size_t)r * kRxThreads + threadIdx.x;
        if (e < n) {
            const uint64_t k = keys[e];
            const uint32_t k32 = k < nb ? (uint32_t)k : nb;
            if (!gate) {
                keys32[e] = k32;
            } else if (keys32[e] != k32) {
                keys32[e] = k32;
                changed = true;
            }
            if (payload) {
                const uint64_t v = payload[e];
                const uint32_t v32 = v < 0xffffffffull ? (uint32_t)v : 0xffffffffu;
                if (!gate) {
                    peer0[e] = v32;
                } else if (peer0[e] != v32) {
                    peer0[e] = v32;
                    changed = true;
                }
            }
            atomicAdd(&hist[k32 & (kRxBins - 1)], 1u);  // LDS: the order of the increments does not matter
        }
    }
    if (gate && __any(changed) && (threadIdx.x & 63) == 0) gate[0] = 1u;  // every writer stores the same value
    __syncthreads();
    for (int i = threadIdx.x; i < kRxBins; i += kRxThreads) counts[(size_t)blockIdx.x * kRxBins + i] = hist[i];
}

template <int BITS>
__global__ __launch_bounds__(kRxThreads) void rx_count_kernel(const uint32_t* keys32, size_t n, int shift, uint32_t* counts,
                                                              const uint32_t* gate) {
    if (gate && *gate == 0) return;
    constexpr int kRxBins = 1 << BITS;
    __shared__ uint32_t hist[kRxBins];
    for (int i = threadIdx.x; i < kRxBins; i += kRxThreads) hist[i] = 0;
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * kRxTile;
#pragma unroll 4
    for (int r = 0; r < kRxPerThread; r++) {
        const size_t e = base + (size_t)r * kRxThreads + threadIdx.x;
        if (e < n) atomicAdd(&hist[(keys32[e] >> shift) & (kRxBins - 1)], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kRxBins; i += kRxThreads) counts[(size_t)blockIdx.x * kRxBins + i] = hist[i];
}

// counts[tile][digit] -> first output position of that tile's entries with that digit: all of digit 0 by tile, then
// all of digit 1, ...  A workgroup of 1024 threads takes 256 digits: thread (part, d) owns a quarter of the tiles of
// digit d, so a thread's two walks over its counts are a few batches of independent loads (a thread per digit took
// 20 us on 245 tiles, and so did one workgroup for 512 digits).  With 9-bit digits a second workgroup takes the upper
// 256 and finds what lies before them without the first one's help.
constexpr int kRxScanThreads = 1024, kRxScanDigits = 256, kRxScanParts = kRxScanThreads / kRxScanDigits;
template <int BITS>
__global__ __launch_bounds__(kRxScanThreads) void rx_scan_kernel(uint32_t* __restrict__ counts, size_t n_tiles, RxGate gate,
                                                                  uint32_t* long_list, uint32_t n_entries) {
    constexpr int kRxBins = 1 << BITS;
    static_assert(kRxBins <= 2 * kRxScanDigits, "the second workgroup finds its base from the total: two groups at most");
    if (gate.in) {
        // every workgroup of this launch reads the word; the one that set it is cleared by a later launch (the first
        // scatter pass), which does not read it
        const uint32_t go = *gate.in;
        if (gate.move_to && blockIdx.x == 0 && threadIdx.x == 0) {
            *gate.move_to = go;
            const uint32_t seen = gate.tally[go ? 1 : 0] + 1u;
            gate.tally[go ? 1 : 0] = seen;
            gate.tally_host[go ? 1 : 0] = seen;
        }
        if (go == 0) return;
    }
    if (long_list && blockIdx.x == 0 && threadIdx.x == 0) long_list[0] = 0;  // first scan: the finish kernel appends to the list
    __shared__ uint32_t part_sum[kRxScanParts][kRxScanDigits];
    __shared__ uint32_t digit_base[kRxScanDigits];
    __shared__ uint32_t wave_tot[kRxScanDigits / 64];
    const int dl = threadIdx.x & (kRxScanDigits - 1), part = threadIdx.x / kRxScanDigits;
    const int d = blockIdx.x * kRxScanDigits + dl;  // 256 digits a workgroup: one workgroup, or two for 9-bit digits
    const size_t per_part = (n_tiles + kRxScanParts - 1) / kRxScanParts;
    const size_t t0 = (size_t)part * per_part, t1 = (t0 + per_part < n_tiles) ? t0 + per_part : n_tiles;
    uint32_t total = 0;
    size_t t = t0;
    for (; t < t1; t += 16) {  // sixteen independent loads a batch, the last batch predicated
        uint32_t c[16];
#pragma unroll
        for (int u = 0; u < 16; u++) c[u] = (t + u < t1) ? counts[(t + u) * kRxBins + d] : 0u;
#pragma unroll
        for (int u = 0; u < 16; u++) total += c[u];
    }
    part_sum[part][dl] = total;
    __syncthreads();
    if (part == 0) {
        const int lane = dl & 63, wave = dl >> 6;
        uint32_t all = 0;
#pragma unroll
        for (int p = 0; p < kRxScanParts; p++) all += part_sum[p][dl];
        uint32_t inc = all;
#pragma unroll
        for (int s = 1; s < 64; s <<= 1) {
            const uint32_t v = __shfl_up(inc, s, 64);
            if (lane >= s) inc += v;
        }
        if (lane == 63) wave_tot[wave] = inc;
        digit_base[dl] = inc - all;  // within the wave; the earlier waves' totals are added below
    }
    __syncthreads();
    uint32_t run = digit_base[dl];
    for (int w = 0; w < (dl >> 6); w++) run += wave_tot[w];
    if (blockIdx.x != 0) {
        // the second workgroup's digits come after all of the first's: every entry has one digit, so what lies before
        // them is the number of entries less what this workgroup counted
        uint32_t group = 0;
        for (int w = 0; w < kRxScanDigits / 64; w++) group += wave_tot[w];
        run += n_entries - group;
    }
    for (int p = 0; p < part; p++) run += part_sum[p][dl];
    for (t = t0; t < t1; t += 16) {
        uint32_t c[16];
#pragma unroll
        for (int u = 0; u < 16; u++) c[u] = (t + u < t1) ? counts[(t + u) * kRxBins + d] : 0u;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            if (t + u < t1) counts[(t + u) * kRxBins + d] = run;
            run += c[u];
        }
    }
}

// Entry e of a tile belongs to round r = (e / 256) and wave w: "wave-round" q = 4 r + w, lanes in input order, so
// (q, lane) ascending is input order.  Rank of an entry among the tile's entries of its digit = entries of its digit in
// earlier wave-rounds (a prefix over q of table[q][digit]) + entries of its digit in lower lanes of its own wave-round
// (ballots).  The tile is then put in digit order in LDS and written out from there, so that the lanes of a store
// instruction write runs of consecutive addresses (one run per digit present) instead of 64 scattered words.
template <int BITS>
__global__ __launch_bounds__(kRxThreads) void rx_scatter_kernel(const uint32_t* __restrict__ keys_in,
                                                                const uint32_t* __restrict__ vals_in, size_t n, int shift,
                                                                const uint32_t* __restrict__ starts,
                                                                uint32_t* __restrict__ keys_out,
                                                                uint32_t* __restrict__ vals_out, const uint32_t* gate,
                                                                uint32_t* gate_clear) {
    if (gate && *gate == 0) return;
    if (gate_clear && blockIdx.x == 0 && threadIdx.x == 0) *gate_clear = 0u;  // the word no workgroup of this launch reads
    constexpr int kRxBits = BITS, kRxBins = 1 << BITS;
    constexpr int DPT = kRxBins / kRxThreads;  // digits a thread owns in the prefix step: t * DPT .. t * DPT + DPT - 1
    constexpr int Q = kRxPerThread * (kRxThreads / 64);
    // the ranking table, then (once every entry knows its place) the tile in digit order: keys, then values
    __shared__ __align__(16) uint32_t lds[Q * kRxBins / 2];
    static_assert(sizeof(lds) >= 2 * kRxTile * sizeof(uint32_t), "the sorted tile reuses the table's memory");
    uint16_t(*table)[kRxBins] = reinterpret_cast<uint16_t(*)[kRxBins]>(lds);
    __shared__ uint32_t first[kRxBins];       // where the tile's entries of a digit go in the output
    __shared__ uint32_t tile_start[kRxBins];  // where they start in the sorted tile
    __shared__ uint32_t wave_tot[kRxThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t base = (size_t)blockIdx.x * kRxTile;
    const uint32_t in_tile = (uint32_t)((n - base < (size_t)kRxTile) ? n - base : (size_t)kRxTile);
    uint32_t key[kRxPerThread], val[kRxPerThread];
    uint16_t rank[kRxPerThread];
#pragma unroll
    for (int r = 0; r < kRxPerThread; r++) {  // every load of the tile is in flight before the first use
        const size_t e = base + (size_t)r * kRxThreads + threadIdx.x;
        key[r] = e < n ? keys_in[e] : 0xffffffffu;
        val[r] = (e < n && vals_in) ? vals_in[e] : (uint32_t)e;
    }
    uint32_t my_first[DPT];
#pragma unroll
    for (int j = 0; j < DPT; j++) my_first[j] = starts[(size_t)blockIdx.x * kRxBins + threadIdx.x + j * kRxThreads];
    for (int i = threadIdx.x; i < Q * kRxBins / 2; i += kRxThreads) lds[i] = 0;
#pragma unroll
    for (int j = 0; j < DPT; j++) first[threadIdx.x + j * kRxThreads] = my_first[j];
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kRxPerThread; r++) {
        const size_t e = base + (size_t)r * kRxThreads + threadIdx.x;
        const bool live = e < n;
        const uint32_t digit = (key[r] >> shift) & (kRxBins - 1);
        // the lanes of this wave-round that hold the same digit (dead lanes match nobody)
        unsigned long long peers = __ballot(live);
#pragma unroll
        for (int b = 0; b < kRxBits; b++) {
            const unsigned long long set = __ballot(live && ((digit >> b) & 1u));
            peers &= ((digit >> b) & 1u) ? set : ~set;
        }
        const unsigned long long below = peers & ((1ull << lane) - 1ull);
        rank[r] = (uint16_t)__popcll(below);
        if (live && below == 0) table[r * (kRxThreads / 64) + wave][digit] = (uint16_t)__popcll(peers);
    }
    __syncthreads();
    {  // a thread's digits: exclusive prefix over the wave-rounds of each, then over the digits of the tile
        uint32_t tot[DPT], mine = 0;
#pragma unroll
        for (int j = 0; j < DPT; j++) {
            const int d = threadIdx.x * DPT + j;
            uint16_t c[Q];
#pragma unroll
            for (int q = 0; q < Q; q++) c[q] = table[q][d];  // all reads first: one LDS round trip, not Q
            uint32_t run = 0;
#pragma unroll
            for (int q = 0; q < Q; q++) {
                table[q][d] = (uint16_t)run;
                run += c[q];
            }
            tot[j] = run;
            mine += run;
        }
        uint32_t inc = mine;
#pragma unroll
        for (int s = 1; s < 64; s <<= 1) {
            const uint32_t v = __shfl_up(inc, s, 64);
            if (lane >= s) inc += v;
        }
        if (lane == 63) wave_tot[wave] = inc;
        __syncthreads();
        uint32_t start = inc - mine;
        for (int w = 0; w < wave; w++) start += wave_tot[w];
#pragma unroll
        for (int j = 0; j < DPT; j++) {
            tile_start[threadIdx.x * DPT + j] = start;
            start += tot[j];
        }
    }
    __syncthreads();
    uint32_t place[kRxPerThread];
#pragma unroll
    for (int r = 0; r < kRxPerThread; r++) {
        const uint32_t digit = (key[r] >> shift) & (kRxBins - 1);
        place[r] = tile_start[digit] + table[r * (kRxThreads / 64) + wave][digit] + rank[r];
    }
    __syncthreads();  // the table has been read by everyone: its memory now takes the sorted tile
    uint32_t* skey = lds;
    uint32_t* sval = lds + kRxTile;
#pragma unroll
    for (int r = 0; r < kRxPerThread; r++) {
        const size_t e = base + (size_t)r * kRxThreads + threadIdx.x;
        if (e < n) {
            skey[place[r]] = key[r];
            sval[place[r]] = val[r];
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kRxPerThread; r++) {
        const uint32_t j = (uint32_t)r * kRxThreads + threadIdx.x;
        if (j < in_tile) {
            const uint32_t k = skey[j];
            const uint32_t digit = (k >> shift) & (kRxBins - 1);
            const uint32_t pos = first[digit] + (j - tile_start[digit]);
            keys_out[pos] = k;
            vals_out[pos] = sval[j];
        }
    }
}

// After the last pass.  Thread i <= n looks at sorted keys i - 1 and i (key n counts as nb, key -1 as none): where they
// differ, the buckets (key[i-1], key[i]] start at position i; the lanes of the wave fill such a run of buckets together,
// so an empty stretch of the bucket range costs its length / 64 store rounds at worst.  The first entry of a bucket
// also lists the bucket as long when the entry kLongBucket places further on still has its key.  Thread i < n fetches
// the payload of entry i of the order.
__global__ __launch_bounds__(256) void rx_finish_kernel(const uint32_t* __restrict__ keys_sorted, size_t n, size_t nb,
                                                         const uint32_t* __restrict__ perm,
                                                         const uint32_t* __restrict__ peer0, uint32_t* __restrict__ peer,
                                                         uint32_t* __restrict__ row_ptr, uint32_t* long_list,
                                                         const uint32_t* gate) {
    if (gate && *gate == 0) return;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int lane = threadIdx.x & 63;
    if (peer0 && i < n) peer[i] = peer0[perm[i]];
    long long prev = 0, cur = -1;  // prev >= cur: nothing starts here
    if (i <= n) {
        cur = (i < n) ? (long long)keys_sorted[i] : (long long)nb;
        prev = (i > 0) ? (long long)keys_sorted[i - 1] : -1;
        if (cur > (long long)nb) cur = (long long)nb;
        if (cur > prev && cur < (long long)nb && i + kLongBucket < n && keys_sorted[i + kLongBucket] == (uint32_t)cur)
            long_list[1 + atomicAdd(&long_list[0], 1u)] = (uint32_t)cur;
    }
    unsigned long long todo = __ballot(cur > prev);
    while (todo) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const long long lo = __shfl(prev, src, 64) + 1, hi = __shfl(cur, src, 64);
        const uint32_t pos = (uint32_t)__shfl((unsigned)i, src, 64);
        for (long long b = lo + lane; b <= hi; b += 64) row_ptr[b] = pos;
    }
}

// `gate` null: the plan is built.  Otherwise gate[0..1] are the two words and gate[2..3] the tally of RxGate, tally_host
// its mirror: the plan (built before from arrays whose 32-bit copies it still holds) is rebuilt if the arrays differ.
static int build_plan_radix(zg_hip_ctx* ctx, const uint64_t* keys, const Plan& pl, const uint64_t* payload,
                            uint32_t* gate = nullptr, uint32_t* tally_host = nullptr) {
    hipStream_t st = ctx->stream;
    const size_t n = pl.n, nb = pl.nb;
    const unsigned n_tiles = (unsigned)ceil_div_sz(n, kRxTile);
    int bits = 1;
    while (((size_t)1 << bits) <= nb) bits++;  // values 0 .. nb (nb itself marks a key outside the buckets)
    const bool nine = (bits + 8) / 9 < (bits + 7) / 8;  // 9-bit digits where they save a pass
    const int digit = nine ? 9 : 8, passes = (bits + digit - 1) / digit;
    // the last pass must land in pl.perm: the positions alternate between perm_tmp and perm
    uint32_t* vals[2] = {(passes & 1) ? pl.perm_tmp : pl.perm, (passes & 1) ? pl.perm : pl.perm_tmp};
    // keys: pass 0 reads rx_in0 and writes rx_keys[1], pass 1 writes rx_keys[0], ...
    const uint32_t* later = gate ? gate + 1 : nullptr;
#define ZG_RX(KERNEL, GRID, BLOCK, ...)                                                                \
    do {                                                                                               \
        if (nine) hipLaunchKernelGGL((KERNEL<9>), GRID, BLOCK, 0, st, __VA_ARGS__);                    \
        else hipLaunchKernelGGL((KERNEL<8>), GRID, BLOCK, 0, st, __VA_ARGS__);                         \
        ZG_LAUNCH_CHECK();                                                                             \
    } while (0)
    ZG_RX(rx_count_first_kernel, dim3(n_tiles), dim3(kRxThreads), keys, payload, n, (uint32_t)nb, pl.rx_in0, pl.rx_peer0,
          pl.rx_counts, gate);
    for (int p = 0; p < passes; p++) {
        const uint32_t* kin = p == 0 ? pl.rx_in0 : pl.rx_keys[p & 1];
        uint32_t* kout = pl.rx_keys[(p & 1) ^ 1];
        if (p > 0) {
            ZG_RX(rx_count_kernel, dim3(n_tiles), dim3(kRxThreads), kin, n, p * digit, pl.rx_counts, later);
        }
        RxGate g;
        if (gate) {
            g.in = p == 0 ? gate : later;
            if (p == 0) {
                g.move_to = gate + 1;
                g.tally = gate + 2;
                g.tally_host = tally_host;
            }
        }
        ZG_RX(rx_scan_kernel, dim3(nine ? 2 : 1), dim3(kRxScanThreads), pl.rx_counts, (size_t)n_tiles, g,
              p == 0 ? pl.long_list : (uint32_t*)nullptr, (uint32_t)n);
        // pass 0 reads no positions (an entry's position is its index); pass p writes vals[(p + 1) & 1]... in turn
        ZG_RX(rx_scatter_kernel, dim3(n_tiles), dim3(kRxThreads), kin, p == 0 ? (const uint32_t*)nullptr : vals[p & 1], n,
              p * digit, pl.rx_counts, kout, vals[(p & 1) ^ 1], later, (gate && p == 0) ? gate : (uint32_t*)nullptr);
    }
#undef ZG_RX
    hipLaunchKernelGGL(rx_finish_kernel, dim3((unsigned)ceil_div_sz(n + 1, 256)), dim3(256), 0, st, pl.rx_keys[passes & 1], n,
                       nb, pl.perm, payload ? pl.rx_peer0 : (const uint32_t*)nullptr, pl.peer, pl.row_ptr, pl.long_list, later);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

static int build_plan(zg_hip_ctx* ctx, const uint64_t* keys, const Plan& pl, const uint64_t* payload = nullptr) {
    if (pl.rx_keys[0]) return build_plan_radix(ctx, keys, pl, payload);
    hipStream_t st = ctx->stream;
    const size_t n = pl.n, nb = pl.nb;
    const int g_n = (int)(ceil_div_sz(n ? n : 1, 256) > 4096 ? 4096 : ceil_div_sz(n ? n : 1, 256));
    const int g_b = (int)(ceil_div_sz(nb + 1, 256) > 4096 ? 4096 : ceil_div_sz(nb + 1, 256));
    // the last word of long_list is spare (at most n / (kLongBucket + 1) buckets are long): the sparse build's second count
    uint32_t* mid_count = pl.long_list + n / kLongBucket + 1;
    hipLaunchKernelGGL(zero_u32_kernel, dim3(g_b), dim3(256), 0, st, pl.row_ptr, nb + 1, pl.cursor, nb, pl.long_list, mid_count);
    ZG_LAUNCH_CHECK();
    if (n) {
        hipLaunchKernelGGL(histogram_kernel, dim3(g_n), dim3(256), 0, st, keys, n, nb, pl.row_ptr);
        ZG_LAUNCH_CHECK();
    }
    const size_t tiles = ceil_div_sz(nb + 1, kScanTile);
    if (tiles <= 8) {
        hipLaunchKernelGGL(scan_single_kernel, dim3(1), dim3(256), 0, st, pl.row_ptr, nb + 1);
        ZG_LAUNCH_CHECK();
    } else {
        hipLaunchKernelGGL(scan_tiles_kernel, dim3((unsigned)tiles), dim3(256), 0, st, pl.row_ptr, nb + 1, pl.tile_sums);
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(scan_single_kernel, dim3(1), dim3(256), 0, st, pl.tile_sums, tiles);  // 2048 sums a round
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(scan_add_kernel, dim3((unsigned)tiles), dim3(256), 0, st, pl.row_ptr, nb + 1, pl.tile_sums);
        ZG_LAUNCH_CHECK();
    }
    if (n) {
        hipLaunchKernelGGL(place_kernel, dim3(g_n), dim3(256), 0, st, keys, n, nb, pl.row_ptr, pl.cursor, pl.perm_tmp, payload,
                           pl.peer_tmp);
        ZG_LAUNCH_CHECK();
        const uint32_t* peer_tmp = payload ? pl.peer_tmp : (const uint32_t*)nullptr;
        if (nb / 4 >= n) {
            // the cursors are done with once the entries are placed: their array holds the list of mid-length buckets
            // (at most n / (kSparseSerial + 1) of them, and nb >= 4 n)
            hipLaunchKernelGGL(order_sparse_kernel, dim3((unsigned)ceil_div_sz(nb, 256)), dim3(256), 0, st, pl.row_ptr, nb,
                               pl.perm_tmp, pl.perm, peer_tmp, pl.peer, pl.long_list, mid_count, pl.cursor);
            ZG_LAUNCH_CHECK();
            if (n > kSparseSerial) {
                hipLaunchKernelGGL(order_segments_kernel, dim3((unsigned)ceil_div_sz(n / (kSparseSerial + 1) + 1, 4)), dim3(256),
                                   0, st, pl.row_ptr, nb, pl.perm_tmp, pl.perm, peer_tmp, pl.peer, pl.long_list, pl.cursor,
                                   mid_count);
                ZG_LAUNCH_CHECK();
            }
        } else {
            hipLaunchKernelGGL(order_segments_kernel, dim3((unsigned)ceil_div_sz(nb, 4)), dim3(256), 0, st, pl.row_ptr, nb,
                               pl.perm_tmp, pl.perm, peer_tmp, pl.peer, pl.long_list);
            ZG_LAUNCH_CHECK();
        }
        if (n > kRankMax) {  // only then can a bucket be too long to rank; the workgroups exit at once when none is
            size_t grid = n / kRankMax;
            if (grid > 1024) grid = 1024;
            hipLaunchKernelGGL(order_long_segments_kernel, dim3((unsigned)grid), dim3(kOrderLongThreads), 0, st, keys, n,
                               pl.row_ptr, pl.long_list, pl.perm, payload, pl.peer);
            ZG_LAUNCH_CHECK();
        }
    }
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Plan cache.  The reference's callers keep their index arrays (edge lists, gather offsets) in memory the host
// writes, here pinned host memory from zg_hip_host_alloc, and pass the same arrays call after call: a graph
// convolution step builds eight plans of the same two arrays.  A context therefore keeps the plans it built for
// such arrays, together with a host copy of what the arrays held and a device copy for the kernels, and a later
// call whose arrays hold the same values (compared on the host, byte for byte, at the time of the call) launches
// its apply kernels on the kept plan.  Same plan, same kernels, same results; what is saved is five to six launches
// per plan and the kernels' reads of the indices across the bus.  Arrays in device memory cannot be compared without
// waiting for the GPU and take the uncached path.  A hit while an execution graph is being recorded is noted in the
// context so that the saved graph keeps the plan alive and zg_hip_graph_run can refuse a replay after the caller
// has rewritten the arrays.
// ------------------------------------------------------------------------------------------------
constexpr size_t kPlanCacheMax = 16;
// The host comparison costs about 50 us per MB; the five to six launches it saves take 20 to 30 us of GPU time and
// about as much host time, so arrays of more than 64 Ki entries (512 KiB) are analysed on the GPU every call.
constexpr size_t kPlanCacheMaxEntries = (size_t)1 << 16;

struct CachedPlan {
    std::vector<uint64_t> keys_host, payload_host;  // what the arrays held when the plan was built
    void* mem = nullptr;                             // one device allocation: the plan, then the device copies
    Plan plan;
    uint64_t* keys_dev = nullptr;
    uint64_t* payload_dev = nullptr;  // null: built without payload
    // scatter_gcn_deg_scaled_bwd on an entry with a payload (keys = sources, payload = targets): the incidence plan
    // of the degree gradient, built by the first such call outside a recording
    void* inc_mem = nullptr;
    Plan inc;
    uint32_t* slot_of = nullptr;  // 2 n
    uint64_t last_use = 0;
    int graph_refs = 0;
    // A plan validated on the GPU (see plan_validated): found by the addresses of its arrays, not by their contents
    bool validated = false;
    const void* key_ptr = nullptr;
    const void* payload_ptr = nullptr;
    size_t n = 0, nb = 0, bytes = 0;
    uint32_t* gate = nullptr;        // device: two gate words, two tally words (RxGate)
    uint32_t* tally_host = nullptr;  // pinned host: builds skipped, builds done
    uint32_t seen[2] = {0, 0};       // the tally when the host last judged it
    uint32_t retry_in = 0;           // non-zero: given up on (the arrays change from call to call); calls left before a new try
};

struct PlanCache {
    std::vector<CachedPlan*> entries;
    uint64_t clock = 0;
    uint64_t hits = 0, builds = 0;
};

static bool in_pinned_host(zg_hip_ctx* ctx, const void* p, size_t bytes) {
    auto it = ctx->host_allocs.upper_bound(const_cast<void*>(p));
    if (it == ctx->host_allocs.begin()) return false;
    --it;
    const char* lo = (const char*)it->first;
    return (const char*)p >= lo && (const char*)p + bytes <= lo + it->second;
}

// What an op launches its apply kernels on: a plan and device-readable copies of the arrays it was built from.
struct PlanRef {
    Plan plan;
    const uint64_t* keys;
    const uint64_t* payload;
    CachedPlan* entry = nullptr;  // null: built in the workspace by the caller
};

// True when `out` names a cached plan for these arrays (found, or built and kept by this call).  False: the caller
// builds the plan in the workspace as before (*rc says whether that is because of an error).
static void plan_entry_release(zg_hip_ctx* ctx, CachedPlan* e) {
    if (e->mem) zg_hip_free(ctx, e->mem);
    if (e->inc_mem) zg_hip_free(ctx, e->inc_mem);
    if (e->tally_host) zg_hip_host_free(ctx, e->tally_host);
    e->mem = e->inc_mem = nullptr;
    e->tally_host = nullptr;
}

// Long arrays (the radix build's range), in device memory or in pinned host memory: the plan is kept under the
// ADDRESSES of its arrays, with 32-bit copies of what they held, and every call runs the first kernel of the build,
// which compares the arrays with the copies on the GPU; the nine to twelve launches that follow return at once when
// nothing has changed and rebuild the plan in place when something has.  The result is the plan of the arrays as they
// are now either way, whoever wrote them and however (the host never looks at their contents, so nothing waits for
// the GPU, and a recorded step stays valid when the arrays are rewritten).  One million entries: about 25 us instead
// of 100.  An entry whose arrays turn out to change on most calls is given up (the host reads the tally the scan kernel
// mirrors into pinned memory, without waiting for it) and the address is left alone for the next kValidatedRetry calls.
constexpr size_t kValidatedMaxEntries = (size_t)1 << 24;
constexpr size_t kValidatedMaxBytes = (size_t)4 << 30;
constexpr uint32_t kValidatedRetry = 1024;

static bool plan_validated(zg_hip_ctx* ctx, const uint64_t* keys, const uint64_t* payload, size_t n, size_t nb, PlanRef* out,
                           int* rc) {
    if (!ctx->plan_cache) ctx->plan_cache = new PlanCache();
    PlanCache& pc = *ctx->plan_cache;
    CachedPlan* hit = nullptr;
    size_t at = 0, held = 0;
    for (size_t i = 0; i < pc.entries.size(); i++) {
        CachedPlan* e = pc.entries[i];
        if (!e->validated) continue;
        held += e->bytes;
        if (e->key_ptr == keys && e->payload_ptr == payload && e->n == n && e->nb == nb) {
            hit = e;
            at = i;
        }
    }
    if (hit && hit->retry_in) {
        if (--hit->retry_in == 0) {
            delete hit;
            pc.entries.erase(pc.entries.begin() + at);
        }
        return false;
    }
    if (hit && !ctx->capturing && hit->graph_refs == 0) {
        const volatile uint32_t* tally = hit->tally_host;
        const uint32_t skipped = tally[0] - hit->seen[0], rebuilt = tally[1] - hit->seen[1];  // since the last look
        if (!(rebuilt >= 8 && rebuilt > skipped) && skipped + rebuilt >= 16) {
            hit->seen[0] += skipped;
            hit->seen[1] += rebuilt;
        } else if (rebuilt >= 8 && rebuilt > skipped) {  // these arrays are new on most calls: comparing them is wasted work
            if (hipStreamSynchronize(ctx->stream) != hipSuccess) return false;  // queued kernels may read the entry
            plan_entry_release(ctx, hit);
            hit->retry_in = kValidatedRetry;
            hit->bytes = 0;
            return false;
        }
    }
    if (hit) {
        // work that waits may name this plan's memory (an aggregation, a count): it leaves before the plan can change
        if ((*rc = flush_kinds(ctx, kWaitScatter | kWaitGradDeg | kWaitMaps))) return false;
        if ((*rc = build_plan_radix(ctx, keys, hit->plan, payload, hit->gate, hit->tally_host))) return false;
        pc.hits++;
    } else {
        if (ctx->capturing) return false;  // building one allocates; the recording builds its plan in the workspace
        const size_t pb = align_up(plan_bytes(n, nb), 256), sb = align_up(n * sizeof(uint32_t), 256);
        const size_t bytes = pb + sb + 256;
        while (pc.entries.size() >= kPlanCacheMax || held + bytes > kValidatedMaxBytes) {
            size_t victim = pc.entries.size();
            for (size_t i = 0; i < pc.entries.size(); i++) {
                const CachedPlan* e = pc.entries[i];
                if (e->graph_refs != 0 || (pc.entries.size() < kPlanCacheMax && !(e->validated && e->bytes))) continue;
                if (victim == pc.entries.size() || e->last_use < pc.entries[victim]->last_use) victim = i;
            }
            if (victim == pc.entries.size()) return false;
            if (hipStreamSynchronize(ctx->stream) != hipSuccess) return false;  // queued kernels may read the victim
            CachedPlan* v = pc.entries[victim];
            if (v->validated) held -= v->bytes;
            plan_entry_release(ctx, v);
            delete v;
            pc.entries.erase(pc.entries.begin() + victim);
        }
        void* mem = nullptr;
        void* tally = nullptr;
        if ((*rc = zg_hip_alloc(ctx, bytes, &mem))) return false;
        if ((*rc = zg_hip_host_alloc(ctx, 256, &tally))) {
            zg_hip_free(ctx, mem);
            return false;
        }
        CachedPlan* e = new CachedPlan();
        e->validated = true;
        e->key_ptr = keys;
        e->payload_ptr = payload;
        e->n = n;
        e->nb = nb;
        e->bytes = bytes;
        e->mem = mem;
        e->plan = carve_plan(mem, n, nb);
        e->plan.rx_in0 = (uint32_t*)((char*)mem + pb);
        e->gate = (uint32_t*)((char*)mem + pb + sb);
        e->tally_host = (uint32_t*)tally;
        e->tally_host[0] = e->tally_host[1] = 0;
        hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(64), 0, ctx->stream, e->gate, (size_t)4, (uint32_t*)nullptr, (size_t)0,
                           (uint32_t*)nullptr);
        *rc = hipGetLastError() == hipSuccess ? ZG_HIP_OK : ZG_HIP_ERUNTIME;
        if (!*rc) *rc = build_plan_radix(ctx, keys, e->plan, payload);  // unconditional, and it takes the copies
        if (*rc) {
            (void)hipStreamSynchronize(ctx->stream);
            plan_entry_release(ctx, e);
            delete e;
            return false;
        }
        pc.entries.push_back(e);
        pc.builds++;
        hit = e;
    }
    hit->last_use = ++pc.clock;
    if (ctx->capturing) ctx->plan_uses.push_back(PlanUse{hit, keys, payload});
    out->plan = hit->plan;
    out->keys = keys;
    out->payload = payload;
    out->entry = hit;
    return true;
}

static bool plan_from_cache(zg_hip_ctx* ctx, const uint64_t* keys, const uint64_t* payload, size_t n, size_t nb,
                            PlanRef* out, int* rc) {
    *rc = ZG_HIP_OK;
    if (n == 0) return false;
    if (radix_build_applies(n, nb) && n >= kRadixMinEntries && n <= kValidatedMaxEntries)
        return plan_validated(ctx, keys, payload, n, nb, out, rc);
    if (n > kPlanCacheMaxEntries) return false;
    const size_t bytes = n * sizeof(uint64_t);
    if (!in_pinned_host(ctx, keys, bytes) || (payload && !in_pinned_host(ctx, payload, bytes))) return false;
    if (!ctx->plan_cache) ctx->plan_cache = new PlanCache();
    PlanCache& pc = *ctx->plan_cache;
    CachedPlan* hit = nullptr;
    for (CachedPlan* e : pc.entries) {
        if (e->validated || e->plan.n != n || e->plan.nb != nb) continue;
        if (payload && !e->payload_dev) continue;  // an entry with a payload also serves a call without one
        if (memcmp(e->keys_host.data(), keys, bytes) != 0) continue;
        if (payload && memcmp(e->payload_host.data(), payload, bytes) != 0) continue;
        hit = e;
        break;
    }
    if (!hit) {
        if (ctx->capturing) return false;  // building one allocates; the recording builds its plan in the workspace
        if (pc.entries.size() >= kPlanCacheMax) {
            size_t victim = pc.entries.size();
            for (size_t i = 0; i < pc.entries.size(); i++)
                if (pc.entries[i]->graph_refs == 0 &&
                    (victim == pc.entries.size() || pc.entries[i]->last_use < pc.entries[victim]->last_use))
                    victim = i;
            if (victim == pc.entries.size()) return false;  // every entry is named by a saved graph
            if (hipStreamSynchronize(ctx->stream) != hipSuccess) return false;  // queued kernels may read the victim
            CachedPlan* v = pc.entries[victim];
            plan_entry_release(ctx, v);
            delete v;
            pc.entries.erase(pc.entries.begin() + victim);
        }
        const size_t pb = align_up(plan_bytes(n, nb), 256), ib = align_up(bytes, 256);
        void* mem = nullptr;
        if ((*rc = zg_hip_alloc(ctx, pb + (payload ? 2 : 1) * ib, &mem))) return false;
        CachedPlan* e = new CachedPlan();
        e->mem = mem;
        e->plan = carve_plan(mem, n, nb);
        e->keys_dev = (uint64_t*)((char*)mem + pb);
        e->keys_host.assign(keys, keys + n);
        // the device copies are taken from the host snapshots' source at the same moment; both are pinned memory
        *rc = zg_hip_memcpy_d2d(ctx, e->keys_dev, keys, bytes);
        if (!*rc && payload) {
            e->payload_dev = (uint64_t*)((char*)mem + pb + ib);
            e->payload_host.assign(payload, payload + n);
            *rc = zg_hip_memcpy_d2d(ctx, e->payload_dev, payload, bytes);
        }
        if (!*rc) *rc = build_plan(ctx, e->keys_dev, e->plan, e->payload_dev);
        if (!*rc) {
            // how many long buckets there are is read back once, so that later calls skip the long-bucket kernel's
            // launch when there is none (the usual case: a graph's edge list)
            uint32_t n_long = 0;
            if (hipMemcpyAsync(&n_long, e->plan.long_list, sizeof(n_long), hipMemcpyDeviceToHost, ctx->stream) == hipSuccess &&
                hipStreamSynchronize(ctx->stream) == hipSuccess)
                e->plan.n_long = (long)n_long;
        }
        if (*rc) {
            (void)hipStreamSynchronize(ctx->stream);
            zg_hip_free(ctx, mem);
            delete e;
            return false;
        }
        pc.entries.push_back(e);
        pc.builds++;
        hit = e;
    } else {
        pc.hits++;
    }
    hit->last_use = ++pc.clock;
    if (ctx->capturing) ctx->plan_uses.push_back(PlanUse{hit, keys, payload});
    out->plan = hit->plan;
    out->keys = hit->keys_dev;
    out->payload = hit->payload_dev;
    out->entry = hit;
    return true;
}

__global__ void interleave_keys_kernel(const uint64_t* src_idx, const uint64_t* tgt_idx, size_t n_edge, uint64_t* keys,
                                       uint32_t* slot_of);
__global__ void invert_perm_kernel(const uint32_t* row_ptr, size_t nb, const uint32_t* perm, uint32_t* slot_of);

// The incidence plan of an entry whose keys are edge sources and whose payload is edge targets; false when it does
// not exist and cannot be built now (recording, or an error: *rc).
static bool incidence_plan(zg_hip_ctx* ctx, CachedPlan* e, int* rc) {
    *rc = ZG_HIP_OK;
    if (e->inc_mem) return true;
    if (ctx->capturing || !e->payload_dev) return false;
    const size_t n2 = 2 * e->plan.n, nb = e->plan.nb;
    if (n2 >= 0xffffffffull) return false;
    const size_t pb = align_up(plan_bytes(n2, nb), 256), kb = align_up(n2 * sizeof(uint64_t), 256);
    void* mem = nullptr;
    if ((*rc = zg_hip_alloc(ctx, pb + kb + align_up(n2 * sizeof(uint32_t), 256), &mem))) return false;
    Plan inc = carve_plan(mem, n2, nb);
    uint64_t* keys = (uint64_t*)((char*)mem + pb);
    uint32_t* slot_of = (uint32_t*)((char*)mem + pb + kb);
    hipLaunchKernelGGL(interleave_keys_kernel, dim3((unsigned)ceil_div_sz(e->plan.n, 256)), dim3(256), 0, ctx->stream,
                       e->keys_dev, e->payload_dev, e->plan.n, keys, slot_of);
    *rc = build_plan(ctx, keys, inc);
    if (!*rc) {
        hipLaunchKernelGGL(invert_perm_kernel, dim3((unsigned)ceil_div_sz(n2, 256)), dim3(256), 0, ctx->stream, inc.row_ptr,
                           nb, inc.perm, slot_of);
        if (hipGetLastError() != hipSuccess) *rc = ZG_HIP_ERUNTIME;
    }
    if (*rc) {
        (void)hipStreamSynchronize(ctx->stream);
        zg_hip_free(ctx, mem);
        return false;
    }
    e->inc_mem = mem;
    e->inc = inc;
    e->slot_of = slot_of;
    return true;
}

void plan_cache_destroy(zg_hip_ctx* ctx) {
    if (!ctx->plan_cache) return;
    for (CachedPlan* e : ctx->plan_cache->entries) {
        plan_entry_release(ctx, e);
        delete e;
    }
    delete ctx->plan_cache;
    ctx->plan_cache = nullptr;
}

void plan_uses_retain(const std::vector<PlanUse>& uses, int delta) {
    for (const PlanUse& u : uses) u.entry->graph_refs += delta;
}

int plan_uses_validate(zg_hip_ctx* ctx, const std::vector<PlanUse>& uses) {
    // an array that compared equal to one snapshot equals every snapshot the recording matched it against
    const void* seen[2 * kPlanCacheMax];
    size_t n_seen = 0;
    auto check = [&](const uint64_t* p, const std::vector<uint64_t>& snap) -> int {
        for (size_t i = 0; i < n_seen; i++)
            if (seen[i] == p) return ZG_HIP_OK;
        const size_t bytes = snap.size() * sizeof(uint64_t);
        ZG_REQUIRE(in_pinned_host(ctx, p, bytes),
                   "graph_run: an index array named by the recording is no longer a zg_hip_host_alloc allocation");
        ZG_REQUIRE(memcmp(p, snap.data(), bytes) == 0,
                   "graph_run: an index array was rewritten after the step was recorded; the recorded kernels would "
                   "scatter by its old contents (record the step again)");
        if (n_seen < 2 * kPlanCacheMax) seen[n_seen++] = p;
        return ZG_HIP_OK;
    };
    for (const PlanUse& u : uses) {
        if (u.entry->validated) continue;  // the recorded kernels compare the arrays themselves
        if (int rc = check(u.keys, u.entry->keys_host)) return rc;
        if (u.payload)
            if (int rc = check(u.payload, u.entry->payload_host)) return rc;
    }
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// apply kernels
// ------------------------------------------------------------------------------------------------

// dst[b] += src[e] for the bucket's entries in input order; one thread per destination
// `fresh`: dst is write-only (treated as zero on entry), so the caller needs no zero fill
// src null: every contribution is `src_const` (a source whose fill with one value is still waiting is not read)
__global__ void scatter_add_apply_kernel(const float* src, const uint32_t* row_ptr, const uint32_t* perm, float* dst,
                                         size_t nb, bool fresh, float src_const) {
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nb) return;
    const uint32_t s = row_ptr[b], e = row_ptr[b + 1];
    if (s == e) {
        if (fresh) dst[b] = 0.f;
        return;
    }
    if (e - s > kLongBucket) return;  // long_bucket_kernel's
    float acc = fresh ? 0.f : dst[b];
    // eight entries' loads at a time (positions, then values: two round trips), the additions still in input order
    for (uint32_t k = s; k < e; k += 8) {
        uint32_t pv[8];
        float sv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) pv[u] = (k + u < e) ? perm[k + u] : 0u;
#pragma unroll
        for (int u = 0; u < 8; u++) sv[u] = (k + u < e) ? (src ? src[pv[u]] : src_const) : 0.f;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (k + u < e) acc = __fadd_rn(acc, sv[u]);
    }
    dst[b] = acc;
}

// The long buckets: one wave per destination element (a destination row of `stride` elements: a wave per column).  The
// wave loads 64 contributions at a time (the loads do not depend on the running sum, and the next 64 are in flight
// meanwhile), then adds them one after the other in input order, every lane forming the same sum.  The 64 values go
// through LDS: every lane reads them back four at a time (all lanes the same address, a broadcast), so that the chain of
// additions is all that is serial (a shuffle per value costs 45 ns an entry, a scalar lane read 12 ns, this 10 ns).  LDS
// serves a wave's accesses in order, and the two halves of `vals` alternate, so the wave needs no barrier with itself.
// F::value(k, b, col, stride, ok) is entry k's contribution to column col of destination b; ok false: the entry is
// skipped (an edge whose other endpoint is no node).  Optional tail of a graph-convolution layer as in
// gcn_fwd_apply_kernel: + bias[col], then max(., 0).
struct LongScatterAdd {
    const float* src;  // null: every contribution is src_const
    const uint32_t* perm;
    float src_const;
    __device__ __forceinline__ float value(uint32_t k, uint32_t, size_t col, size_t stride, bool& ok) const {
        ok = true;
        return src ? src[(size_t)perm[k] * stride + col] : src_const;
    }
};
struct LongGcnFwd {  // (deg[s] * deg[t]) * h[s, col] over the edges into t = b
    const float* h;
    const float* deg;
    const uint32_t* peer;
    size_t n_nodes;
    __device__ __forceinline__ float value(uint32_t k, uint32_t b, size_t col, size_t stride, bool& ok) const {
        const uint32_t sv = peer[k];
        ok = sv < n_nodes;
        return ok ? __fmul_rn(__fmul_rn(deg[sv], deg[b]), h[(size_t)sv * stride + col]) : 0.f;
    }
};
struct LongTerms {  // the degree-gradient terms of a node, laid out in the order they are added
    const float* terms;
    __device__ __forceinline__ float value(uint32_t k, uint32_t, size_t, size_t, bool& ok) const {
        ok = true;
        return terms[k];
    }
};
struct LongGcnGradH {  // (go[t, col] * deg[s]) * deg[t] over the edges out of s = b
    const float* go;
    const float* deg;
    const uint32_t* peer;
    size_t n_nodes;
    __device__ __forceinline__ float value(uint32_t k, uint32_t b, size_t col, size_t stride, bool& ok) const {
        const uint32_t tv = peer[k];
        ok = tv < n_nodes;
        return ok ? __fmul_rn(__fmul_rn(go[(size_t)tv * stride + col], deg[b]), deg[tv]) : 0.f;
    }
};
template <class F>
__global__ __launch_bounds__(256) void long_bucket_kernel(F f, const uint32_t* row_ptr, const uint32_t* long_list, float* dst,
                                                           bool fresh, size_t stride, const float* bias, bool relu) {
    __shared__ __align__(16) float vals[4][2][64];
    const int lane = threadIdx.x & 63;
    const size_t n_jobs = (size_t)long_list[0] * stride;
    const size_t wave0 = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = (size_t)gridDim.x * 4;
    for (size_t w = wave0; w < n_jobs; w += n_waves) {
        const uint32_t b = long_list[1 + w / stride];
        const size_t col = w % stride;
        const uint32_t s = row_ptr[b], e = row_ptr[b + 1];
        float* out = dst + (size_t)b * stride + col;
        float acc = fresh ? 0.f : out[0];
        auto fetch = [&](uint32_t k, bool& ok) {
            ok = false;
            return (k < e) ? f.value(k, b, col, stride, ok) : 0.f;
        };
        bool ok;
        float v = fetch(s + lane, ok);
        for (uint32_t k0 = s; k0 < e; k0 += 64) {
            bool ok_next;
            const float v_next = fetch(k0 + 64 + lane, ok_next);
            const unsigned long long mask = __ballot(ok);
            float* slot = vals[threadIdx.x >> 6][(k0 - s) / 64 & 1];
            slot[lane] = v;
            __builtin_amdgcn_wave_barrier();
            if (mask == ~0ull) {
#pragma unroll
                for (int j = 0; j < 64; j += 4) {
                    const float4 q = *reinterpret_cast<const float4*>(slot + j);
                    acc = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(acc, q.x), q.y), q.z), q.w);
                }
            } else {
                for (int j = 0; j < 64; j++)
                    if ((mask >> j) & 1ull) acc = __fadd_rn(acc, slot[j]);
            }
            v = v_next;
            ok = ok_next;
        }
        if (bias) acc = __fadd_rn(acc, bias[col]);
        if (relu) acc = acc > 0.f ? acc : 0.f;
        if (lane == 0) out[0] = acc;
    }
}

// Launches long_bucket_kernel over the long buckets of `pl` (n_long: the host's count of them, -1 unknown).
template <class F>
static int launch_long_buckets(zg_hip_ctx* ctx, const F& f, const uint32_t* row_ptr, const uint32_t* long_list, size_t n_entries,
                               long n_long, float* dst, bool fresh, size_t stride, const float* bias = nullptr,
                               bool relu = false) {
    if (n_entries <= kLongBucket || n_long == 0) return ZG_HIP_OK;
    size_t grid = ceil_div_sz((n_entries / kLongBucket) * stride, 4);
    if (grid > 2048) grid = 2048;
    hipLaunchKernelGGL((long_bucket_kernel<F>), dim3((unsigned)grid), dim3(256), 0, ctx->stream, f, row_ptr, long_list, dst,
                       fresh, stride, bias, relu);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

static int launch_scatter_add_apply(zg_hip_ctx* ctx, const float* src, const Plan& pl, float* dst, bool fresh,
                                    float src_const = 0.f) {
    hipLaunchKernelGGL(scatter_add_apply_kernel, dim3((unsigned)ceil_div_sz(pl.nb, 256)), dim3(256), 0, ctx->stream, src,
                       pl.row_ptr, pl.perm, dst, pl.nb, fresh, src_const);
    ZG_LAUNCH_CHECK();
    return launch_long_buckets(ctx, LongScatterAdd{src, pl.perm, src_const}, pl.row_ptr, pl.long_list, pl.n, pl.n_long, dst, fresh, 1);
}

// The whole of scatter_add for at most kScatterSmallMax entries in one launch of one workgroup: thread i owns entry i,
// and the first entry of each destination walks the later entries in input order, so the additions happen in the
// order of the host loop.  Offsets at or beyond `nb` are skipped, as the bucket path skips them.
// With `fresh` the destination's zero fill was taken over: the workgroup zeroes all of dst first and the sums start
// from +0.0 instead of what dst held (at most kScatterSmallFreshMax destinations).
constexpr int kScatterSmallMax = 256;
constexpr size_t kScatterSmallFreshMax = 16384;
__global__ __launch_bounds__(kScatterSmallMax) void scatter_add_small_kernel(const float* src, const uint64_t* offsets,
                                                                             int n, float* dst, size_t nb, bool fresh,
                                                                             float src_const) {
    __shared__ uint64_t s_off[kScatterSmallMax];
    __shared__ float s_src[kScatterSmallMax];
    const int i = threadIdx.x;
    // slots past n hold an offset no destination has, so the walk below can run in whole groups of eight
    s_off[i] = (i < n) ? offsets[i] : ~0ull;
    s_src[i] = (i < n) ? (src ? src[i] : src_const) : 0.f;  // src null: every contribution is src_const
    if (fresh)
        for (size_t e = i; e < nb; e += kScatterSmallMax) dst[e] = 0.f;
    __syncthreads();  // also orders the zeros before the sums stored below (one workgroup, global memory)
    if (i >= n) return;
    const uint64_t k = s_off[i];
    if (k >= nb) return;
    float acc = fresh ? 0.f : dst[k];
    bool first = true;
    const int n8 = (n + 7) & ~7;
    for (int j0 = 0; j0 < n8; j0 += 8) {
        uint64_t o[8];
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {  // eight LDS reads in flight, then the additions in input order
            o[u] = s_off[j0 + u];
            v[u] = s_src[j0 + u];
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const bool same = o[u] == k;
            first = first && !(same && j0 + u < i);
            acc = (same && j0 + u >= i) ? __fadd_rn(acc, v[u]) : acc;
        }
    }
    if (first) dst[k] = acc;
}

// rows of `stride` elements: dst[b, :] = src_row(e) + dst[b, :] in input order.  G threads per destination row.
// MODE 0: index_select backward  (x_grad[row] = y_grad[e] + x_grad[row], src/ndtensor.zig:1461-1465)
template <int G>
__global__ __launch_bounds__(256) void row_scatter_apply_kernel(const float* src, const uint32_t* row_ptr,
                                                                 const uint32_t* perm, float* dst, size_t nb,
                                                                 size_t stride, size_t span) {
    const size_t b = (size_t)blockIdx.x * (256 / G) + threadIdx.x / G;
    if (b >= nb) return;
    const int lane = threadIdx.x % G;
    const uint32_t s = row_ptr[b], e = row_ptr[b + 1];
    if (s == e) return;
    if (e - s > kLongBucket) return;  // long_bucket_kernel's, a wave per column
    // long rows are cut into spans of columns (blockIdx.y): 32 rows of a million values on 32 lane groups took 15 ms
    const size_t j_begin = (size_t)blockIdx.y * span, j_end = j_begin + span < stride ? j_begin + span : stride;
    for (size_t j = j_begin + lane; j < j_end; j += G) {
        float acc = dst[b * stride + j];
        // eight entries' loads at a time (positions, then row elements: two round trips), the additions still in input
        // order (one entry at a time, a destination of ten thousand entries took 440 ns an entry)
        for (uint32_t k = s; k < e; k += 8) {
            uint32_t pv[8];
            float sv[8];
#pragma unroll
            for (int u = 0; u < 8; u++) pv[u] = (k + u < e) ? perm[k + u] : 0u;
#pragma unroll
            for (int u = 0; u < 8; u++) sv[u] = (k + u < e) ? src[(size_t)pv[u] * stride + j] : 0.f;
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (k + u < e) acc = __fadd_rn(sv[u], acc);
        }
        dst[b * stride + j] = acc;
    }
}

// dst[t, :] += (deg[s] * deg[t]) * h[s, :] over the edges into t, in edge order.  `peer` holds the source of each
// edge in that order; four edges are loaded at a time (the loads do not depend on the running sum) and then added
// one after the other.  Optional tail of a graph-convolution layer: + bias[j], then max(., 0) (the IEEE operations of
// the separate add and relu ops).
template <int G>
__global__ __launch_bounds__(256) void gcn_fwd_apply_kernel(float* dst, const float* h, const float* deg,
                                                             const uint32_t* row_ptr, const uint32_t* peer,
                                                             size_t n_nodes, size_t stride, bool fresh,
                                                             const float* bias, bool relu) {
    const size_t t = (size_t)blockIdx.x * (256 / G) + threadIdx.x / G;
    if (t >= n_nodes) return;
    const int lane = threadIdx.x % G;
    const uint32_t s0 = row_ptr[t], s1 = row_ptr[t + 1];
    if (s0 == s1 && !fresh && !bias && !relu) return;
    if (s1 - s0 > kLongBucket) return;  // long_bucket_kernel's, a wave per column
    const float dt = deg[t];
    for (size_t j = lane; j < stride; j += G) {
        float acc = fresh ? 0.f : dst[t * stride + j];
        for (uint32_t k = s0; k < s1; k += 4) {
            uint32_t sv[4];
            float dv[4], hv[4];
#pragma unroll
            for (int u = 0; u < 4; u++) sv[u] = (k + u < s1) ? peer[k + u] : 0xffffffffu;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const bool ok = sv[u] < n_nodes;
                dv[u] = ok ? deg[sv[u]] : 0.f;
                hv[u] = ok ? h[(size_t)sv[u] * stride + j] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (sv[u] < n_nodes) acc = __fadd_rn(acc, __fmul_rn(__fmul_rn(dv[u], dt), hv[u]));
        }
        if (bias) acc = __fadd_rn(acc, bias[j]);
        if (relu) acc = acc > 0.f ? acc : 0.f;
        dst[t * stride + j] = acc;
    }
}

// grad_h[s, :] += (go[t, :] * deg[s]) * deg[t] over the edges out of s, in edge order; `peer` holds the targets
template <int G>
__global__ __launch_bounds__(256) void gcn_bwd_gradh_kernel(float* grad_h, const float* go, const float* deg,
                                                             const uint32_t* row_ptr, const uint32_t* peer,
                                                             size_t n_nodes, size_t stride, bool fresh) {
    const size_t s = (size_t)blockIdx.x * (256 / G) + threadIdx.x / G;
    if (s >= n_nodes) return;
    const int lane = threadIdx.x % G;
    const uint32_t s0 = row_ptr[s], s1 = row_ptr[s + 1];
    if (s0 == s1) {
        if (fresh)
            for (size_t j = lane; j < stride; j += G) grad_h[s * stride + j] = 0.f;
        return;
    }
    if (s1 - s0 > kLongBucket) return;  // long_bucket_kernel's, a wave per column
    const float ds = deg[s];
    for (size_t j = lane; j < stride; j += G) {
        float acc = fresh ? 0.f : grad_h[s * stride + j];
        for (uint32_t k = s0; k < s1; k += 4) {
            uint32_t tv[4];
            float dv[4], gv[4];
#pragma unroll
            for (int u = 0; u < 4; u++) tv[u] = (k + u < s1) ? peer[k + u] : 0xffffffffu;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const bool ok = tv[u] < n_nodes;
                dv[u] = ok ? deg[tv[u]] : 0.f;
                gv[u] = ok ? go[(size_t)tv[u] * stride + j] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (tv[u] < n_nodes) acc = __fadd_rn(acc, __fmul_rn(__fmul_rn(gv[u], ds), dv[u]));
        }
        grad_h[s * stride + j] = acc;
    }
}

// The two degree-gradient terms of an edge, each summed over the feature dimension in index order, for rows of more than
// 16 features: a thread per edge, but the rows reach it through LDS.  A wave copies 32 columns of the two rows of each of
// its 64 edges into LDS with loads that follow the rows (32 lanes on the 128 contiguous bytes of a row, two edges per
// instruction), then every lane walks its own edge's 32 values in order; left to itself a lane reads its rows value by
// value and every load instruction of the wave touches 64 different rows (a million edges of 64 features: 1766 us that
// way, 12 times what the bytes take).  Called by every thread of a workgroup of kEtThreads.
constexpr int kEtThreads = 128, kEtCols = 32;
constexpr size_t kEtStagedMinStride = 16;  // rows of up to 64 bytes are one cache line either way
__device__ __forceinline__ void edge_terms_staged(const float* go, const float* h, const float* deg, uint64_t s, uint64_t t,
                                                  bool valid, size_t stride, float& gs, float& gt) {
    __shared__ float tg[kEtThreads / 64][64][kEtCols + 1], th[kEtThreads / 64][64][kEtCols + 1];
    __shared__ uint32_t ss[kEtThreads / 64][64], ts[kEtThreads / 64][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    ss[w][lane] = valid ? (uint32_t)s : 0xffffffffu;
    ts[w][lane] = valid ? (uint32_t)t : 0xffffffffu;
    const float ds = valid ? deg[s] : 0.f, dt = valid ? deg[t] : 0.f;
    gs = 0.f;
    gt = 0.f;
    const int col = lane & 31;
    for (size_t c0 = 0; c0 < stride; c0 += kEtCols) {
        __syncthreads();  // the node numbers are in place, and the last chunk has been used up
        const size_t c = c0 + col;
#pragma unroll 8
        for (int it = 0; it < 32; it++) {
            const int ed = it * 2 + (lane >> 5);
            const uint32_t se = ss[w][ed], te = ts[w][ed];
            const bool ok = se != 0xffffffffu && c < stride;
            tg[w][ed][col] = ok ? go[(size_t)te * stride + c] : 0.f;
            th[w][ed][col] = ok ? h[(size_t)se * stride + c] : 0.f;
        }
        __syncthreads();
        if (valid) {
            const int lim = stride - c0 < (size_t)kEtCols ? (int)(stride - c0) : kEtCols;
            for (int j = 0; j < lim; j++) {
                const float g = tg[w][lane][j], hv = th[w][lane][j];
                gs = __fadd_rn(gs, __fmul_rn(__fmul_rn(g, dt), hv));
                gt = __fadd_rn(gt, __fmul_rn(__fmul_rn(g, ds), hv));
            }
        }
    }
}

// STAGED: the workgroup is kEtThreads wide and the rows go through LDS (edge_terms_staged)
template <bool STAGED>
__global__ void gcn_bwd_edge_terms_kernel(const float* go, const float* h, const float* deg, const uint64_t* src_idx,
                                          const uint64_t* tgt_idx, size_t n_edge, size_t n_nodes, size_t stride,
                                          float* term_src, float* term_tgt, uint32_t* zero_me) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (zero_me && e == 0) zero_me[0] = 0;  // the counter of a list that a later kernel appends to
    if (STAGED) {
        const bool in = e < n_edge;
        const uint64_t s = in ? src_idx[e] : 0, t = in ? tgt_idx[e] : 0;
        float gs, gt;
        edge_terms_staged(go, h, deg, s, t, in && s < n_nodes && t < n_nodes, stride, gs, gt);
        if (in) {
            term_src[e] = gs;
            term_tgt[e] = gt;
        }
        return;
    }
    if (e >= n_edge) return;
    const uint64_t s = src_idx[e], t = tgt_idx[e];
    float gs = 0.f, gt = 0.f;
    if (s < n_nodes && t < n_nodes) {
        const float ds = deg[s], dt = deg[t];
        for (size_t j = 0; j < stride; j++) {
            const float g = go[t * stride + j], hv = h[s * stride + j];
            gs = __fadd_rn(gs, __fmul_rn(__fmul_rn(g, dt), hv));
            gt = __fadd_rn(gt, __fmul_rn(__fmul_rn(g, ds), hv));
        }
    }
    term_src[e] = gs;
    term_tgt[e] = gt;
}

// grad_deg[v] += terms of the edges touching v, merged in edge order (an edge v->v adds its source term first)
__global__ void gcn_bwd_graddeg_kernel(float* grad_deg, const float* term_src, const float* term_tgt,
                                       const uint32_t* rp_src, const uint32_t* perm_src, const uint32_t* rp_tgt,
                                       const uint32_t* perm_tgt, size_t n_nodes, bool fresh) {
    size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= n_nodes) return;
    uint32_t a = rp_src[v], a1 = rp_src[v + 1], b = rp_tgt[v], b1 = rp_tgt[v + 1];
    if (a == a1 && b == b1) {
        if (fresh) grad_deg[v] = 0.f;
        return;
    }
    float acc = fresh ? 0.f : grad_deg[v];
    while (a < a1 || b < b1) {
        const uint32_t ea = (a < a1) ? perm_src[a] : 0xffffffffu;
        const uint32_t eb = (b < b1) ? perm_tgt[b] : 0xffffffffu;
        if (ea <= eb) {
            acc = __fadd_rn(acc, term_src[ea]);
            a++;
        } else {
            acc = __fadd_rn(acc, term_tgt[eb]);
            b++;
        }
    }
    grad_deg[v] = acc;
}

// The same sums through an incidence plan: the 2 * n_edge endpoint items (item 2e = edge e's source, item 2e + 1 = its
// target) bucketed by node.  Ascending item order inside a bucket is the merged order above and the order of the
// host loop (per edge: the source's term, then the target's).  slot_of[item] is the item's position in bucket order
// (0xffffffff: its node is out of range), so the edge kernel writes each term where the node's thread will read
// it, and that thread reads one contiguous run, eight loads at a time: no chain of dependent index loads.
__global__ void interleave_keys_kernel(const uint64_t* src_idx, const uint64_t* tgt_idx, size_t n_edge, uint64_t* keys,
                                       uint32_t* slot_of) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n_edge) return;
    keys[2 * e] = src_idx[e];
    keys[2 * e + 1] = tgt_idx[e];
    slot_of[2 * e] = 0xffffffffu;
    slot_of[2 * e + 1] = 0xffffffffu;
}

__global__ void invert_perm_kernel(const uint32_t* row_ptr, size_t nb, const uint32_t* perm, uint32_t* slot_of) {
    size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k < row_ptr[nb]) slot_of[perm[k]] = (uint32_t)k;
}

template <bool STAGED>
__global__ void gcn_bwd_edge_terms_slots_kernel(const float* go, const float* h, const float* deg,
                                                const uint64_t* src_idx, const uint64_t* tgt_idx, size_t n_edge,
                                                size_t n_nodes, size_t stride, const uint32_t* slot_of, float* terms,
                                                bool vec4) {
    size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (STAGED) {
        const bool in = e < n_edge;
        const uint64_t s = in ? src_idx[e] : 0, t = in ? tgt_idx[e] : 0;
        float gs, gt;
        edge_terms_staged(go, h, deg, s, t, in && s < n_nodes && t < n_nodes, stride, gs, gt);
        if (in) {
            const uint32_t slot_s = slot_of[2 * e], slot_t = slot_of[2 * e + 1];
            if (slot_s != 0xffffffffu) terms[slot_s] = gs;
            if (slot_t != 0xffffffffu) terms[slot_t] = gt;
        }
        return;
    }
    if (e >= n_edge) return;
    const uint64_t s = src_idx[e], t = tgt_idx[e];
    const uint32_t slot_s = slot_of[2 * e], slot_t = slot_of[2 * e + 1];
    float gs = 0.f, gt = 0.f;
    if (s < n_nodes && t < n_nodes) {
        const float ds = deg[s], dt = deg[t];
        const float* gr = go + t * stride;
        const float* hr = h + s * stride;
        auto term = [&](float g, float hv) {
            gs = __fadd_rn(gs, __fmul_rn(__fmul_rn(g, dt), hv));
            gt = __fadd_rn(gt, __fmul_rn(__fmul_rn(g, ds), hv));
        };
        if (vec4) {  // stride a multiple of 4 and both matrices 16-byte aligned: a row is whole 16-byte pieces
            for (size_t j = 0; j < stride; j += 16) {  // up to four pieces of each row in flight
                float4 gv[4], hv[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    if (j + 4 * u < stride) {
                        gv[u] = *reinterpret_cast<const float4*>(gr + j + 4 * u);
                        hv[u] = *reinterpret_cast<const float4*>(hr + j + 4 * u);
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    if (j + 4 * u < stride) {
                        term(gv[u].x, hv[u].x);
                        term(gv[u].y, hv[u].y);
                        term(gv[u].z, hv[u].z);
                        term(gv[u].w, hv[u].w);
                    }
                }
            }
        } else {
            for (size_t j = 0; j < stride; j++) term(gr[j], hr[j]);
        }
    }
    if (slot_s != 0xffffffffu) terms[slot_s] = gs;
    if (slot_t != 0xffffffffu) terms[slot_t] = gt;
}

// The degree gradient of a node is the sum of its edges' terms in edge order, the source term of an edge before its target
// term; a node's edges are in two lists (by source, by target), each in edge order.  Instead of merging the two lists
// while adding (a node of a hundred thousand edges: one dependent load after the other, 140 ns a term), every term is
// first put where it belongs in the merged order, which it can find on its own: entry i of the node's source list goes
// behind the i source terms before it and the target terms of earlier edges (a binary search of the target list), entry
// j of the target list behind j target terms and the source terms of edges up to its own.  The merged lists of all nodes
// lie one after the other, node v's at rp_src[v] + rp_tgt[v]; then the terms are contiguous per node and are added by
// gcn_bwd_graddeg_slots_kernel, or by long_bucket_kernel for a node of many terms.
__global__ void graddeg_rows_kernel(const uint32_t* rp_src, const uint32_t* rp_tgt, size_t n_nodes, uint32_t* rp_merged,
                                    uint32_t* long_list) {
    const size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v > n_nodes) return;
    const uint32_t at = rp_src[v] + rp_tgt[v];
    rp_merged[v] = at;
    if (v < n_nodes && rp_src[v + 1] + rp_tgt[v + 1] - at > kLongBucket) long_list[1 + atomicAdd(&long_list[0], 1u)] = (uint32_t)v;
}

__global__ void graddeg_place_kernel(const uint64_t* src_idx, const uint64_t* tgt_idx, const float* term_src,
                                     const float* term_tgt, const uint32_t* rp_src, const uint32_t* perm_src,
                                     const uint32_t* rp_tgt, const uint32_t* perm_tgt, size_t n_nodes, size_t n_edge,
                                     float* merged) {
    const size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_edge) return;
    if (k < rp_src[n_nodes]) {  // entry k of the by-source ordering
        const uint32_t e = perm_src[k];
        const size_t v = (size_t)src_idx[e];
        const uint32_t* other = perm_tgt + rp_tgt[v];
        uint32_t lo = 0, hi = rp_tgt[v + 1] - rp_tgt[v];  // target terms of edges before e
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (other[mid] < e) lo = mid + 1;
            else hi = mid;
        }
        merged[(size_t)rp_tgt[v] + k + lo] = term_src[e];
    }
    if (k < rp_tgt[n_nodes]) {  // entry k of the by-target ordering
        const uint32_t e = perm_tgt[k];
        const size_t v = (size_t)tgt_idx[e];
        const uint32_t* other = perm_src + rp_src[v];
        uint32_t lo = 0, hi = rp_src[v + 1] - rp_src[v];  // source terms of edges up to e
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (other[mid] <= e) lo = mid + 1;
            else hi = mid;
        }
        merged[(size_t)rp_src[v] + k + lo] = term_tgt[e];
    }
}

__global__ void gcn_bwd_graddeg_slots_kernel(float* grad_deg, const float* terms, const uint32_t* row_ptr,
                                             size_t n_nodes, bool fresh) {
    size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= n_nodes) return;
    const uint32_t s = row_ptr[v], e = row_ptr[v + 1];
    if (s == e) {
        if (fresh) grad_deg[v] = 0.f;
        return;
    }
    if (e - s > kLongBucket) return;  // long_bucket_kernel's
    float acc = fresh ? 0.f : grad_deg[v];
    for (uint32_t k = s; k < e; k += 8) {
        float tv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) tv[u] = (k + u < e) ? terms[k + u] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (k + u < e) acc = __fadd_rn(acc, tv[u]);
    }
    grad_deg[v] = acc;
}

// src/ndarray.zig:614-624
struct GatherMeta {
    uint64_t v[24];  // [idx_strides(8) | src_strides(8) | src_shape(8)]
};
// offsets[i] = flat position in the source of idx coordinate i with its `dim` coordinate replaced by indices[i]
// (src/ndarray.zig:607-624); with `src` the values are taken in the same pass (mem_take, :625-633).  An index
// beyond the source's dim raises the status flag (when there is one) and yields offset 0 and no value.
__global__ void gather_offsets_kernel(const uint64_t* indices, size_t n, int rank, size_t dim, GatherMeta gm,
                                      uint64_t* offsets, int* status, const float* src, float* dst) {
    const uint64_t* meta = gm.v;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t rem = i, off = 0;
    bool bad = false;
    for (int d = 0; d < rank; d++) {
        uint64_t c = rem / meta[d];
        rem = rem % meta[d];
        if ((size_t)d == dim) {
            c = indices[i];
            if (c >= meta[16 + d]) bad = true;
        }
        off += c * meta[8 + d];
    }
    if (bad) {
        if (status) *status = 2;
        offsets[i] = 0;
    } else {
        offsets[i] = off;
        if (src) dst[i] = src[off];
    }
}

__global__ void index_select_fwd_kernel(const float* src, size_t src_len, const uint64_t* indices, size_t n_idx,
                                        size_t stride, float* dst) {
    size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nt = (size_t)gridDim.x * blockDim.x;
    const size_t total = n_idx * stride;
    for (; o < total; o += nt) {
        const size_t d = o / stride, j = o % stride;
        const uint64_t r = indices[d];
        if ((r + 1) * stride <= src_len) dst[o] = src[r * stride + j];
    }
}

// The same for rows of whole 16-byte pieces: G lanes share a row (G a power of two up to the wave), four rows per lane
// group in flight (two or eight measured no better: a gather of random 1 KiB rows runs at the rate DRAM opens pages) (their indices are loaded first, then their pieces), one piece per lane and trip along the row.
template <int G>
__global__ __launch_bounds__(256) void index_select_fwd_vec4_kernel(const float4* src, size_t src_rows, const uint64_t* indices,
                                                                     size_t n_idx, size_t s4, float4* dst, size_t span) {
    constexpr int kRows = 4;
    const int lane = threadIdx.x % G;
    // long rows are cut into spans of pieces (blockIdx.y), so that a few rows of a million values still fill the machine
    const size_t j_begin = (size_t)blockIdx.y * span, j_end = j_begin + span < s4 ? j_begin + span : s4;
    const size_t slot = (size_t)blockIdx.x * (256 / G) + threadIdx.x / G, n_slots = (size_t)gridDim.x * (256 / G);
    for (size_t d0 = slot; d0 < n_idx; d0 += kRows * n_slots) {
        uint64_t r[kRows];
#pragma unroll
        for (int u = 0; u < kRows; u++) {
            const size_t d = d0 + (size_t)u * n_slots;
            r[u] = d < n_idx ? indices[d] : ~(uint64_t)0;
        }
        for (size_t j = j_begin + lane; j < j_end; j += G) {
            float4 v[kRows];
#pragma unroll
            for (int u = 0; u < kRows; u++)
                if (r[u] < src_rows) v[u] = src[r[u] * s4 + j];
#pragma unroll
            for (int u = 0; u < kRows; u++)
                if (r[u] < src_rows) dst[(d0 + (size_t)u * n_slots) * s4 + j] = v[u];
        }
    }
}

static int group_for(size_t stride) {
    if (stride <= 4) return 4;
    if (stride <= 8) return 8;
    if (stride <= 16) return 16;
    if (stride <= 32) return 32;
    return 64;
}

#define ZG_G_DISPATCH(g, CALL)                          \
    switch (g) {                                        \
        case 4: { constexpr int G = 4; CALL; } break;   \
        case 8: { constexpr int G = 8; CALL; } break;   \
        case 16: { constexpr int G = 16; CALL; } break; \
        case 32: { constexpr int G = 32; CALL; } break; \
        default: { constexpr int G = 64; CALL; } break; \
    }

}  // namespace zg

using namespace zg;

static int gather_impl(zg_hip_ctx* ctx, const char* name, const uint64_t* src_shape, const uint64_t* idx_shape, size_t rank,
                       const uint64_t* indices, size_t dim, uint64_t* offsets, int* status, const float* src,
                       float* dst) {
    ZG_REQUIRE(src_shape && idx_shape && indices && offsets, "%s: null pointer", name);
    ZG_REQUIRE(rank >= 1 && rank <= 8 && dim < rank, "%s: bad rank %zu / dim %zu", name, rank, dim);
    if (status) *status = 0;
    for (size_t i = 0; i < rank; i++) {
        if (i != dim && idx_shape[i] > src_shape[i]) {  // src/ndarray.zig:602-604
            if (status) *status = 1;
            set_error("%s: InvalidIndexShape at dim %zu", name, i);
            return ZG_HIP_EINVAL;
        }
    }
    GatherMeta gm;
    uint64_t* meta = gm.v;
    for (int i = 0; i < 24; i++) meta[i] = 0;
    uint64_t a = 1, b = 1;
    for (size_t i = rank; i-- > 0;) {
        meta[i] = a;
        a *= idx_shape[i];
        meta[8 + i] = b;
        b *= src_shape[i];
        meta[16 + i] = src_shape[i];
    }
    const size_t n = (size_t)a;
    if (n == 0) return ZG_HIP_OK;
    // the out-of-bounds flag costs a launch to clear, so it exists only for callers that read it
    int* d_status = status ? (int*)(ctx->scalar_slot + 2) : nullptr;
    if (d_status) {
        hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(64), 0, ctx->stream, (uint32_t*)d_status, (size_t)1,
                           (uint32_t*)nullptr, (size_t)0, (uint32_t*)nullptr);
        ZG_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(gather_offsets_kernel, dim3((unsigned)ceil_div_sz(n, 256)), dim3(256), 0, ctx->stream, indices, n,
                       (int)rank, dim, gm, offsets, d_status, src, dst);
    ZG_LAUNCH_CHECK();
    if (status) {
        ZG_NOT_CAPTURING(ctx, "a gather with a status read-back");
        int h = 0;
        if (int rc = small_d2h(ctx, &h, d_status, sizeof(int))) return rc;
        *status = h;
        if (h) {
            set_error("%s: IndexOutOfBounds", name);
            return ZG_HIP_EINVAL;
        }
    }
    return ZG_HIP_OK;
}

ZG_API int zg_hip_gather_offsets(zg_hip_ctx* ctx, const uint64_t* src_shape, const uint64_t* idx_shape, size_t rank,
                                 const uint64_t* indices, size_t dim, uint64_t* offsets, int* status) {
    ZG_CTX(ctx);
    return gather_impl(ctx, "gather_offsets", src_shape, idx_shape, rank, indices, dim, offsets, status, nullptr, nullptr);
}

ZG_API int zg_hip_gather(zg_hip_ctx* ctx, const float* src, const uint64_t* src_shape, const uint64_t* idx_shape,
                         size_t rank, const uint64_t* indices, size_t dim, uint64_t* offsets, float* dst, int* status) {
    ZG_CTX(ctx);
    ZG_REQUIRE(src && dst, "gather: null pointer");
    return gather_impl(ctx, "gather", src_shape, idx_shape, rank, indices, dim, offsets, status, src, dst);
}

ZG_API int zg_hip_scatter_add(zg_hip_ctx* ctx, const float* src, const uint64_t* offsets, size_t n, float* dst,
                              size_t dst_len) {
    ZG_ENTER(ctx, kWaitAll);
    const bool args_ok = n == 0 || (src && offsets && dst && dst_len > 0 && n < 0xffffffffull && dst_len < 0xffffffffull);
    if (n == 0 || !args_ok) {
        if (int rc = flush_pending(ctx)) return rc;
        if (n == 0) return ZG_HIP_OK;
        ZG_REQUIRE(src && offsets && dst, "scatter_add: null pointer");
        ZG_REQUIRE(dst_len > 0, "scatter_add: empty destination");
        ZG_REQUIRE(false, "scatter_add: sizes beyond 2^32-1");
    }
    // A zero fill of exactly dst that still waits is taken over: the sums are written, untouched elements get their
    // zero from the same launch (GatherBwd fills the gradient, then scatters into it: src/ndtensor.zig:1367-1380).
    // The other waiting fills stay unless they meet an operand.
    const bool small = n <= (size_t)kScatterSmallMax;
    const char *s0 = (const char*)src, *s1 = s0 + n * sizeof(float), *d0 = (const char*)dst, *d1 = d0 + dst_len * sizeof(float);
    const bool apart = !(s0 < d1 && d0 < s1);
    const bool fresh = apart && (!small || dst_len <= kScatterSmallFreshMax) && absorb_zero_fill(ctx, dst, dst_len);
    // A source that is exactly a fill still waiting (a buffer of ones scattered to count edges, examples/gcn/src/
    // model.zig:116-224) is not read: its value is the contribution.  The fill stays queued for whoever reads the
    // buffer next; a caller that frees it right away never pays for it.
    float src_const = 0.f;
    bool const_src = false;
    if (apart)
        for (int i = 0; i < ctx->n_pending_fills && !const_src; i++)
            if (ctx->pending_fills[i].x == src && ctx->pending_fills[i].n == n) {
                const_src = true;
                src_const = ctx->pending_fills[i].value;
            }
    auto owed = [&](int rc_in) {  // refused after the fill was taken over: the zeros are still owed
        if (fresh) (void)zg_hip_mem_fill(ctx, dst, dst_len, 0.f);
        return rc_in;
    };
    {
        const void* ptrs[3] = {const_src ? nullptr : src, offsets, dst};
        const size_t bytes[3] = {n * sizeof(float), n * sizeof(uint64_t), dst_len * sizeof(float)};
        if (int rc = flush_pending_but_fills(ctx, ptrs, bytes, 3)) return owed(rc);
    }
    const float* src_read = const_src ? nullptr : src;
    if (small) {
        hipLaunchKernelGGL(scatter_add_small_kernel, dim3(1), dim3(kScatterSmallMax), 0, ctx->stream, src_read, offsets,
                           (int)n, dst, dst_len, fresh, src_const);
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    PlanRef pr;
    int rc = 0;
    if (!plan_from_cache(ctx, offsets, nullptr, n, dst_len, &pr, &rc)) {
        if (rc) return owed(rc);
        void* mem = workspace(ctx, plan_bytes(n, dst_len));
        if (!mem) return owed(ZG_HIP_EOOM);
        pr.plan = carve_plan(mem, n, dst_len);
        if ((rc = build_plan(ctx, offsets, pr.plan))) return owed(rc);
    }
    if (const_src && fresh && pr.plan.n_long == 0 && dst_len <= kWaitingMapMaxLen) {
        // counting: every destination gets the constant added once per entry of its bucket, which needs neither the
        // source nor the order of the entries; it waits with the small elementwise ops (the GCN adds one and takes
        // the reciprocal square root next, examples/gcn/src/model.zig:116-224: one launch for the three)
        int rc_push = ZG_HIP_OK;
        if (maps_push_count(ctx, dst, pr.plan.row_ptr, dst_len, src_const, &rc_push)) return rc_push;
        if (rc_push) return owed(rc_push);
    }
    return launch_scatter_add_apply(ctx, src_read, pr.plan, dst, fresh, src_const);
}

ZG_API int zg_hip_index_select_fwd(zg_hip_ctx* ctx, const float* src, size_t src_len, const uint64_t* indices,
                                   size_t n_idx, size_t stride, float* dst) {
    ZG_CTX(ctx);
    if (n_idx == 0 || stride == 0) return ZG_HIP_OK;
    ZG_REQUIRE(src && indices && dst, "index_select_fwd: null pointer");
    ZG_REQUIRE(src_len >= stride, "index_select_fwd: source shorter than one row");
    const size_t total = n_idx * stride;
    if (stride % 4 == 0 && aligned16(src) && aligned16(dst)) {
        // rows of whole 16-byte pieces: a lane group per row (an out-of-range index is skipped, as below)
        const size_t s4 = stride / 4;
        const int g = group_for(s4);
        size_t vblocks = ceil_div_sz(n_idx, (size_t)(256 / g) * 4);
        // a workgroup per 16 to 64 rows at any count (a million rows of 1 KiB: 355 -> 339 us against a grid capped at 16
        // workgroups per compute unit)
        if (vblocks > 0x7fffffffull) vblocks = 0x7fffffffull;
        // rows of more than 32 KiB in spans of 16 KiB (1024 rows of 32768 values: 18 % of 8 TB/s as whole rows)
        const size_t span = s4 > 2048 ? 1024 : s4;
        const size_t gy = ceil_div_sz(s4, span);
        ZG_REQUIRE(gy <= 65535, "index_select_fwd: rows of %zu values are too long", stride);
        ZG_G_DISPATCH(g, hipLaunchKernelGGL((index_select_fwd_vec4_kernel<G>), dim3((unsigned)vblocks, (unsigned)gy), dim3(256),
                                            0, ctx->stream, (const float4*)src, src_len / stride, indices, n_idx, s4,
                                            (float4*)dst, span));
        ZG_LAUNCH_CHECK();
        return ZG_HIP_OK;
    }
    size_t blocks = ceil_div_sz(total, 256);
    if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
    hipLaunchKernelGGL(index_select_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, src, src_len, indices,
                       n_idx, stride, dst);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_index_select_bwd(zg_hip_ctx* ctx, const float* y_grad, const uint64_t* indices, size_t n_idx,
                                   size_t stride, float* x_grad, size_t x_len) {
    ZG_CTX(ctx);
    if (n_idx == 0 || stride == 0) return ZG_HIP_OK;
    ZG_REQUIRE(y_grad && indices && x_grad, "index_select_bwd: null pointer");
    ZG_REQUIRE(x_len >= stride, "index_select_bwd: gradient shorter than one row");
    const size_t nb = x_len / stride;
    ZG_REQUIRE(n_idx < 0xffffffffull && nb < 0xffffffffull, "index_select_bwd: sizes beyond 2^32-1");
    PlanRef pr;
    int rc = 0;
    if (!plan_from_cache(ctx, indices, nullptr, n_idx, nb, &pr, &rc)) {
        if (rc) return rc;
        void* mem = workspace(ctx, plan_bytes(n_idx, nb));
        if (!mem) return ZG_HIP_EOOM;
        pr.plan = carve_plan(mem, n_idx, nb);
        if ((rc = build_plan(ctx, indices, pr.plan))) return rc;
    }
    const Plan& pl = pr.plan;
    const int g = group_for(stride);
    const unsigned grid = (unsigned)ceil_div_sz(nb, 256 / g);
    const size_t span = stride > 2048 ? 1024 : stride;
    const size_t gy = ceil_div_sz(stride, span);
    ZG_REQUIRE(gy <= 65535, "index_select_bwd: rows of %zu values are too long", stride);
    ZG_G_DISPATCH(g, hipLaunchKernelGGL((row_scatter_apply_kernel<G>), dim3(grid, (unsigned)gy), dim3(256), 0, ctx->stream,
                                        y_grad, pl.row_ptr, pl.perm, x_grad, nb, stride, span));
    ZG_LAUNCH_CHECK();
    // rows that more than kLongBucket entries select: a wave per column, 64 entries' loads in flight (a row selected
    // ten thousand times: 4.6 ms a thread group walking its entries one by one, 0.2 ms this way)
    return launch_long_buckets(ctx, LongScatterAdd{y_grad, pl.perm, 0.f}, pl.row_ptr, pl.long_list, pl.n, pl.n_long, x_grad, false,
                               stride);
}

namespace zg {
static bool span_meets(const void* p, size_t bytes, const char* lo, const char* hi) {
    return p && (const char*)p < hi && lo < (const char*)p + bytes;
}
// (the orderings and term arrays of both live in plan memory that no caller can name)
bool scatter_wait_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi) {
    const zg_waiting_scatter& w = ctx->scatter_wait;
    if (!w.active) return false;
    const size_t n = w.n_nodes * w.stride * sizeof(float);
    return span_meets(w.dst, n, lo, hi) || span_meets(w.h, n, lo, hi) || span_meets(w.deg, w.n_nodes * sizeof(float), lo, hi) ||
           span_meets(w.bias, w.stride * sizeof(float), lo, hi);
}
bool graddeg_wait_touches(const zg_hip_ctx* ctx, const char* lo, const char* hi) {
    const zg_waiting_graddeg& w = ctx->graddeg_wait;
    if (!w.active) return false;
    const size_t n = w.n_nodes * w.stride * sizeof(float);
    return span_meets(w.grad_output, n, lo, hi) || span_meets(w.h, n, lo, hi) ||
           span_meets(w.deg, w.n_nodes * sizeof(float), lo, hi) || span_meets(w.grad_deg, w.n_nodes * sizeof(float), lo, hi) ||
           span_meets(w.src_idx, w.n_edge * sizeof(uint64_t), lo, hi) || span_meets(w.tgt_idx, w.n_edge * sizeof(uint64_t), lo, hi);
}

int flush_scatter(zg_hip_ctx* ctx) {
    const zg_waiting_scatter w = ctx->scatter_wait;
    if (!w.active) return ZG_HIP_OK;
    ctx->scatter_wait.active = false;
    const int g = group_for(w.stride);
    const unsigned grid = (unsigned)ceil_div_sz(w.n_nodes, 256 / g);
    ZG_G_DISPATCH(g, hipLaunchKernelGGL((gcn_fwd_apply_kernel<G>), dim3(grid), dim3(256), 0, ctx->stream, w.dst, w.h, w.deg,
                                        w.row_ptr, w.peer, w.n_nodes, w.stride, w.fresh, w.bias, w.relu != 0));
    ZG_LAUNCH_CHECK();
    return launch_long_buckets(ctx, LongGcnFwd{w.h, w.deg, w.peer, w.n_nodes}, w.row_ptr, w.long_list, w.n_entries, w.n_long,
                               w.dst, w.fresh, w.stride, w.bias, w.relu != 0);
}

// The sums of the degree-gradient terms through the merged layout (see graddeg_rows_kernel); `long_list[0]` is zero.
static int launch_graddeg_merged(zg_hip_ctx* ctx, const uint64_t* src_idx, const uint64_t* tgt_idx, const float* term_src,
                                 const float* term_tgt, const uint32_t* rp_src, const uint32_t* perm_src,
                                 const uint32_t* rp_tgt, const uint32_t* perm_tgt, size_t n_nodes, size_t n_edge, float* merged,
                                 uint32_t* rp_merged, uint32_t* long_list, float* grad_deg, bool fresh) {
    hipLaunchKernelGGL(graddeg_rows_kernel, dim3((unsigned)ceil_div_sz(n_nodes + 1, 256)), dim3(256), 0, ctx->stream, rp_src,
                       rp_tgt, n_nodes, rp_merged, long_list);
    ZG_LAUNCH_CHECK();
    hipLaunchKernelGGL(graddeg_place_kernel, dim3((unsigned)ceil_div_sz(n_edge, 256)), dim3(256), 0, ctx->stream, src_idx,
                       tgt_idx, term_src, term_tgt, rp_src, perm_src, rp_tgt, perm_tgt, n_nodes, n_edge, merged);
    ZG_LAUNCH_CHECK();
    hipLaunchKernelGGL(gcn_bwd_graddeg_slots_kernel, dim3((unsigned)ceil_div_sz(n_nodes, 256)), dim3(256), 0, ctx->stream,
                       grad_deg, merged, rp_merged, n_nodes, fresh);
    ZG_LAUNCH_CHECK();
    return launch_long_buckets(ctx, LongTerms{merged}, rp_merged, long_list, 2 * n_edge, -1, grad_deg, fresh, 1);
}

// Room behind the two term arrays for the merged layout: 2 * n_edge terms, n_nodes + 1 row pointers, the list of long nodes.
static size_t graddeg_merged_bytes(size_t n_edge, size_t n_nodes) {
    if (2 * n_edge >= 0xffffffffull) return 0;  // positions would not fit 32 bits: the lists are merged as they are read
    return align_up(2 * n_edge * sizeof(float), 256) + align_up((n_nodes + 1) * sizeof(uint32_t), 256) +
           align_up((2 * n_edge / kLongBucket + 2) * sizeof(uint32_t), 256);
}

int flush_graddeg(zg_hip_ctx* ctx) {
    const zg_waiting_graddeg w = ctx->graddeg_wait;
    if (!w.active) return ZG_HIP_OK;
    ctx->graddeg_wait.active = false;
    if (w.by_incidence) {
        // 2 * n_edge terms in bucket order; the two separate term arrays' room holds them
        float* terms = w.term_src;
        if (w.stride > kEtStagedMinStride)
            hipLaunchKernelGGL(gcn_bwd_edge_terms_slots_kernel<true>, dim3((unsigned)ceil_div_sz(w.n_edge, kEtThreads)),
                               dim3(kEtThreads), 0, ctx->stream, w.grad_output, w.h, w.deg, w.src_idx, w.tgt_idx, w.n_edge,
                               w.n_nodes, w.stride, w.slot_of, terms, false);
        else
            hipLaunchKernelGGL(gcn_bwd_edge_terms_slots_kernel<false>, dim3((unsigned)ceil_div_sz(w.n_edge, 256)), dim3(256), 0,
                               ctx->stream, w.grad_output, w.h, w.deg, w.src_idx, w.tgt_idx, w.n_edge, w.n_nodes, w.stride,
                               w.slot_of, terms, w.stride % 4 == 0 && aligned16(w.grad_output) && aligned16(w.h));
        ZG_LAUNCH_CHECK();
        hipLaunchKernelGGL(gcn_bwd_graddeg_slots_kernel, dim3((unsigned)ceil_div_sz(w.n_nodes, 256)), dim3(256), 0,
                           ctx->stream, w.grad_deg, terms, w.inc_row_ptr, w.n_nodes, w.fresh);
        ZG_LAUNCH_CHECK();
        return launch_long_buckets(ctx, LongTerms{terms}, w.inc_row_ptr, w.inc_long_list, 2 * w.n_edge, -1, w.grad_deg, w.fresh, 1);
    }
    if (w.stride > kEtStagedMinStride)
        hipLaunchKernelGGL(gcn_bwd_edge_terms_kernel<true>, dim3((unsigned)ceil_div_sz(w.n_edge, kEtThreads)), dim3(kEtThreads),
                           0, ctx->stream, w.grad_output, w.h, w.deg, w.src_idx, w.tgt_idx, w.n_edge, w.n_nodes, w.stride,
                           w.term_src, w.term_tgt, w.long_merged);
    else
        hipLaunchKernelGGL(gcn_bwd_edge_terms_kernel<false>, dim3((unsigned)ceil_div_sz(w.n_edge, 256)), dim3(256), 0,
                           ctx->stream, w.grad_output, w.h, w.deg, w.src_idx, w.tgt_idx, w.n_edge, w.n_nodes, w.stride,
                           w.term_src, w.term_tgt, w.long_merged);
    ZG_LAUNCH_CHECK();
    if (w.merged)
        return launch_graddeg_merged(ctx, w.src_idx, w.tgt_idx, w.term_src, w.term_tgt, w.rp_src, w.perm_src, w.rp_tgt,
                                     w.perm_tgt, w.n_nodes, w.n_edge, w.merged, w.rp_merged, w.long_merged, w.grad_deg, w.fresh);
    hipLaunchKernelGGL(gcn_bwd_graddeg_kernel, dim3((unsigned)ceil_div_sz(w.n_nodes, 256)), dim3(256), 0, ctx->stream,
                       w.grad_deg, w.term_src, w.term_tgt, w.rp_src, w.perm_src, w.rp_tgt, w.perm_tgt, w.n_nodes, w.fresh);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

// y._add(bias): z = x + y in place on the aggregation's output, the other operand a row of `stride` values
bool scatter_take_add(zg_hip_ctx* ctx, const float* x, size_t xl, const float* y, size_t yl, const float* z, size_t zl) {
    zg_waiting_scatter& w = ctx->scatter_wait;
    const size_t n = w.n_nodes * w.stride;
    if (!w.active || w.bias || w.relu || z != w.dst || zl != n || w.stride == n) return false;
    const float* row = nullptr;
    if (y == w.dst && yl == n && xl == w.stride) row = x;
    else if (x == w.dst && xl == n && yl == w.stride) row = y;
    if (!row) return false;
    if (row < w.dst + n && w.dst < row + w.stride) return false;
    w.bias = row;
    return true;
}

// relu_(y) in place on the aggregation's output: the last thing the layer does, so the kernel goes out
bool scatter_take_relu(zg_hip_ctx* ctx, const float* x, const float* y, size_t n, int* rc) {
    zg_waiting_scatter& w = ctx->scatter_wait;
    if (!w.active || w.relu || x != w.dst || y != w.dst || n != w.n_nodes * w.stride) return false;
    w.relu = 1;
    *rc = flush_scatter(ctx);
    return true;
}
}  // namespace zg

static int check_gcn(const char* name, size_t stride, size_t n_edge, size_t n_nodes) {
    ZG_REQUIRE(stride > 0 && n_nodes > 0, "%s: stride and n_nodes must be positive", name);
    ZG_REQUIRE(n_edge < 0xffffffffull && n_nodes < 0xffffffffull, "%s: sizes beyond 2^32-1", name);
    return ZG_HIP_OK;
}

ZG_API int zg_hip_scatter_gcn_deg_scaled(zg_hip_ctx* ctx, float* dst, const float* h, const float* deg,
                                         const uint64_t* src_indices, const uint64_t* tgt_indices, size_t stride,
                                         size_t n_edge, size_t n_nodes) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    // the output's zero fill (the layer allocates it zeroed, examples/gcn/src/model.zig:100-112) may still be waiting:
    // then the sums are written instead of added to zeros
    const bool fresh = n_edge > 0 && dst && stride > 0 && n_nodes > 0 && absorb_zero_fill(ctx, dst, n_nodes * stride);
    auto owed = [&](int rc_in) {  // refused after the fill was taken over: the zeros are still owed
        if (fresh) (void)zg_hip_mem_fill(ctx, dst, n_nodes * stride, 0.f);
        return rc_in;
    };
    if (int rc = flush_pending(ctx)) return owed(rc);
    if (n_edge == 0) return ZG_HIP_OK;
    if (!(dst && h && deg && src_indices && tgt_indices)) {
        set_error("scatter_gcn_deg_scaled: null pointer");
        return owed(ZG_HIP_EINVAL);
    }
    if (int rc = check_gcn("scatter_gcn_deg_scaled", stride, n_edge, n_nodes)) return owed(rc);
    PlanRef pr;
    int rc = 0;
    if (!plan_from_cache(ctx, tgt_indices, src_indices, n_edge, n_nodes, &pr, &rc)) {
        if (rc) return owed(rc);
        void* mem = workspace(ctx, plan_bytes(n_edge, n_nodes));
        if (!mem) return owed(ZG_HIP_EOOM);
        pr.plan = carve_plan(mem, n_edge, n_nodes);
        if ((rc = build_plan(ctx, tgt_indices, pr.plan, src_indices))) return owed(rc);
    }
    // The plan is ready; the apply kernel waits for the layer's bias add and ReLU (examples/gcn/src/model.zig:100-112,
    // :36), which become its tail.  Whatever else comes next launches it first.
    zg_waiting_scatter& w = ctx->scatter_wait;
    w = zg_waiting_scatter{};
    w.active = true;
    w.dst = dst;
    w.h = h;
    w.deg = deg;
    w.row_ptr = pr.plan.row_ptr;
    w.peer = pr.plan.peer;
    w.long_list = pr.plan.long_list;
    w.n_entries = pr.plan.n;
    w.n_long = pr.plan.n_long;
    w.n_nodes = n_nodes;
    w.stride = stride;
    w.fresh = fresh;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_scatter_gcn_deg_scaled_bwd(zg_hip_ctx* ctx, const float* grad_output, const float* h,
                                             const float* deg, const uint64_t* src_indices,
                                             const uint64_t* tgt_indices, float* grad_h, float* grad_deg, size_t stride,
                                             size_t n_edge, size_t n_nodes) {
    ZG_ENTER(ctx, kWaitFills | kWaitProducts | kWaitSteps);
    // the zero fills of the two gradients (ensure_grad(0), src/ndtensor.zig:221-228) may still be waiting: a gradient
    // whose fill is taken over is written instead of added to zeros
    const bool sized = n_edge > 0 && stride > 0 && n_nodes > 0;
    const bool fresh_h = sized && grad_h && absorb_zero_fill(ctx, grad_h, n_nodes * stride);
    const bool fresh_d = sized && grad_deg && absorb_zero_fill(ctx, grad_deg, n_nodes);
    if (int rc = flush_pending(ctx)) {
        if (fresh_h) (void)zg_hip_mem_fill(ctx, grad_h, n_nodes * stride, 0.f);
        if (fresh_d) (void)zg_hip_mem_fill(ctx, grad_deg, n_nodes, 0.f);
        return rc;
    }
    const int rc_body = [&]() -> int {
    if (n_edge == 0) return ZG_HIP_OK;
    ZG_REQUIRE(grad_output && h && deg && src_indices && tgt_indices && grad_h && grad_deg,
               "scatter_gcn_deg_scaled_bwd: null pointer");
    if (int rc = check_gcn("scatter_gcn_deg_scaled_bwd", stride, n_edge, n_nodes)) return rc;
    const size_t pb = align_up(plan_bytes(n_edge, n_nodes), 256);
    const size_t tb = align_up(n_edge * sizeof(float), 256);
    const size_t mb = graddeg_merged_bytes(n_edge, n_nodes);
    char* mem = (char*)workspace(ctx, 2 * pb + 2 * tb + mb);
    if (!mem) return ZG_HIP_EOOM;
    float* term_src = (float*)(mem + 2 * pb);
    float* term_tgt = (float*)(mem + 2 * pb + tb);
    char* merged_mem = mb ? mem + 2 * pb + 2 * tb : nullptr;
    PlanRef rs, rt;
    int rc = 0;
    if (!plan_from_cache(ctx, src_indices, tgt_indices, n_edge, n_nodes, &rs, &rc)) {
        if (rc) return rc;
        rs.plan = carve_plan(mem, n_edge, n_nodes);
        if ((rc = build_plan(ctx, src_indices, rs.plan, tgt_indices))) return rc;
        rs.keys = src_indices;
        rs.payload = tgt_indices;
    }
    const bool by_incidence = rs.entry && incidence_plan(ctx, rs.entry, &rc);
    if (rc) return rc;
    if (!by_incidence && !plan_from_cache(ctx, tgt_indices, nullptr, n_edge, n_nodes, &rt, &rc)) {
        if (rc) return rc;
        rt.plan = carve_plan(mem + pb, n_edge, n_nodes);
        if ((rc = build_plan(ctx, tgt_indices, rt.plan))) return rc;
    }
    const Plan &by_src = rs.plan, &by_tgt = rt.plan;
    // the edge-term kernel reads both arrays entry by entry: from the cache's device copies when there are any
    src_indices = rs.keys;
    tgt_indices = rs.payload;
    const int g = group_for(stride);
    const unsigned grid = (unsigned)ceil_div_sz(n_nodes, 256 / g);
    ZG_G_DISPATCH(g, hipLaunchKernelGGL((gcn_bwd_gradh_kernel<G>), dim3(grid), dim3(256), 0, ctx->stream, grad_h,
                                        grad_output, deg, by_src.row_ptr, by_src.peer, n_nodes, stride, fresh_h));
    ZG_LAUNCH_CHECK();
    if (int rc2 = launch_long_buckets(ctx, LongGcnGradH{grad_output, deg, by_src.peer, n_nodes}, by_src.row_ptr, by_src.long_list,
                                      by_src.n, by_src.n_long, grad_h, fresh_h, stride))
        return rc2;
    // The degree gradient waits: whatever comes next launches it (its orderings and term arrays live in the cache or in
    // the workspace, which no call touches before it has sent waiting work out), except a free of the block it would
    // write, which drops it.
    zg_waiting_graddeg& w = ctx->graddeg_wait;
    w = zg_waiting_graddeg{};
    w.active = true;
    w.by_incidence = by_incidence;
    w.grad_output = grad_output;
    w.h = h;
    w.deg = deg;
    w.src_idx = src_indices;
    w.tgt_idx = tgt_indices;
    w.n_edge = n_edge;
    w.n_nodes = n_nodes;
    w.stride = stride;
    w.grad_deg = grad_deg;
    w.fresh = fresh_d;
    w.term_src = term_src;
    w.term_tgt = term_tgt;
    if (by_incidence) {
        w.slot_of = rs.entry->slot_of;
        w.inc_row_ptr = rs.entry->inc.row_ptr;
        w.inc_long_list = rs.entry->inc.long_list;
    } else {
        w.rp_src = by_src.row_ptr;
        w.perm_src = by_src.perm;
        w.rp_tgt = by_tgt.row_ptr;
        w.perm_tgt = by_tgt.perm;
        if (merged_mem) {
            w.merged = (float*)merged_mem;
            w.rp_merged = (uint32_t*)(merged_mem + align_up(2 * n_edge * sizeof(float), 256));
            w.long_merged = (uint32_t*)(merged_mem + align_up(2 * n_edge * sizeof(float), 256) +
                                        align_up((n_nodes + 1) * sizeof(uint32_t), 256));
        }
    }
    return ZG_HIP_OK;
    }();
    if (rc_body) {  // refused before its kernels ran: the zeros that were taken over are still owed
        if (fresh_h) (void)zg_hip_mem_fill(ctx, grad_h, n_nodes * stride, 0.f);
        if (fresh_d) (void)zg_hip_mem_fill(ctx, grad_deg, n_nodes, 0.f);
    }
    return rc_body;
}

// ------------------------------------------------------------------------------------------------
// CSR forms (src/device/host_device.zig:1325-1353): segments are given by their boundaries, so no plan is needed.
// ------------------------------------------------------------------------------------------------
namespace zg {

// dst[j] += src[i] for j in [row_ptr[i], row_ptr[i + 1]): one wave per segment.  A boundary beyond dst is clipped.
__global__ __launch_bounds__(256) void scatter_add_csr_kernel(const float* src, const uint64_t* row_ptr, size_t n_seg,
                                                               float* dst, size_t dst_len) {
    const size_t i = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n_seg) return;
    const int lane = threadIdx.x & 63;
    uint64_t s = row_ptr[i], e = row_ptr[i + 1];
    if (e > dst_len) e = dst_len;
    const float v = src[i];
    for (uint64_t j = s + lane; j < e; j += 64) dst[j] = __fadd_rn(dst[j], v);
}

// dst[i] = sum of src[row_ptr[i] .. row_ptr[i + 1]): one wave per segment, four loads in flight per lane, lanes
// combined by a fixed butterfly (the host sums in SIMD lanes: there is no order to match)
__global__ __launch_bounds__(256) void segment_sum_csr_kernel(const float* src, size_t src_len, const uint64_t* row_ptr,
                                                               size_t n_seg, float* dst) {
    const size_t i = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n_seg) return;
    const int lane = threadIdx.x & 63;
    uint64_t s = row_ptr[i], e = row_ptr[i + 1];
    if (e > src_len) e = src_len;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    uint64_t j = s + lane;
    for (; j + 192 < e; j += 256) {
        a0 += src[j];
        a1 += src[j + 64];
        a2 += src[j + 128];
        a3 += src[j + 192];
    }
    for (; j < e; j += 64) a0 += src[j];
    float acc = (a0 + a1) + (a2 + a3);
    for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
    if (lane == 0) dst[i] = acc;
}

}  // namespace zg

ZG_API int zg_hip_scatter_add_csr(zg_hip_ctx* ctx, const float* src, const uint64_t* row_ptr, size_t n_segments,
                                  float* dst, size_t dst_len) {
    ZG_CTX(ctx);
    if (n_segments == 0) return ZG_HIP_OK;
    ZG_REQUIRE(src && row_ptr && dst, "scatter_add_csr: null pointer");
    hipLaunchKernelGGL(scatter_add_csr_kernel, dim3((unsigned)ceil_div_sz(n_segments, 4)), dim3(256), 0, ctx->stream, src,
                       row_ptr, n_segments, dst, dst_len);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_segment_sum_csr(zg_hip_ctx* ctx, const float* src, size_t src_len, const uint64_t* row_offsets,
                                  size_t n_segments, float* dst) {
    ZG_CTX(ctx);
    if (n_segments == 0) return ZG_HIP_OK;
    ZG_REQUIRE(src && row_offsets && dst, "segment_sum_csr: null pointer");
    hipLaunchKernelGGL(segment_sum_csr_kernel, dim3((unsigned)ceil_div_sz(n_segments, 4)), dim3(256), 0, ctx->stream, src,
                       src_len, row_offsets, n_segments, dst);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}

ZG_API int zg_hip_plan_cache_stats(zg_hip_ctx* ctx, uint64_t* hits, uint64_t* builds) {
    ZG_CTX(ctx);
    if (hits) *hits = ctx->plan_cache ? ctx->plan_cache->hits : 0;
    if (builds) *builds = ctx->plan_cache ? ctx->plan_cache->builds : 0;
    return ZG_HIP_OK;
}

// ------------------------------------------------------------------------------------------------
// Edge plans: the segment plans of an edge list that does not change between calls (a dataset's graph), built once.
// The planned ops launch the same apply kernels on the same plans as the ops above, so their results are identical;
// what they save is the plan construction (five launches per plan, two plans in the backward op).
// ------------------------------------------------------------------------------------------------
struct zg_hip_edge_plan {
    void* mem;          // one device allocation: both plans, then device copies of the two index arrays
    zg::Plan by_tgt;    // buckets = targets, peer = source of each edge
    zg::Plan by_src;    // buckets = sources, peer = target of each edge
    uint64_t* src_dev;  // the index arrays as the unplanned ops receive them, in device memory
    uint64_t* tgt_dev;
    size_t n_edge, n_nodes;
};

ZG_API int zg_hip_edge_plan_create(zg_hip_ctx* ctx, const uint64_t* src_indices, const uint64_t* tgt_indices,
                                   size_t n_edge, size_t n_nodes, zg_hip_edge_plan** out) {
    ZG_CTX(ctx);
    ZG_NOT_CAPTURING(ctx, "edge_plan_create");
    ZG_REQUIRE(out != nullptr, "edge_plan_create: null output");
    *out = nullptr;
    ZG_REQUIRE(src_indices && tgt_indices, "edge_plan_create: null pointer");
    ZG_REQUIRE(n_edge > 0, "edge_plan_create: empty edge list");
    if (int rc = check_gcn("edge_plan_create", 1, n_edge, n_nodes)) return rc;
    const size_t pb = align_up(plan_bytes(n_edge, n_nodes), 256), ib = align_up(n_edge * sizeof(uint64_t), 256);
    void* mem = nullptr;
    if (int rc = zg_hip_alloc(ctx, 2 * pb + 2 * ib, &mem)) return rc;
    zg_hip_edge_plan* pl = new zg_hip_edge_plan;
    pl->mem = mem;
    pl->by_tgt = carve_plan(mem, n_edge, n_nodes);
    pl->by_src = carve_plan((char*)mem + pb, n_edge, n_nodes);
    pl->src_dev = (uint64_t*)((char*)mem + 2 * pb);
    pl->tgt_dev = (uint64_t*)((char*)mem + 2 * pb + ib);
    pl->n_edge = n_edge;
    pl->n_nodes = n_nodes;
    int rc = zg_hip_memcpy_d2d(ctx, pl->src_dev, src_indices, n_edge * sizeof(uint64_t));  // device or pinned source
    if (!rc) rc = zg_hip_memcpy_d2d(ctx, pl->tgt_dev, tgt_indices, n_edge * sizeof(uint64_t));
    if (!rc) rc = build_plan(ctx, pl->tgt_dev, pl->by_tgt, pl->src_dev);
    if (!rc) rc = build_plan(ctx, pl->src_dev, pl->by_src, pl->tgt_dev);
    if (!rc) {
        // how many nodes have more than kLongBucket edges is read back once: the calls that use the plan skip the launch of
        // the kernel for such nodes when there is none
        uint32_t n_long[2] = {0, 0};
        if (hipMemcpyAsync(&n_long[0], pl->by_tgt.long_list, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream) == hipSuccess &&
            hipMemcpyAsync(&n_long[1], pl->by_src.long_list, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream) == hipSuccess &&
            hipStreamSynchronize(ctx->stream) == hipSuccess) {
            pl->by_tgt.n_long = (long)n_long[0];
            pl->by_src.n_long = (long)n_long[1];
        } else {
            (void)hipGetLastError();  // the counts stay unknown: the kernel is launched and finds the lists empty or not
        }
    }
    if (rc) {
        zg_hip_free(ctx, mem);
        delete pl;
        return rc;
    }
    *out = pl;
    return ZG_HIP_OK;
}

ZG_API int zg_hip_edge_plan_free(zg_hip_ctx* ctx, zg_hip_edge_plan* plan) {
    ZG_CTX(ctx);
    if (!plan) return ZG_HIP_OK;
    ZG_NOT_CAPTURING(ctx, "edge_plan_free");
    ZG_HIP_TRY(hipStreamSynchronize(ctx->stream));  // kernels that read the plan may still be queued
    int rc = zg_hip_free(ctx, plan->mem);
    delete plan;
    return rc;
}

// dst[tgt[e]] += src[e] in edge order (zg_hip_scatter_add with offsets = the plan's targets)
ZG_API int zg_hip_scatter_add_planned(zg_hip_ctx* ctx, const float* src, const zg_hip_edge_plan* plan, float* dst,
                                      int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(plan && src && dst, "scatter_add_planned: null pointer");
    return launch_scatter_add_apply(ctx, src, plan->by_tgt, dst, accumulate == 0);
}

ZG_API int zg_hip_scatter_gcn_deg_scaled_planned(zg_hip_ctx* ctx, float* dst, const float* h, const float* deg,
                                                 const zg_hip_edge_plan* plan, const float* bias, int relu, size_t stride,
                                                 int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(plan && dst && h && deg, "scatter_gcn_deg_scaled_planned: null pointer");
    ZG_REQUIRE(stride > 0, "scatter_gcn_deg_scaled_planned: stride is 0");
    const size_t n_nodes = plan->n_nodes;
    const int g = group_for(stride);
    const unsigned grid = (unsigned)ceil_div_sz(n_nodes, 256 / g);
    ZG_G_DISPATCH(g, hipLaunchKernelGGL((gcn_fwd_apply_kernel<G>), dim3(grid), dim3(256), 0, ctx->stream, dst, h, deg,
                                        plan->by_tgt.row_ptr, plan->by_tgt.peer, n_nodes, stride, accumulate == 0, bias,
                                        relu != 0));
    ZG_LAUNCH_CHECK();
    return launch_long_buckets(ctx, LongGcnFwd{h, deg, plan->by_tgt.peer, n_nodes}, plan->by_tgt.row_ptr, plan->by_tgt.long_list,
                               plan->by_tgt.n, plan->by_tgt.n_long, dst, accumulate == 0, stride, bias, relu != 0);
}

ZG_API int zg_hip_scatter_gcn_deg_scaled_bwd_planned(zg_hip_ctx* ctx, const float* grad_output, const float* h,
                                                     const float* deg, const zg_hip_edge_plan* plan, float* grad_h,
                                                     float* grad_deg, size_t stride, int accumulate) {
    ZG_CTX(ctx);
    ZG_REQUIRE(plan && grad_output && h && deg && grad_h, "scatter_gcn_deg_scaled_bwd_planned: null pointer");
    const bool fresh = accumulate == 0;
    ZG_REQUIRE(stride > 0, "scatter_gcn_deg_scaled_bwd_planned: stride is 0");
    const size_t n_nodes = plan->n_nodes, n_edge = plan->n_edge;
    const size_t tb = align_up(n_edge * sizeof(float), 256);
    const size_t mb = graddeg_merged_bytes(n_edge, n_nodes);
    char* mem = (char*)workspace(ctx, 2 * tb + mb);
    if (!mem) return ZG_HIP_EOOM;
    float* term_src = (float*)mem;
    float* term_tgt = (float*)(mem + tb);
    float* merged = mb ? (float*)(mem + 2 * tb) : nullptr;
    uint32_t* rp_merged = mb ? (uint32_t*)(mem + 2 * tb + align_up(2 * n_edge * sizeof(float), 256)) : nullptr;
    uint32_t* long_merged = mb ? (uint32_t*)((char*)rp_merged + align_up((n_nodes + 1) * sizeof(uint32_t), 256)) : nullptr;
    const int g = group_for(stride);
    const unsigned grid = (unsigned)ceil_div_sz(n_nodes, 256 / g);
    ZG_G_DISPATCH(g, hipLaunchKernelGGL((gcn_bwd_gradh_kernel<G>), dim3(grid), dim3(256), 0, ctx->stream, grad_h,
                                        grad_output, deg, plan->by_src.row_ptr, plan->by_src.peer, n_nodes, stride, fresh));
    ZG_LAUNCH_CHECK();
    if (int rc = launch_long_buckets(ctx, LongGcnGradH{grad_output, deg, plan->by_src.peer, n_nodes}, plan->by_src.row_ptr,
                                     plan->by_src.long_list, plan->by_src.n, plan->by_src.n_long, grad_h, fresh, stride))
        return rc;
    if (!grad_deg) return ZG_HIP_OK;  // the degrees need no gradient (they are data of the graph)
    if (stride > kEtStagedMinStride)
        hipLaunchKernelGGL(gcn_bwd_edge_terms_kernel<true>, dim3((unsigned)ceil_div_sz(n_edge, kEtThreads)), dim3(kEtThreads), 0,
                           ctx->stream, grad_output, h, deg, plan->src_dev, plan->tgt_dev, n_edge, n_nodes, stride, term_src,
                           term_tgt, long_merged);
    else
        hipLaunchKernelGGL(gcn_bwd_edge_terms_kernel<false>, dim3((unsigned)ceil_div_sz(n_edge, 256)), dim3(256), 0, ctx->stream,
                           grad_output, h, deg, plan->src_dev, plan->tgt_dev, n_edge, n_nodes, stride, term_src, term_tgt,
                           long_merged);
    ZG_LAUNCH_CHECK();
    if (merged)
        return launch_graddeg_merged(ctx, plan->src_dev, plan->tgt_dev, term_src, term_tgt, plan->by_src.row_ptr,
                                     plan->by_src.perm, plan->by_tgt.row_ptr, plan->by_tgt.perm, n_nodes, n_edge, merged, rp_merged,
                                     long_merged, grad_deg, fresh);
    hipLaunchKernelGGL(gcn_bwd_graddeg_kernel, dim3((unsigned)ceil_div_sz(n_nodes, 256)), dim3(256), 0, ctx->stream,
                       grad_deg, term_src, term_tgt, plan->by_src.row_ptr, plan->by_src.perm, plan->by_tgt.row_ptr,
                       plan->by_tgt.perm, n_nodes, fresh);
    ZG_LAUNCH_CHECK();
    return ZG_HIP_OK;
}
