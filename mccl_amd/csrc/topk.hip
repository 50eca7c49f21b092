// Top-k gradient sparsifier with error feedback for gfx950.
//
// Semantics (csrc/compression/TopKCompression.cpp:38-120): per bucket,
// adjusted = grad + residual; the k elements of largest |adjusted| go on the
// wire in ascending index order as [u32 k][k x {u32 index, f32 value}];
// residual = adjusted everywhere except 0.0f at the picks.  Ties at the
// threshold magnitude go to the lower index.
//
// Ordering by fabs() is ordering of the 31-bit pattern `key = bits & 0x7FFFFFFF`
// (NaN patterns sort above infinity), so selection is an exact radix select on
// that key.  All buckets of a gradient run in the same launches.
//
// SINGLE-PASS PATH (one pass over the gradient, 12 B/element of HBM traffic, two
// launches; default for buckets of 2^18 elements and more): see the section
// "single-pass path" below.
// EXACT PATH (any input; small buckets and topk_path = 1; six launches):
//   [pass A]   residual <- grad + residual, histogram of key[30:20]
//   refine x2  histograms of key[19:10], key[9:0] among prefix matches
//   count      per 4096-element tile: #(key > T), #(key == T)
//   emit       an element at index i lands at gt_before(i) + min(eq_before(i),
//              need); ties are accepted while eq_before(i) < need
//   Each kernel first derives the previous round's pick from the finished
//   histogram (every block redundantly; the result is identical), so no
//   separate pick launches are needed.
#include "common.hip.h"
#include "runtime.h"

#include <atomic>
#include <vector>

namespace mcclhip {

namespace {

constexpr int kTile = 4096;    // exact path: elements per compaction tile
constexpr int kBins0 = 2048;   // key[30:20]
constexpr int kBinsR = 1024;   // key[19:10], key[9:0]
constexpr int kHistWords = kBins0 + 2 * kBinsR;
constexpr int kStateWords = 32;
constexpr uint32_t kDense = 0xFFFFFFFFu;  // tile count: more candidates than slots, read the residual range itself
constexpr uint64_t kFastMinBucket = 1u << 18;

// per-bucket state words
enum {
    // single-pass path: the candidate window, published by its sample block with ONE 16-byte store
    S_LO_KEY = 0,         // candidates have key >= this
    S_HI_KEY = 1,         // keys >= this fall into the top coarse bin
    S_THAT = 2,           // predicted threshold key; the streaming blocks store 0.0f for keys >= this
    S_READY = 3,          // the call's epoch number once the other three are valid; 0 after the call
    S_P0 = 4, S_R0 = 5,   // exact path: key prefix / picks still to place after round 0
    S_P1 = 6, S_R1 = 7,   // after round 1
    S_T = 8, S_NEED = 9,  // exact threshold key, number of keys == T that are taken
    S_ISTAR = 10,         // single-pass path: ties are taken while index <= this
    S_OK = 11,            // single-pass path: 1 when the window selection succeeded for this bucket
    S_EXACT_HIST = 12,    // 1 when hist round 0 holds the full histogram
    S_TIMEOUT = 13,       // single-pass path: a block gave up waiting (result invalid, payload header poisoned)
    S_BARF = 16           // 16..19: barriers of the exact selection inside the select launch
};

struct Geometry {
    uint64_t n_total;
    uint64_t bucket_elems;
    uint32_t nbuckets;
    uint32_t tiles;    // exact-path tiles per (full) bucket
    uint32_t k_full;   // k of a bucket with bucket_elems elements
    uint32_t k_last;   // k of the last bucket
    uint32_t listed;   // single-pass path: 1 when the buckets are separate buffers (see Buckets)
    uint32_t ftiles;   // single-pass path: streaming tiles allotted per bucket
    uint32_t lcapb;    // single-pass path: capacity of one coarse bin's list (entries)
};

struct Workspace {
    // zeroed at the start of every exact-path call; the single-pass path zeroes what it uses itself
    uint32_t* hist;         // [nbuckets][kHistWords]
    uint32_t* state;        // [nbuckets][kStateWords]
    // scratch, written before read
    uint32_t* tile_gt;      // [nbuckets][tiles]
    uint32_t* tile_eq;      // [nbuckets][tiles]
    uint32_t* blk_above;    // [nbuckets][64] exact selection inside the select launch: keys above the threshold per group
    uint32_t* blk_eq;       // [nbuckets][64] ... keys equal to the threshold per group
    // single-pass path
    uint32_t* tile_cnt;     // [nbuckets][ftiles] candidates in the tile's slots, or kDense
    uint64_t* slots;        // [nbuckets][ftiles][128] (bits << 32) | index, index order
    uint32_t* grp_cnt;      // [nbuckets][64][kCntStride] finished tiles per group (first word of each 256 bytes)
    uint32_t* gsuf;         // [nbuckets][128 bins][64 groups] a group's candidates in the bins above bin j
    uint32_t* bin_fill;     // [nbuckets][128] the bucket's candidates per coarse window bin (= entries of the bin's list)
    uint64_t* blist;        // [nbuckets][63][lcapb] the window's candidates by coarse bin, any order
    int* status;            // caller's device word (may be null): receives MCCL_HIP_ERR_TIMEOUT when a block gives up
};

__device__ __forceinline__ uint64_t bucket_count(const Geometry& g, uint32_t b) {
    const uint64_t start = (uint64_t)b * g.bucket_elems;
    const uint64_t left = g.n_total - start;
    return left < g.bucket_elems ? left : g.bucket_elems;
}
__device__ __forceinline__ uint32_t bucket_k(const Geometry& g, uint32_t b) {
    return b + 1 == g.nbuckets ? g.k_last : g.k_full;
}
__device__ __forceinline__ uint32_t key_of(float v) { return f2u(v) & 0x7FFFFFFFu; }

// Where the buckets of a single-pass call live.  Uniform layout: the buckets are
// consecutive ranges of one gradient (mccl_hip_topk_compress).  Listed layout
// (Geometry::listed): every bucket is a buffer of its own with its own length
// (mccl_hip_topk_compress_list); g.bucket_elems is then the longest bucket.
constexpr uint32_t kMaxListed = MCCL_HIP_TOPK_LIST_MAX;
struct Buckets {
    const float* grad;
    float* residual;
    uint8_t* wire;
    uint64_t wire_stride;
    const float* lgrad[kMaxListed];
    float* lresidual[kMaxListed];
    uint8_t* lwire[kMaxListed];
    uint32_t lcount[kMaxListed];
    uint32_t lk[kMaxListed];
};
// The kernels index the table by bucket number.  Indexing the by-value parameter would make
// the compiler copy all of it to per-lane scratch memory first (2 KiB per lane, and a launch
// that sets up scratch starts several microseconds later); the kernels read it where it
// already lies instead, in the kernel-argument segment, through scalar loads.  Buckets is
// therefore the FIRST parameter of every kernel that takes one.
typedef const __attribute__((address_space(4))) Buckets* BucketsArg;
__device__ __forceinline__ BucketsArg buckets_arg() { return (BucketsArg)__builtin_amdgcn_kernarg_segment_ptr(); }
__device__ __forceinline__ uint64_t bucket_count(const Geometry& g, BucketsArg bk, uint32_t b) {
    return g.listed ? (uint64_t)bk->lcount[b] : bucket_count(g, b);
}
__device__ __forceinline__ uint32_t bucket_k(const Geometry& g, BucketsArg bk, uint32_t b) {
    return g.listed ? bk->lk[b] : bucket_k(g, b);
}
__device__ __forceinline__ const float* bucket_grad(const Geometry& g, BucketsArg bk, uint32_t b) {
    return g.listed ? bk->lgrad[b] : bk->grad + (uint64_t)b * g.bucket_elems;
}
__device__ __forceinline__ float* bucket_residual(const Geometry& g, BucketsArg bk, uint32_t b) {
    return g.listed ? bk->lresidual[b] : bk->residual + (uint64_t)b * g.bucket_elems;
}
__device__ __forceinline__ uint32_t* bucket_wire(const Geometry& g, BucketsArg bk, uint32_t b) {
    return (uint32_t*)(g.listed ? bk->lwire[b] : bk->wire + (uint64_t)b * bk->wire_stride);
}

__global__ __launch_bounds__(kBlock) void k_zero_words(uint32_t* p, uint64_t n) {
    // n is a multiple of 4 and p is 16-byte aligned (see carve())
    u4a* v = (u4a*)p;
    const u4a z = {0u, 0u, 0u, 0u};
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n / 4; i += (uint64_t)gridDim.x * kBlock)
        v[i] = z;
}

// Adds the block's LDS histogram into the bucket's global one (non-empty bins only).
template <int THREADS>
__device__ __forceinline__ void flush_hist(const uint32_t* lds, uint32_t* global, int bins) {
    for (int i = threadIdx.x; i < bins; i += THREADS) {
        uint32_t c = lds[i];
        if (c) atomicAdd(&global[i], c);
    }
}

// Scans a finished histogram from its top bin downwards and returns the bin in
// which the running count reaches `remaining`, and through *left how many of
// the remaining picks fall inside that bin.  Called by all THREADS threads of a
// block with identical arguments; every thread receives the result.
// `floor_bin`: bins below it count as empty.  Returns BINS when the histogram
// holds fewer than `remaining` elements.
template <int BINS, int THREADS>
__device__ __forceinline__ uint32_t pick_bin(const uint32_t* h, uint32_t remaining, uint32_t floor_bin,
                                             uint32_t* left, uint32_t* scratch /* THREADS/kWave + 2 words */) {
    constexpr int PER = (BINS + THREADS - 1) / THREADS;
    uint32_t c[PER];
    uint32_t sum = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int r = threadIdx.x * PER + j;  // reversed bin number
        const int bin = BINS - 1 - r;
        c[j] = (r < BINS && (uint32_t)bin >= floor_bin) ? h[bin] : 0u;
        sum += c[j];
    }
    uint32_t total;
    uint32_t above = block_exclusive_scan_n<THREADS>(sum, scratch, &total);
    uint32_t* res = scratch + THREADS / kWave;
    if (threadIdx.x == 0) { res[0] = BINS; res[1] = 0; }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; j++) {
        if (above < remaining && remaining <= above + c[j]) {
            res[0] = BINS - 1 - (threadIdx.x * PER + j);
            res[1] = remaining - above;
        }
        above += c[j];
    }
    __syncthreads();
    const uint32_t bin = res[0];
    *left = res[1];
    __syncthreads();
    return bin;
}

// pick_bin for NR histograms (or NR ranks in one histogram) at once, in the same
// three barriers.  remaining[z] == 0 switches rank z off (bin[z] = BINS).
// scratch: NR * (THREADS / kWave + 2) words.
template <int BINS, int THREADS, int NR>
__device__ __forceinline__ void pick_bins(const uint32_t* const (&h)[NR], const uint32_t (&remaining)[NR],
                                          uint32_t (&bin)[NR], uint32_t (&left)[NR], uint32_t* scratch) {
    constexpr int PER = (BINS + THREADS - 1) / THREADS;
    constexpr int NW = THREADS / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    uint32_t c[NR][PER], sum[NR], inc[NR];
#pragma unroll
    for (int z = 0; z < NR; z++) {
        sum[z] = 0;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int r = threadIdx.x * PER + j;  // reversed bin number
            c[z][j] = r < BINS ? h[z][BINS - 1 - r] : 0u;
            sum[z] += c[z][j];
        }
        inc[z] = wave_inclusive_scan(sum[z]);
        if (lane == kWave - 1) scratch[z * NW + wave] = inc[z];
    }
    uint32_t* res = scratch + NR * NW;
    if (threadIdx.x < NR) { res[2 * threadIdx.x] = BINS; res[2 * threadIdx.x + 1] = 0; }
    __syncthreads();
#pragma unroll
    for (int z = 0; z < NR; z++) {
        uint32_t above = inc[z] - sum[z];
#pragma unroll
        for (int w2 = 0; w2 < NW; w2++) {  // all reads issued together; a loop up to `wave` waits for each
            const uint32_t s = scratch[z * NW + w2];
            if (w2 < wave) above += s;
        }
#pragma unroll
        for (int j = 0; j < PER; j++) {
            if (above < remaining[z] && remaining[z] <= above + c[z][j]) {
                res[2 * z] = BINS - 1 - (threadIdx.x * PER + j);
                res[2 * z + 1] = remaining[z] - above;
            }
            above += c[z][j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int z = 0; z < NR; z++) {
        bin[z] = res[2 * z];
        left[z] = res[2 * z + 1];
    }
    __syncthreads();
}

// ================================ exact path ======================================

// residual <- grad + residual, histogram of key[30:20].
__global__ __launch_bounds__(kBlock) void k_topk_pass_a(const float* __restrict__ grad, float* residual,
                                                        Geometry g, Workspace w) {
    __shared__ uint32_t lh[kBins0];
    for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
    __syncthreads();
    const uint32_t b = blockIdx.y;
    const uint64_t bn = bucket_count(g, b);
    const float* gp = grad + (uint64_t)b * g.bucket_elems;
    float* rp = residual + (uint64_t)b * g.bucket_elems;
    const uint64_t nvec = bn / 4;
    constexpr int U = 2;
    const uint64_t tile = (uint64_t)kBlock * U;
    for (uint64_t base = (uint64_t)blockIdx.x * tile; base < nvec; base += (uint64_t)gridDim.x * tile) {
        u4a gv[U], rv[U];
        uint64_t idx[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            idx[u] = base + (uint64_t)u * kBlock + threadIdx.x;
            if (idx[u] < nvec) {
                gv[u] = *(const u4u4*)(gp + idx[u] * 4);
                rv[u] = *(const u4u4*)(rp + idx[u] * 4);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (idx[u] < nvec) {
                u4a a;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    float adj = u2f(gv[u][q]) + u2f(rv[u][q]);
                    a[q] = f2u(adj);
                    atomicAdd(&lh[key_of(adj) >> 20], 1u);
                }
                *(u4u4*)(rp + idx[u] * 4) = a;
            }
        }
    }
    const uint64_t gtid = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < 4 && nvec * 4 + gtid < bn) {
        const uint64_t i = nvec * 4 + gtid;
        float adj = gp[i] + rp[i];
        rp[i] = adj;
        atomicAdd(&lh[key_of(adj) >> 20], 1u);
    }
    __syncthreads();
    flush_hist<kBlock>(lh, w.hist + (uint64_t)b * kHistWords, kBins0);
    if (blockIdx.x == 0 && threadIdx.x == 0) w.state[(uint64_t)b * kStateWords + S_EXACT_HIST] = 1;
}

// Derives (prefix, remaining) after `rounds_done` rounds for bucket b from the
// finished histograms; block (0, b) also records them in the state.
__device__ __forceinline__ void exact_prefix(const Geometry& g, const Workspace& w, uint32_t b, int rounds_done,
                                             bool record, uint32_t* prefix, uint32_t* remaining,
                                             uint32_t* scratch) {
    const uint32_t* h = w.hist + (uint64_t)b * kHistWords;
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    uint32_t p = 0, r = bucket_k(g, b);
    if (rounds_done >= 1) {
        uint32_t left;
        const uint32_t bin = pick_bin<kBins0, kBlock>(h, r, 0, &left, scratch);
        p = bin << 20;
        r = left;
        if (record && rounds_done == 1 && threadIdx.x == 0) { st[S_P0] = p; st[S_R0] = r; }
    }
    if (rounds_done >= 2) {
        uint32_t left;
        const uint32_t bin = pick_bin<kBinsR, kBlock>(h + kBins0, r, 0, &left, scratch);
        p |= bin << 10;
        r = left;
        if (record && rounds_done == 2 && threadIdx.x == 0) { st[S_P1] = p; st[S_R1] = r; }
    }
    if (rounds_done >= 3) {
        uint32_t left;
        const uint32_t bin = pick_bin<kBinsR, kBlock>(h + kBins0 + kBinsR, r, 0, &left, scratch);
        p |= bin;
        r = left;
        if (record && threadIdx.x == 0) { st[S_T] = p; st[S_NEED] = r; }
    }
    *prefix = p;
    *remaining = r;
}

// round 0: full histogram of key[30:20] (only for buckets the fast path gave up on);
// round 1 / 2: histogram of the next 10 key bits among elements matching the prefix.
__global__ __launch_bounds__(kBlock) void k_topk_refine(const float* residual, Geometry g, Workspace w,
                                                        int round, int only_failed) {
    __shared__ uint32_t lh[kBins0];
    __shared__ uint32_t scratch[kBlock / kWave + 2];
    const uint32_t b = blockIdx.y;
    const uint32_t* st = w.state + (uint64_t)b * kStateWords;
    if (only_failed && st[S_OK]) return;
    if (round == 0 && st[S_EXACT_HIST]) return;
    const int bins = round == 0 ? kBins0 : kBinsR;
    for (int i = threadIdx.x; i < bins; i += kBlock) lh[i] = 0;
    uint32_t prefix = 0, remaining = 0;
    if (round > 0) exact_prefix(g, w, b, round, blockIdx.x == 0, &prefix, &remaining, scratch);
    __syncthreads();
    const uint64_t bn = bucket_count(g, b);
    const float* rp = residual + (uint64_t)b * g.bucket_elems;
    const int shift = round == 0 ? 20 : (round == 1 ? 10 : 0);
    const int hi_shift = round == 0 ? 31 : shift + 10;
    const uint32_t want = round == 0 ? 0u : prefix >> hi_shift;
    const uint32_t mask = (uint32_t)bins - 1u;
    const uint64_t nvec = bn / 4;
    constexpr int U = 4;
    const uint64_t tile = (uint64_t)kBlock * U;
    for (uint64_t base = (uint64_t)blockIdx.x * tile; base < nvec; base += (uint64_t)gridDim.x * tile) {
        u4a v[U];
        uint64_t idx[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            idx[u] = base + (uint64_t)u * kBlock + threadIdx.x;
            if (idx[u] < nvec) v[u] = *(const u4u4*)(rp + idx[u] * 4);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (idx[u] < nvec) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t key = v[u][q] & 0x7FFFFFFFu;
                    if ((key >> hi_shift) == want) atomicAdd(&lh[(key >> shift) & mask], 1u);
                }
            }
        }
    }
    const uint64_t gtid = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < 4 && nvec * 4 + gtid < bn) {
        const uint32_t key = key_of(rp[nvec * 4 + gtid]);
        if ((key >> hi_shift) == want) atomicAdd(&lh[(key >> shift) & mask], 1u);
    }
    __syncthreads();
    const int off = round == 0 ? 0 : (round == 1 ? kBins0 : kBins0 + kBinsR);
    flush_hist<kBlock>(lh, w.hist + (uint64_t)b * kHistWords + off, bins);
}

// Four consecutive elements of a tile; elements past the bucket end are invalid.
struct Quad {
    uint32_t bits[4];
    bool valid[4];
    uint64_t e;  // bucket-relative index of bits[0]
};

__device__ __forceinline__ Quad load_quad(const float* rp, uint64_t bn, uint32_t t, int it) {
    Quad q;
    q.e = (uint64_t)t * kTile + (uint64_t)it * (kBlock * 4) + (uint64_t)threadIdx.x * 4;
    if (q.e + 4 <= bn) {
        u4a v = *(const u4u4*)(rp + q.e);
#pragma unroll
        for (int j = 0; j < 4; j++) { q.bits[j] = v[j]; q.valid[j] = true; }
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            q.valid[j] = q.e + j < bn;
            q.bits[j] = q.valid[j] ? f2u(rp[q.e + j]) : 0u;
        }
    }
    return q;
}

__global__ __launch_bounds__(kBlock) void k_topk_count(const float* residual, Geometry g, Workspace w,
                                                       int only_failed) {
    __shared__ uint32_t scratch[kBlock / kWave + 2];
    const uint32_t b = blockIdx.y;
    if (only_failed && w.state[(uint64_t)b * kStateWords + S_OK]) return;
    const uint64_t bn = bucket_count(g, b);
    const float* rp = residual + (uint64_t)b * g.bucket_elems;
    uint32_t T, need;
    exact_prefix(g, w, b, 3, blockIdx.x == 0, &T, &need, scratch);
    for (uint32_t t = blockIdx.x; t < g.tiles; t += gridDim.x) {
        uint32_t packed = 0;  // gt in the low half, eq in the high half (each <= 4096)
        if ((uint64_t)t * kTile < bn) {
#pragma unroll
            for (int it = 0; it < kTile / (kBlock * 4); it++) {
                Quad q = load_quad(rp, bn, t, it);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t key = q.bits[j] & 0x7FFFFFFFu;
                    if (q.valid[j]) packed += (key > T ? 1u : 0u) + (key == T ? 0x10000u : 0u);
                }
            }
        }
        uint32_t total;
        block_exclusive_scan(packed, scratch, &total);
        if (threadIdx.x == 0) {
            w.tile_gt[(uint64_t)b * g.tiles + t] = total & 0xFFFFu;
            w.tile_eq[(uint64_t)b * g.tiles + t] = total >> 16;
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_topk_emit(float* residual, Geometry g, Workspace w,
                                                      uint8_t* wire, uint64_t wire_stride, int only_failed) {
    __shared__ uint32_t smem[kBlock / kWave + 2];
    const uint32_t b = blockIdx.y;
    const uint32_t* st = w.state + (uint64_t)b * kStateWords;
    if (only_failed && st[S_OK]) return;
    const uint64_t bn = bucket_count(g, b);
    uint32_t* out = (uint32_t*)(wire + (uint64_t)b * wire_stride);
    if (blockIdx.x == 0 && threadIdx.x == 0) out[0] = bucket_k(g, b);
    float* rp = residual + (uint64_t)b * g.bucket_elems;
    const uint32_t T = st[S_T];
    const uint32_t need = st[S_NEED];
    const uint32_t* tgt = w.tile_gt + (uint64_t)b * g.tiles;
    const uint32_t* teq = w.tile_eq + (uint64_t)b * g.tiles;
    for (uint32_t t = blockIdx.x; t < g.tiles; t += gridDim.x) {
        if ((uint64_t)t * kTile >= bn) break;
        // picks before this tile: sum of the counts of all earlier tiles
        uint32_t sg = 0, se = 0;
        for (uint32_t i = threadIdx.x; i < t; i += kBlock) { sg += tgt[i]; se += teq[i]; }
        uint32_t gt_run, eq_run;
        block_exclusive_scan(sg, smem, &gt_run);
        block_exclusive_scan(se, smem, &eq_run);
#pragma unroll 1
        for (int it = 0; it < kTile / (kBlock * 4); it++) {
            Quad q = load_quad(rp, bn, t, it);
            uint32_t packed = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t key = q.bits[j] & 0x7FFFFFFFu;
                if (q.valid[j]) packed += (key > T ? 1u : 0u) + (key == T ? 0x10000u : 0u);
            }
            uint32_t total;
            const uint32_t ex = block_exclusive_scan(packed, smem, &total);
            uint32_t gt_b = gt_run + (ex & 0xFFFFu);
            uint32_t eq_b = eq_run + (ex >> 16);
            if (packed) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t key = q.bits[j] & 0x7FFFFFFFu;
                    const bool is_gt = q.valid[j] && key > T;
                    const bool is_eq = q.valid[j] && key == T;
                    if (is_gt || (is_eq && eq_b < need)) {
                        const uint32_t pos = gt_b + (eq_b < need ? eq_b : need);
                        out[1 + 2 * (uint64_t)pos] = (uint32_t)(q.e + j);
                        out[2 + 2 * (uint64_t)pos] = q.bits[j];
                        rp[q.e + j] = 0.0f;
                    }
                    gt_b += is_gt ? 1u : 0u;
                    eq_b += is_eq ? 1u : 0u;
                }
            }
            gt_run += total & 0xFFFFu;
            eq_run += total >> 16;
        }
    }
}

// ---- what blocks of one launch use to talk to each other ----------------------------------
__device__ __forceinline__ uint32_t ld_agent(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Histogram add called by all lanes of a wavefront (m: this lane has a key).  When all
// keys of the wavefront fall into one bin - zeros, constants: the inputs that reach the
// dense-region and exact paths - one lane adds the count; 64 adds to one LDS address
// would serialise.
__device__ __forceinline__ void wave_hist_add(uint32_t* lh, bool m, uint32_t bin) {
    const uint64_t act = __ballot(m);
    if (!act) return;
    const int first = __ffsll((long long)act) - 1;
    const uint32_t fb = (uint32_t)__shfl((int)bin, first, kWave);
    if (__ballot(m && bin == fb) == act) {
        if ((int)(threadIdx.x & (kWave - 1)) == first) atomicAdd(&lh[fb], (uint32_t)__popcll(act));
    } else if (m) {
        atomicAdd(&lh[bin], 1u);
    }
}

// All threads of the block call it.  Returns false when the wait timed out.
// Everything blocks hand to each other goes through agent-scope stores, atomics
// and loads (they bypass the per-XCD L2 copies), so the barrier needs no cache
// write-back or invalidate: each wavefront only waits until its own stores and
// atomics have been acknowledged before the block's arrival is counted.  (Whole-
// cache fences here, repeated by a thousand polling blocks, made the kernel ten
// times slower.)
__device__ __forceinline__ bool bucket_barrier(uint32_t* counter, uint32_t parties, uint32_t* flag /* LDS */,
                                               uint64_t limit_ticks) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint64_t t0 = 0;
        uint32_t ok = 1, polls = 0;
        while (ld_agent(counter) < parties) {
            __builtin_amdgcn_s_sleep(8);
            if ((++polls & 63u) == 0) {  // look at the clock now and then
                const uint64_t now = (uint64_t)wall_clock64();
                if (t0 == 0) t0 = now;
                else if (now - t0 > limit_ticks) {
                    ok = 0;
                    break;
                }
            }
        }
        *flag = ok;
    }
    __syncthreads();
    return *flag != 0;
}


// ================================ single-pass path ==================================
// Two launches.
//
// k_topk_stream - blocks of the 1D grid, in dispatch order:
//   sample blocks   one per bucket, the first blocks of the grid.  8192 evenly spread
//                   elements of grad + residual -> the candidate window [lo, hi) and the
//                   predicted threshold; the block clears the bucket's counters and then
//                   publishes the call's epoch number in S_READY.
//   then, segment by segment (segment s = the tiles of bucket s, then the bin blocks of
//   bucket s - 1; the bin blocks of the last bucket close the grid):
//   streaming blocks one per 4096-element tile, in address order.  A wavefront loads its
//                   1024 elements, waits until the bucket's S_READY shows the epoch, stores
//                   residual <- grad + residual (0.0f at or above the predicted threshold)
//                   and stages its candidates (key >= lo) in LDS in index order; the block
//                   writes them to the tile's slots and counts itself into its group of
//                   tiles (at most 64 groups per bucket).
//   bin blocks      64 per bucket.  Block g waits until group g's tiles are finished (when it
//                   is dispatched - one bucket later - they are, except in the last bucket),
//                   counts the group's candidates per coarse window bin (128 bins), publishes
//                   the counts and copies the candidates, binned, to the bucket's per-bin
//                   lists.  It waits for nothing else.
// k_topk_select - 64 blocks per bucket; nothing crosses blocks any more: every block
//                   redundantly finds the bin that holds the k-th largest key (from the
//                   groups' counts), the exact threshold and the tie rule (from that bin's
//                   list) and the number of picks in the groups before its own, then writes
//                   its group's picks, in index order, at that offset of the payload and
//                   repairs the residual where the predicted threshold and the true one
//                   disagree.  A failed selection (threshold outside the window, a bin list
//                   overflow) hands the bucket to the exact selection, run by the bucket's 64
//                   blocks together through counter barriers; the launch covers at most 16
//                   buckets, so that all its blocks are resident at the same time.
//
// Progress in k_topk_stream.  The hardware deals the blocks of a grid to the XCDs round-robin
// and every XCD dispatches its share in grid order.  A streaming block waits only for its
// bucket's sample block, which precedes every streaming block in the grid.  A bin block waits
// only for streaming blocks that precede it in the grid.  Nothing waits for a later block.
// (Variants in which blocks of the streaming launch also performed the selection were built
// and measured: with the streaming block that finishes a group last going on as the group's
// emitter, the slowest XCD collects every emitter, slows down further and jams; with
// dedicated selection blocks in the grid nothing jams, but every dependent memory round trip
// of the selection takes 5 to 8 microseconds while the stream is in flight, the blocks live
// 50 to 100 microseconds each, and the stream loses a quarter of its block slots to them.
// With every bucket's selection blocks at the very end of the grid the launch boundary
// disappears, but the kernel then carries the selection's registers: at 125 registers four
// blocks fit a CU instead of six and the stream - whose blocks idle while their stores are
// acknowledged - takes 15.3 microseconds per bucket instead of 11.8; trimmed to 89 registers
// it streams at 12.6, while the bin blocks' lists and counts have to be written through
// (scattered 8-byte stores, a memory transaction each: 10 microseconds per call; an L2
// write-back per bin block instead costs 380) and every selection block reads its bucket's
// list past its L2.  Whole call 228 microseconds against 221 for the two launches.  Two tiles
// per streaming block, the second tile's loads under way while the first tile's stores are
// acknowledged, stream slower as well: 220 against 205 microseconds.)
// All waits are bounded all the same (`limit_ticks`): a block that gives up sets S_TIMEOUT,
// overwrites the bucket's payload header with kPoisonK and leaves; k_topk_select leaves such
// a bucket alone.
//
// Everything that crosses blocks inside a launch is written and read with agent-scope
// accesses (the XCDs' L2 caches are not coherent for plain ones), and a writer waits for
// its stores' acknowledgements before it signals.

constexpr int kFRegion = 1024;                // elements one wavefront streams
constexpr int kFWaves = kBlock / kWave;       // 4
constexpr int kFTile = kFRegion * kFWaves;    // elements per streaming block
constexpr int kFVecs = kFRegion / (kWave * 4);  // 16-byte vectors per lane and array: all issued at once
constexpr int kTileSlots = 128;               // candidate slots per tile
constexpr int kCoarse = 128;                  // coarse window bins; the last one holds keys >= hi
constexpr int kBinsPerLane = kCoarse / kWave; // 2
constexpr int kGroups = 64;                   // at most this many groups of tiles per bucket
constexpr int kCntStride = 64;                // words between two groups' arrival counters: 256 bytes, so that the
                                              // arrivals of a bucket's tiles spread over memory channels
constexpr int kHeld = 7;                      // tiles per wavefront whose slots a bin / select block keeps in registers
constexpr int kFSample = 8192;                // sampled elements per bucket
constexpr int kSelBuckets = 16;               // buckets per k_topk_select launch: 1024 blocks, all resident
constexpr uint32_t kPoisonK = 0xFFFFFFFFu;    // payload header of a bucket whose selection was abandoned
constexpr uint32_t kGaveUp = 0xFFFFFFFEu;     // a wavefront's count: its wait for the sample timed out
static_assert(kFVecs == 4, "the streaming role is written for four vectors per lane");

__device__ __forceinline__ uint64_t ld_agent64(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent64(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte streaming store written through to memory (agent scope): a later 4-byte
// repair of the same line by a block on another XCD must not be overwritten by a
// delayed write-back of this one.  A store of more than 8 bytes reads its data
// registers over the following cycles: the compiler keeps the next vector
// instruction from overwriting them for stores it emits itself, not for this one,
// hence the wait states inside the statement.
__device__ __forceinline__ void store_through(float* p, u4a v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 2" ::"v"(p), "v"(v) : "memory");
}

// The window of a bucket, one 16-byte store and one 16-byte load: the four words change together.
__device__ __forceinline__ void store16_agent(uint32_t* p, u4a v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" ::"v"(p), "v"(v) : "memory");
}
// (waits for every earlier load of the wavefront as well: they complete in order)
__device__ __forceinline__ u4a load16_agent(const uint32_t* p) {
    u4a v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
// The kCoarse - 1 bins below the top one divide [lo, hi) evenly: bin = ((key - lo) * mul) >> 32.
__device__ __forceinline__ uint32_t window_mul(uint32_t lo, uint32_t hi) {
    const uint32_t range = hi - lo;  // key - lo < range for every key below hi
    if (range <= (uint32_t)(kCoarse - 1)) return 0xFFFFFFFFu;  // a bin per key
    return (uint32_t)((((uint64_t)(kCoarse - 1)) << 32) / range);
}
// The smallest key of bin j (1 <= j <= kCoarse - 1; bin 0 starts at lo): lo + ceil(j * 2^32 / mul).
__device__ __forceinline__ uint32_t window_bin_lo(uint32_t lo, uint32_t mul, uint32_t j) {
    if (j == 0) return lo;
    return lo + (uint32_t)((((uint64_t)j << 32) + mul - 1) / mul);
}

struct FusedGeo {       // per-bucket tiling, derived the same way by every block
    uint64_t bn;        // elements
    uint32_t k;
    uint32_t ntiles;    // streaming tiles
    uint32_t tpg;       // tiles per group
    uint32_t ng;        // groups
};
__device__ __forceinline__ FusedGeo fused_geo(const Geometry& g, BucketsArg bk, uint32_t b) {
    FusedGeo f;
    f.bn = bucket_count(g, bk, b);
    f.k = bucket_k(g, bk, b);
    f.ntiles = (uint32_t)((f.bn + kFTile - 1) / kFTile);
    f.tpg = (f.ntiles + kGroups - 1) / kGroups;
    f.ng = (f.ntiles + f.tpg - 1) / f.tpg;
    return f;
}

// Coarse window bin of a candidate key (key >= lo).
__device__ __forceinline__ uint32_t coarse_bin(uint32_t key, uint32_t lo, uint32_t hi, uint32_t mul) {
    return key >= hi ? (uint32_t)(kCoarse - 1) : __umulhi(key - lo, mul);
}

// Waits until *p == want.  Called by a whole wavefront or a single thread; false when the wait timed out.
// Every poll is a memory transaction on one address (agent-scope loads are not cached):
// few pollers and a pause between polls, or the channel that holds the word becomes the
// bottleneck of every stream that crosses it.
__device__ __forceinline__ bool wait_word(const uint32_t* p, uint32_t want, uint64_t limit_ticks) {
    uint64_t t0 = 0;
    uint32_t polls = 0;
    while ((uint32_t)__builtin_amdgcn_readfirstlane((int)ld_agent(p)) != want) {
        __builtin_amdgcn_s_sleep(16);
        if ((++polls & 63u) == 0) {
            const uint64_t now = (uint64_t)wall_clock64();
            if (t0 == 0) t0 = now;
            else if (now - t0 > limit_ticks) return false;
        }
    }
    asm volatile("" ::: "memory");
    return true;
}

// Waits until the bucket's window is published (S_READY == epoch); called by a whole wavefront
// or a single thread.  win[3] = 0 when the wait timed out.
__device__ __forceinline__ u4a wait_window(const uint32_t* st, uint32_t epoch, uint64_t limit_ticks) {
    uint64_t t0 = 0;
    uint32_t polls = 0;
    for (;;) {
        u4a v = load16_agent(st + S_LO_KEY);
        if ((uint32_t)__builtin_amdgcn_readfirstlane((int)v[3]) == epoch) {
            v[3] = 1u;
            return v;
        }
        __builtin_amdgcn_s_sleep(16);
        if ((++polls & 63u) == 0) {
            const uint64_t now = (uint64_t)wall_clock64();
            if (t0 == 0) t0 = now;
            else if (now - t0 > limit_ticks) {
                v[3] = 0u;
                return v;
            }
        }
    }
}

struct StreamLds {
    union {
        struct {  // sample block
            uint32_t lh[3][kBinsR] __attribute__((aligned(16)));
            uint32_t wsum[3][kBlock / kWave];
            uint32_t res[3][2];
        } s;
        struct {  // streaming block
            uint64_t stage[kFWaves][kWave];  // a wavefront's candidates, (bits << 32) | index, in index order
            uint32_t wcnt[kFWaves];
            uint32_t win[4];                 // the bucket's window as wavefront 0 read it: lo, hi, predicted threshold, ready
        } a;
        struct {  // bin block
            uint32_t dbuf[kFWaves][16 * kWave];  // dense_tile_walk's staging area, one per wavefront
            uint32_t cnt[kCoarse];
            uint32_t base[kCoarse];
            uint32_t win[4];
        } e;
    };
};
struct SelectLds {
    uint32_t lh[kBins0] __attribute__((aligned(16)));  // radix rounds, tie-break, exact fallback
    uint32_t dbuf[kFWaves][16 * kWave];  // dense_tile_walk's staging area, one per wavefront
    uint32_t wsum[1][kBlock / kWave];
    uint32_t res[1][2];
    uint32_t rcnt[kFWaves][kHeld];
    uint32_t wtot[kFWaves];
    uint32_t scratch[kBlock / kWave + 2];
    uint32_t flag;
};

// ---- sample ------------------------------------------------------------------------
// For NR ranks at once: the bin in which a top-down scan of histogram h[z] reaches rank[z],
// and how many of the rank's elements fall inside that bin.  Thread t owns the PER bins below
// BINS - PER t (16-byte LDS reads).  res[z] = {bin, left}; bin = BINS when the histogram holds
// fewer than rank[z] elements or rank[z] == 0.  SHARED: all ranks are read off h[0].  Called
// by all threads of the block.
template <int BINS, int NR, bool SHARED = false>
__device__ __forceinline__ void sample_pick(const uint32_t* const (&h)[NR], const uint32_t (&rank)[NR],
                                            uint32_t (*wsum)[kBlock / kWave], uint32_t (*res)[2]) {
    constexpr int PER = BINS / kBlock;
    constexpr int NH = SHARED ? 1 : NR;  // histograms actually scanned
    static_assert(PER % 4 == 0, "16-byte LDS reads");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    uint32_t c[NH][PER], sum[NH], inc[NH];  // c[z][j]: bin BINS - 1 - PER t - j
#pragma unroll
    for (int z = 0; z < NH; z++) {
        const u4a* row = (const u4a*)&h[z][BINS - PER * (threadIdx.x + 1)];
        sum[z] = 0;
#pragma unroll
        for (int v4 = 0; v4 < PER / 4; v4++) {
            const u4a x = row[PER / 4 - 1 - v4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                c[z][v4 * 4 + q] = x[3 - q];
                sum[z] += x[3 - q];
            }
        }
        inc[z] = wave_inclusive_scan(sum[z]);
        if (lane == kWave - 1) wsum[z][wave] = inc[z];
    }
    if (threadIdx.x < NR) { res[threadIdx.x][0] = BINS; res[threadIdx.x][1] = 0; }
    __syncthreads();
    uint32_t above0[NH];
#pragma unroll
    for (int z = 0; z < NH; z++) {
        above0[z] = inc[z] - sum[z];
#pragma unroll
        for (int i = 0; i < kBlock / kWave; i++)
            if (i < wave) above0[z] += wsum[z][i];
    }
#pragma unroll
    for (int z = 0; z < NR; z++) {
        constexpr int zz_shared = 0;
        const int zh = SHARED ? zz_shared : z;
        uint32_t above = above0[zh];
#pragma unroll
        for (int j = 0; j < PER; j++) {
            if (above < rank[z] && rank[z] <= above + c[zh][j]) {
                res[z][0] = (uint32_t)(BINS - 1 - PER * (int)threadIdx.x - j);
                res[z][1] = rank[z] - above;
            }
            above += c[zh][j];
        }
    }
    __syncthreads();
}

// Radix-selects (11 + 10 key bits) three ranks of the sample, whose keys stay in registers:
// upper and lower end of the candidate window, 6 sigma of the sampling noise away from the
// expected rank of the k-th largest key, and the predicted threshold.  Clears what the
// launches accumulate into, then publishes the window and the epoch with one store.
__device__ __forceinline__ void fused_sample(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                             uint32_t epoch, StreamLds& L) {
    const FusedGeo fg = fused_geo(g, bk, b);
    const uint64_t bn = fg.bn;
    const float* gp = bucket_grad(g, bk, b);
    const float* rp = bucket_residual(g, bk, b);
    const uint64_t nvec = bn / 4;
    constexpr int SV = kFSample / 4;     // sampled vectors
    constexpr int PV = SV / kBlock;      // vectors per thread; their 4 * PV keys stay in registers
    // sampled in runs of 8 vectors (one 128-byte line per array), runs evenly spread
    const uint32_t nsv = nvec < (uint64_t)SV ? (uint32_t)(nvec & ~7ull) : (uint32_t)SV;
    const uint64_t stride = nsv ? (nvec / (nsv / 8)) : 8;  // vectors between run starts (>= 8)
    u4a gv[PV], rv[PV];
#pragma unroll
    for (int j = 0; j < PV; j++) {
        const uint32_t i = (uint32_t)j * kBlock + threadIdx.x;
        const uint32_t ii = i < nsv ? i : 0;
        const uint64_t v = (uint64_t)(ii >> 3) * stride + (ii & 7);
        gv[j] = nsv ? *(const u4u4*)(gp + v * 4) : u4a{0u, 0u, 0u, 0u};
        rv[j] = nsv ? *(const u4u4*)(rp + v * 4) : u4a{0u, 0u, 0u, 0u};
    }
    // while the loads are under way: clear what the launches accumulate into (the
    // acknowledgements are back long before the window is published)
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    if (threadIdx.x < kGroups) st_agent(w.grp_cnt + ((uint64_t)b * kGroups + threadIdx.x) * kCntStride, 0u);
    if (threadIdx.x < kCoarse) st_agent(w.bin_fill + (uint64_t)b * kCoarse + threadIdx.x, 0u);
    if (threadIdx.x == 0) {
        st_agent(st + S_OK, 0u);
        st_agent(st + S_TIMEOUT, 0u);
        st_agent(st + S_BARF, 0u); st_agent(st + S_BARF + 1, 0u); st_agent(st + S_BARF + 2, 0u); st_agent(st + S_BARF + 3, 0u);
    }
    uint32_t* const h0 = &L.s.lh[0][0];  // round 0 uses 2048 bins: lh[0] and lh[1] are adjacent
    {
        const u4a z = {0u, 0u, 0u, 0u};
        for (int i = threadIdx.x; i < 3 * kBinsR / 4; i += kBlock) ((u4a*)h0)[i] = z;
    }
    uint32_t key[PV][4];
#pragma unroll
    for (int j = 0; j < PV; j++) {
        // an element past the sample gets the key 0xFFFFFFFF, which no histogram counts
        const bool have = (uint32_t)j * kBlock + threadIdx.x < nsv;
#pragma unroll
        for (int q = 0; q < 4; q++) key[j][q] = have ? key_of(u2f(gv[j][q]) + u2f(rv[j][q])) : 0xFFFFFFFFu;
    }
    const uint32_t S = nsv * 4;
    const float ks = (float)fg.k * (float)S / (float)bn;
    const float margin = 6.0f * sqrtf(ks) + 16.0f;
    // ranks: 0 upper end of the window, 1 lower end, 2 the predicted threshold itself
    constexpr int NR = 3;
    uint32_t rank[NR];
    rank[0] = ks - margin >= 1.0f ? (uint32_t)(ks - margin) : 0u;  // 0: no upper end
    rank[1] = (uint32_t)(ks + margin) + 1u;                       // > S: no lower end
    rank[2] = ks >= 1.0f ? (uint32_t)ks : 1u;
    const bool active[NR] = {rank[0] >= 1u && rank[0] <= S, rank[1] <= S, rank[2] <= S};
    uint32_t prefix[NR];
    __syncthreads();
    // round 0: key[30:20], one histogram for all ranks
#pragma unroll
    for (int j = 0; j < PV; j++)
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (key[j][q] != 0xFFFFFFFFu) atomicAdd(&h0[key[j][q] >> 20], 1u);
    __syncthreads();
    {
        const uint32_t* const hs[NR] = {h0, h0, h0};
        const uint32_t want[NR] = {active[0] ? rank[0] : 0u, active[1] ? rank[1] : 0u, active[2] ? rank[2] : 0u};
        sample_pick<kBins0, NR, true>(hs, want, L.s.wsum, L.s.res);
    }
#pragma unroll
    for (int z = 0; z < NR; z++) {
        prefix[z] = L.s.res[z][0] << 20;
        rank[z] = L.s.res[z][1];
    }
    __syncthreads();
    // round 1: key[19:10] among the keys that share a rank's first digit
    {
        const u4a z = {0u, 0u, 0u, 0u};
        for (int i = threadIdx.x; i < 3 * kBinsR / 4; i += kBlock) ((u4a*)h0)[i] = z;
    }
    __syncthreads();
    // (three comparisons per key; the few keys that share a rank's first digit take the branch)
    const uint32_t d0 = active[0] ? prefix[0] >> 20 : 0xFFFFFFFFu, d1 = active[1] ? prefix[1] >> 20 : 0xFFFFFFFFu,
                   d2 = active[2] ? prefix[2] >> 20 : 0xFFFFFFFFu;
#pragma unroll
    for (int j = 0; j < PV; j++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t kq = key[j][q], d = kq >> 20;
            if (d == d0 || d == d1 || d == d2) {
                const uint32_t bin = (kq >> 10) & (kBinsR - 1);
                if (d == d0) atomicAdd(&L.s.lh[0][bin], 1u);
                if (d == d1) atomicAdd(&L.s.lh[1][bin], 1u);
                if (d == d2) atomicAdd(&L.s.lh[2][bin], 1u);
            }
        }
    __syncthreads();
    {
        const uint32_t* const hs[NR] = {L.s.lh[0], L.s.lh[1], L.s.lh[2]};
        const uint32_t want[NR] = {active[0] ? rank[0] : 0u, active[1] ? rank[1] : 0u, active[2] ? rank[2] : 0u};
        sample_pick<kBinsR, NR>(hs, want, L.s.wsum, L.s.res);
    }
    if (threadIdx.x == 0) {
#pragma unroll
        for (int z = 0; z < NR; z++) prefix[z] |= (L.s.res[z][0] & (uint32_t)(kBinsR - 1)) << 10;
        const uint32_t lo = active[1] ? prefix[1] : 0u;
        uint32_t hi = active[0] ? (prefix[0] | 0x3FFu) : 0x7FFFFFFFu;  // upper end of the window: rounded up
        if (hi < lo) hi = lo;
        // predicted threshold: middle of its 1024-key cell; never below lo: every pre-zeroed
        // element must be a listed candidate
        uint32_t that = active[2] ? (prefix[2] | 0x200u) : 0x7FFFFFFFu;
        if (that < lo) that = lo;
        // every store above must have arrived before the window is published
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        store16_agent(st + S_LO_KEY, u4a{lo, hi, that, epoch});
    }
    // off the critical path: the histograms of the exact selection, should the select launch need it
    for (int i = threadIdx.x; i < kHistWords; i += kBlock) w.hist[(uint64_t)b * kHistWords + i] = 0u;
}

// ---- a dense tile's elements ---------------------------------------------------------
// Calls f(index, bits, in_range) for every element of tile t of the bucket, 64 elements per
// step, every lane of the wavefront taking part in every step; the loads of 16 steps are in
// flight together and parked in LDS, so the code stays a loop.  AGENT: the residual was
// written by other blocks of the same launch.
template <bool AGENT, class F>
__device__ __forceinline__ void dense_tile_walk(const float* rp, uint64_t bn, uint32_t t, uint32_t* buf, F&& f) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t e0 = (uint64_t)t * kFTile;
    const uint64_t e1 = e0 + kFTile < bn ? e0 + kFTile : bn;
    constexpr int B = 16;
#pragma unroll 1
    for (uint64_t base = e0; base < e1; base += (uint64_t)B * kWave) {
        uint32_t v[B];
#pragma unroll
        for (int j = 0; j < B; j++) {
            const uint64_t i = base + (uint64_t)j * kWave + lane;
            if constexpr (AGENT) v[j] = i < e1 ? ld_agent((const uint32_t*)rp + i) : 0u;
            else v[j] = i < e1 ? f2u(rp[i]) : 0u;
        }
#pragma unroll
        for (int j = 0; j < B; j++) buf[j * kWave + lane] = v[j];  // a lane reads back only what it wrote
#pragma unroll 1
        for (int j = 0; j < B && base + (uint64_t)j * kWave < e1; j++) {  // wave-uniform trip count
            const uint64_t i = base + (uint64_t)j * kWave + lane;
            f((uint32_t)i, buf[j * kWave + lane], i < e1);
        }
    }
}

// ---- a group's tiles as a bin block / select block sees them ------------------------------
// The slots of up to kHeld tiles per wavefront stay in registers, the rest (buckets of more
// than 64 * 4 * kHeld tiles) are re-read from memory on every sweep.  AGENT: the slots were
// written by other blocks of the same launch (agent-scope loads), else by an earlier launch.
template <bool AGENT>
struct GroupTiles {
    const uint32_t* tcnt;
    const uint64_t* slots;
    uint32_t t0;        // the group's first tile
    uint32_t wt0, wt1;  // this wavefront's tiles: a contiguous quarter of the group's
    int lane;
    bool more;          // wave-uniform: dense tiles, or tiles past the register window
    uint32_t cnt[kHeld];            // candidates in the tile's slots, or kDense (wave-uniform)
    uint64_t e0[kHeld], e1[kHeld];  // slot `lane` and slot `64 + lane`

    static __device__ __forceinline__ uint32_t ld32(const uint32_t* p) {
        if constexpr (AGENT) return ld_agent(p);
        else return *p;
    }
    static __device__ __forceinline__ uint64_t ld64(const uint64_t* p) {
        if constexpr (AGENT) return ld_agent64(p);
        else return *p;
    }
    // every load issued at once
    __device__ __forceinline__ void load(const Geometry& g, const Workspace& w, uint32_t b, uint32_t grp,
                                         const FusedGeo& fg) {
        constexpr int NW = kBlock / kWave;
        lane = threadIdx.x & (kWave - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
        tcnt = w.tile_cnt + (uint64_t)b * g.ftiles;
        slots = w.slots + (uint64_t)b * g.ftiles * kTileSlots;
        t0 = grp * fg.tpg;
        const uint32_t t1 = t0 + fg.tpg < fg.ntiles ? t0 + fg.tpg : fg.ntiles;
        const uint32_t pw = (t1 - t0 + NW - 1) / NW;
        wt0 = t0 + wave * pw < t1 ? t0 + wave * pw : t1;
        wt1 = wt0 + pw < t1 ? wt0 + pw : t1;
#pragma unroll
        for (int h = 0; h < kHeld; h++) {
            const uint32_t t = wt0 + h < wt1 ? wt0 + h : t0;  // stays inside the bucket's arrays
            cnt[h] = (uint32_t)__builtin_amdgcn_readfirstlane((int)ld32(tcnt + t));
            e0[h] = ld64(slots + (uint64_t)t * kTileSlots + lane);  // slots past the count: ignored by the sweeps
            e1[h] = ld64(slots + (uint64_t)t * kTileSlots + kWave + lane);
        }
        bool any_dense = false;
#pragma unroll
        for (int h = 0; h < kHeld; h++) any_dense |= wt0 + h < wt1 && cnt[h] == kDense;
        more = any_dense || wt1 > wt0 + kHeld;
    }
    // nd(h, t, cnt, e0, e1) for every ordinary tile (h < kHeld: register-held, else ~0u), dn(h, t)
    // for every dense one.  Order: register-held ordinary tiles first, then the dense ones and
    // those past the register window, in index order.
    template <class ND, class DN>
    __device__ __forceinline__ void sweep(ND&& nd, DN&& dn) const {
#pragma unroll
        for (int h = 0; h < kHeld; h++)
            if (wt0 + h < wt1 && cnt[h] != kDense) nd((uint32_t)h, wt0 + h, cnt[h], e0[h], e1[h]);
        if (more) {
#pragma unroll 1
            for (uint32_t t = wt0; t < wt1; t++) {
                const uint32_t h = t - wt0 < (uint32_t)kHeld ? t - wt0 : ~0u;
                const uint32_t c = (uint32_t)__builtin_amdgcn_readfirstlane((int)ld32(tcnt + t));
                if (c == kDense) {
                    dn(h, t);
                } else if (h == ~0u) {
                    const uint64_t a0 = ld64(slots + (uint64_t)t * kTileSlots + lane);
                    const uint64_t a1 = ld64(slots + (uint64_t)t * kTileSlots + kWave + lane);
                    nd(h, t, c, a0, a1);
                }
            }
        }
    }
};
__device__ __forceinline__ uint32_t key64(uint64_t e) { return (uint32_t)(e >> 32) & 0x7FFFFFFFu; }

__device__ __forceinline__ void fused_give_up(const Workspace& w, uint32_t* st, uint32_t* out) {
    if (threadIdx.x == 0) {
        st_agent(st + S_TIMEOUT, 1u);
        if (w.status) st_agent((uint32_t*)w.status, (uint32_t)MCCL_HIP_ERR_TIMEOUT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        st_agent(out, kPoisonK);
    }
}

// ---- bin block -----------------------------------------------------------------------------
__device__ __forceinline__ void fused_bin(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                          uint32_t grp, const FusedGeo& fg, uint32_t epoch, uint64_t limit_ticks,
                                          StreamLds& L) {
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    // the group's tiles are finished: all its streaming blocks have arrived
    {
        const uint32_t tg0 = grp * fg.tpg;
        const uint32_t in_group = (tg0 + fg.tpg < fg.ntiles ? tg0 + fg.tpg : fg.ntiles) - tg0;
        // the counter is only meaningful once the sample block has cleared it
        if (threadIdx.x == 0) {
            u4a wn = wait_window(st, epoch, limit_ticks);
            if (wn[3] && !wait_word(w.grp_cnt + ((uint64_t)b * kGroups + grp) * kCntStride, in_group, limit_ticks)) wn[3] = 0u;
            L.e.win[0] = wn[0]; L.e.win[1] = wn[1]; L.e.win[2] = wn[2]; L.e.win[3] = wn[3];
        }
        __syncthreads();
        if (!L.e.win[3]) {
            fused_give_up(w, st, bucket_wire(g, bk, b));
            return;
        }
    }
    const uint32_t lo = L.e.win[0], hi = L.e.win[1], wmul = window_mul(L.e.win[0], L.e.win[1]);
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const float* rp = bucket_residual(g, bk, b);
    GroupTiles<true> G;
    G.load(g, w, b, grp, fg);
    // candidates per coarse bin
    if (threadIdx.x < kCoarse) L.e.cnt[threadIdx.x] = 0;
    static_assert(kCoarse <= kBlock, "one thread per coarse bin");
    __syncthreads();
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                if ((uint32_t)lane < cnt) atomicAdd(&L.e.cnt[coarse_bin(key64(a0), lo, hi, wmul)], 1u);
                if ((uint32_t)(kWave + lane) < cnt) atomicAdd(&L.e.cnt[coarse_bin(key64(a1), lo, hi, wmul)], 1u);
            },
            [&](uint32_t, uint32_t t) {
                dense_tile_walk<true>(rp, bn, t, L.e.dbuf[wave], [&](uint32_t, uint32_t v, bool in) {
                    const uint32_t key = v & 0x7FFFFFFFu;
                    const bool cand = in && key >= lo;
                    wave_hist_add(L.e.cnt, cand, cand ? coarse_bin(key, lo, hi, wmul) : 0u);
                });
            });
    __syncthreads();
    if (threadIdx.x < kCoarse) {
        // the bucket's count per bin; what it held before is where this group's entries go in the
        // bin's list (the top bin, keys >= hi, holds picks for certain as long as the window holds
        // and has no list)
        const uint32_t c = L.e.cnt[threadIdx.x];
        L.e.base[threadIdx.x] = c ? __hip_atomic_fetch_add(w.bin_fill + (uint64_t)b * kCoarse + threadIdx.x, c,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                  : 0u;
    }
    if (wave == 0) {
        // this group's candidates above each bin: lane l takes bins 127 - 2 l and 126 - 2 l
        const uint32_t c_hi = L.e.cnt[kCoarse - 1 - 2 * lane], c_lo = L.e.cnt[kCoarse - 2 - 2 * lane];
        const uint32_t inc = wave_inclusive_scan(c_hi + c_lo);
        uint32_t* col = w.gsuf + (uint64_t)b * kCoarse * kGroups + grp;
        col[(uint64_t)(kCoarse - 1 - 2 * lane) * kGroups] = inc - c_hi - c_lo;
        col[(uint64_t)(kCoarse - 2 - 2 * lane) * kGroups] = inc - c_lo;
    }
    __syncthreads();
    // binned copies (read by the next launch: plain stores)
    uint64_t* bl = w.blist + (uint64_t)b * (kCoarse - 1) * g.lcapb;
    auto put = [&](bool valid, uint32_t cb, uint64_t e) {
        if (valid && cb < (uint32_t)(kCoarse - 1)) {
            const uint32_t pos = atomicAdd(&L.e.base[cb], 1u);
            if (pos < g.lcapb) bl[(uint64_t)cb * g.lcapb + pos] = e;
        }
    };
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                put((uint32_t)lane < cnt, coarse_bin(key64(a0), lo, hi, wmul), a0);
                put((uint32_t)(kWave + lane) < cnt, coarse_bin(key64(a1), lo, hi, wmul), a1);
            },
            [&](uint32_t, uint32_t t) {
                dense_tile_walk<true>(rp, bn, t, L.e.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                    const uint32_t key = v & 0x7FFFFFFFu;
                    const bool cand = in && key >= lo;
                    put(cand, cand ? coarse_bin(key, lo, hi, wmul) : 0u, (uint64_t)i | ((uint64_t)v << 32));
                });
            });
}

// ---- the streaming launch ------------------------------------------------------------------
__global__ __launch_bounds__(kBlock, 6) void k_topk_stream(Buckets, Geometry g, Workspace w, uint32_t epoch,
                                                        uint32_t published, uint32_t first_wave,
                                                        uint64_t limit_ticks) {
    const BucketsArg bk = buckets_arg();
    __shared__ StreamLds L;
    if (blockIdx.x < g.nbuckets) {
        fused_sample(bk, g, w, blockIdx.x, published, L);
        return;
    }
    // segment s of the grid: the tiles of bucket s, then the bin blocks of bucket s - 1 (whose
    // tiles are finished or about to be by then: a bin block that is dispatched early only
    // polls); after the last segment the bin blocks of the last bucket
    const uint32_t per = g.ftiles + kGroups;
    const uint32_t j = blockIdx.x - g.nbuckets;
    uint32_t b = j / per, t = j - b * per;
    bool emit = false;
    if (b >= g.nbuckets) {
        t = j - g.nbuckets * per;
        b = g.nbuckets - 1;
        emit = true;
    } else if (t >= g.ftiles) {
        if (b == 0) return;
        t -= g.ftiles;
        b -= 1;
        emit = true;
    }
    const FusedGeo fg = fused_geo(g, bk, b);
    if (emit) {
        if (t < fg.ng) fused_bin(bk, g, w, b, t, fg, epoch, limit_ticks, L);
        return;
    }
    if (t >= fg.ntiles) return;
    // The blocks that start together with the sample blocks would bury the samples' few loads under
    // 40 MB of their own and then wait for the samples all the same: they hold back for two
    // microseconds, and the memory system is busy with their loads while the samples are evaluated.
    if (blockIdx.x < first_wave) __builtin_amdgcn_s_sleep(80);
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint64_t w0 = (uint64_t)t * kFTile + (uint64_t)wave * kFRegion;  // first element of this wave's region
    const bool live = w0 < bn;                                             // wave-uniform
    float* const rbase = bucket_residual(g, bk, b);
    const float* gp = bucket_grad(g, bk, b) + w0;
    float* rp = rbase + w0;
    const uint32_t len = live ? (uint32_t)((bn - w0) < (uint64_t)kFRegion ? (bn - w0) : (uint64_t)kFRegion) : 0u;
    const uint32_t nfull = len / 4;  // full vectors in this region
    u4a gv[kFVecs], rv[kFVecs];
#pragma unroll
    for (int u = 0; u < kFVecs; u++) {
        const uint32_t vi = (uint32_t)u * kWave + lane;
        if (vi < nfull) {
            gv[u] = __builtin_nontemporal_load((const u4u4*)(gp + vi * 4));
            rv[u] = __builtin_nontemporal_load((const u4u4*)(rp + vi * 4));
        }
    }
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    uint32_t* out = bucket_wire(g, bk, b);
    // the window of this bucket: wait for its sample block (one wavefront polls for the block)
    if (wave == 0) {
        const u4a wn = wait_window(st, epoch, limit_ticks);
        if (lane == 0) { L.a.win[0] = wn[0]; L.a.win[1] = wn[1]; L.a.win[2] = wn[2]; L.a.win[3] = wn[3]; }
    }
    __syncthreads();
    const bool ready = L.a.win[3] != 0;
    const uint32_t lo_key = L.a.win[0], that_key = L.a.win[2];
    // both the same in every lane, and kept in scalar registers by saying so at every update
    uint32_t staged = 0;  // candidates of the region so far
    uint32_t dense = 0;   // 1: more candidates than slots
    uint64_t* const slots = L.a.stage[wave];
    auto lanes_below = [&](uint64_t m) {
        return (uint32_t)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
    };
    auto pick = [](const u4a& a, uint32_t q) {
        uint32_t v = a[0];
        v = q == 1 ? a[1] : v;
        v = q == 2 ? a[2] : v;
        return q == 3 ? a[3] : v;
    };
    // Puts back the region's staged candidates that were stored as zeros.
    auto restore_staged = [&]() {
        if ((uint32_t)lane < staged) {
            const uint64_t e = slots[lane];
            if (((uint32_t)(e >> 32) & 0x7FFFFFFFu) >= that_key) st_agent((uint32_t*)rbase + (uint32_t)e, (uint32_t)(e >> 32));
        }
    };
    // Appends the lanes' candidates (mask4: which of a lane's four elements) in index
    // order: lane-major, element-minor.  Nearly every call finds a few lanes with one
    // candidate each: one ballot, one 8-byte LDS store.
    auto append = [&](uint32_t mask4, const u4a& a, uint32_t first_idx) {
        const uint64_t m1 = __ballot(mask4 != 0);
        if (!m1) return;  // wave-uniform
        const uint32_t c = __popc(mask4);
        uint32_t before = lanes_below(m1), total = __popcll(m1);
        const uint64_t m2 = __ballot(c >= 2);
        if (m2) {  // wave-uniform
            before += lanes_below(m2);
            total += __popcll(m2);
            const uint64_t m3 = __ballot(c >= 3);
            if (m3) {
                const uint64_t m4 = __ballot(c >= 4);
                before += lanes_below(m3) + lanes_below(m4);
                total += __popcll(m3) + __popcll(m4);
            }
        }
        if (dense) return;
        total = (uint32_t)__builtin_amdgcn_readfirstlane((int)total);
        if (staged + total > (uint32_t)kWave) {
            // the region goes dense: its earlier candidates were stored as zeros where
            // they reached the predicted threshold; put those values back
            dense = 1u;
            restore_staged();
            return;
        }
        if (mask4) {
            uint32_t pos = staged + before;
            const uint32_t q = (uint32_t)__ffs((int)mask4) - 1u;
            slots[pos] = (uint64_t)(first_idx + q) | ((uint64_t)pick(a, q) << 32);
            uint32_t rest = mask4 & (mask4 - 1u);
            while (rest) {
                const uint32_t q2 = (uint32_t)__ffs((int)rest) - 1u;
                slots[++pos] = (uint64_t)(first_idx + q2) | ((uint64_t)pick(a, q2) << 32);
                rest &= rest - 1u;
            }
        }
        staged = (uint32_t)__builtin_amdgcn_readfirstlane((int)(staged + total));
    };
    if (ready) {
#pragma unroll
        for (int u = 0; u < kFVecs; u++) {
            const uint32_t vi = (uint32_t)u * kWave + lane;
            u4a a = {0u, 0u, 0u, 0u}, z = {0u, 0u, 0u, 0u};
            uint32_t mask4 = 0;
            if (vi < nfull) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float adj = u2f(gv[u][q]) + u2f(rv[u][q]);
                    a[q] = f2u(adj);
                    z[q] = key_of(adj) >= that_key ? 0u : a[q];
                    mask4 |= (key_of(adj) >= lo_key ? 1u : 0u) << q;
                }
            }
            append(mask4, a, (uint32_t)w0 + vi * 4);  // may turn the region dense
            if (vi < nfull) store_through(rp + vi * 4, dense ? a : z);
        }
        // the bucket's last partial vector (bucket length not a multiple of 4) lies in its last region
        if (len & 3) {
            u4a a = {0u, 0u, 0u, 0u};
            uint32_t mask4 = 0;
            if (lane == 0) {
                for (uint32_t q = 0; q < (len & 3); q++) {
                    const float adj = gp[nfull * 4 + q] + rp[nfull * 4 + q];
                    a[q] = f2u(adj);
                    mask4 |= (key_of(adj) >= lo_key ? 1u : 0u) << q;
                }
            }
            append(mask4, a, (uint32_t)w0 + nfull * 4);
            if (lane == 0) {
                for (uint32_t q = 0; q < (len & 3); q++)
                    st_agent((uint32_t*)rp + nfull * 4 + q, (!dense && (a[q] & 0x7FFFFFFFu) >= that_key) ? 0u : a[q]);
            }
        }
    }
    // ---- the tile's candidates, in index order, to its slots ------------------------------
    if (lane == 0) L.a.wcnt[wave] = !ready ? kGaveUp : (dense ? kDense : staged);
    __syncthreads();
    uint32_t before = 0, total = 0;
    bool tile_dense = false, gave_up = false;
#pragma unroll
    for (int i = 0; i < kFWaves; i++) {
        const uint32_t c = L.a.wcnt[i];
        gave_up |= c == kGaveUp;
        tile_dense |= c == kDense;
        if (i < wave) before += c;
        total += c;
    }
    if (gave_up) {  // a wavefront never saw the sample arrive: the bucket's result is invalid
        fused_give_up(w, st, out);
        return;     // without counting the tile: the bucket's bin blocks give up as well
    }
    tile_dense |= total > (uint32_t)kTileSlots;
    if (tile_dense) {
        if (!dense) restore_staged();  // a tile is dense as a whole: its residual holds plain sums
    } else if ((uint32_t)lane < staged) {
        st_agent64(w.slots + ((uint64_t)b * g.ftiles + t) * kTileSlots + before + lane, slots[lane]);
    }
    if (threadIdx.x == 0) st_agent(w.tile_cnt + (uint64_t)b * g.ftiles + t, tile_dense ? kDense : total);
    // ---- the block counts itself into its group once all its stores have arrived ----------
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        __hip_atomic_fetch_add(w.grp_cnt + ((uint64_t)b * kGroups + t / fg.tpg) * kCntStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The need-th smallest index among the list's entries with key == T: radix select over
// the index, 11 + 11 + 10 bits.  for_list(f) calls f(index, key) for every entry of the list
// this thread looks at.  Called by all threads of the block.
template <class ForList>
__device__ __forceinline__ uint32_t resolve_ties64(ForList&& for_list, uint32_t T, uint32_t need,
                                                   uint32_t* lh /* kBins0 words */, uint32_t* scratch) {
    uint32_t iwant = need, iprefix = 0;
    const int shifts[3] = {21, 10, 0};
    const int widths[3] = {11, 11, 10};
    for (int r = 0; r < 3; r++) {
        const int bins = 1 << widths[r];
        for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
        __syncthreads();
        const int hs = shifts[r] + widths[r];
        for_list([&](uint32_t idx, uint32_t key) {
            const bool match = hs >= 32 ? true : ((idx >> hs) == (iprefix >> hs));
            // bins stored reversed, so that pick_bin's top-down scan runs over ascending indices
            if (key == T && match) atomicAdd(&lh[(bins - 1) - ((idx >> shifts[r]) & (bins - 1))], 1u);
        });
        __syncthreads();
        uint32_t left;
        const uint32_t rb = pick_bin<kBins0, kBlock>(lh, iwant, 0, &left, scratch);
        iprefix |= ((uint32_t)(bins - 1) - (rb - (uint32_t)(kBins0 - bins))) << shifts[r];
        iwant = left;
    }
    return iprefix;
}


// The exact selection of one bucket by its select blocks together (same algorithm as the exact
// path: three radix rounds over the key, then an ordered emit), each on its own group's
// element range; four barriers.  Returns false when a barrier wait timed out.
__device__ __forceinline__ bool select_exact_group(BucketsArg bk, const Geometry& g, const Workspace& w, uint32_t b,
                                                   uint32_t grp, const FusedGeo& fg, uint32_t that_key,
                                                   const GroupTiles<false>& G, SelectLds& L, uint64_t limit_ticks) {
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const uint64_t bn = fg.bn;
    float* rp = bucket_residual(g, bk, b);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
    const uint64_t e0 = (uint64_t)grp * fg.tpg * kFTile;
    const uint64_t e1r = e0 + (uint64_t)fg.tpg * kFTile;
    const uint64_t e1 = e1r < bn ? e1r : bn;
    // 1: put back what the streaming blocks stored as 0.0f in this group's tiles
    G.sweep([&](uint32_t, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
                if ((uint32_t)lane < cnt && key64(a0) >= that_key) rp[(uint32_t)a0] = u2f((uint32_t)(a0 >> 32));
                if ((uint32_t)(kWave + lane) < cnt && key64(a1) >= that_key) rp[(uint32_t)a1] = u2f((uint32_t)(a1 >> 32));
            },
            [&](uint32_t, uint32_t) {});
    __syncthreads();  // a block only ever reads the range it restored itself: plain accesses
    // 2: radix select; every wavefront walks a contiguous quarter of the group's range
    constexpr int NW = kBlock / kWave;
    const uint64_t quarter = ((e1 - e0 + NW - 1) / NW + kWave - 1) / kWave * kWave;
    const uint64_t ws0 = e0 + (uint64_t)wave * quarter < e1 ? e0 + (uint64_t)wave * quarter : e1;
    const uint64_t ws1 = ws0 + quarter < e1 ? ws0 + quarter : e1;
    auto walk = [&](auto&& f) {
        constexpr int B = 8;
#pragma unroll 1
        for (uint64_t base = ws0; base < ws1; base += (uint64_t)B * kWave) {
            uint32_t v[B];
#pragma unroll
            for (int j = 0; j < B; j++) {
                const uint64_t i = base + (uint64_t)j * kWave + lane;
                v[j] = i < ws1 ? f2u(rp[i]) : 0u;
            }
#pragma unroll
            for (int j = 0; j < B; j++) {
                const uint64_t i = base + (uint64_t)j * kWave + lane;
                if (base + (uint64_t)j * kWave < ws1) f(i, v[j], i < ws1);  // wave-uniform
            }
        }
    };
    uint32_t* lh = L.lh;
    uint32_t* gh = w.hist + (uint64_t)b * kHistWords;  // cleared by the bucket's sample block
    uint32_t prefix = 0, remaining = fg.k;
#pragma unroll 1
    for (int round = 0; round < 3; round++) {
        const int bins = round == 0 ? kBins0 : kBinsR;
        const int shift = round == 0 ? 20 : (round == 1 ? 10 : 0);
        const int hi_shift = round == 0 ? 31 : shift + 10;
        uint32_t* ghr = gh + (round == 0 ? 0 : (round == 1 ? kBins0 : kBins0 + kBinsR));
        for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
        __syncthreads();
        walk([&](uint64_t, uint32_t v, bool valid) {
            const uint32_t key = v & 0x7FFFFFFFu;
            wave_hist_add(lh, valid && (key >> hi_shift) == (prefix >> hi_shift), (key >> shift) & (uint32_t)(bins - 1));
        });
        __syncthreads();
        for (int i = threadIdx.x; i < bins; i += kBlock) {
            const uint32_t c = lh[i];
            if (c) __hip_atomic_fetch_add(&ghr[i], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (!bucket_barrier(st + S_BARF + round, fg.ng, &L.flag, limit_ticks)) return false;
        for (int i = threadIdx.x; i < bins; i += kBlock) lh[i] = ld_agent(&ghr[i]);
        __syncthreads();
        uint32_t left, bin;
        if (round == 0) bin = pick_bin<kBins0, kBlock>(lh, remaining, 0, &left, L.scratch);
        else bin = pick_bin<kBinsR, kBlock>(lh, remaining, 0, &left, L.scratch);
        prefix |= bin << shift;
        remaining = left;
    }
    const uint32_t T = prefix, need = remaining;
    // 3: keys above and at the threshold per wavefront range, per group, and in the groups before
    uint32_t gt_w = 0, eq_w = 0;  // wave-uniform
    walk([&](uint64_t, uint32_t v, bool valid) {
        const uint32_t key = v & 0x7FFFFFFFu;
        gt_w += (uint32_t)__popcll(__ballot(valid && key > T));
        eq_w += (uint32_t)__popcll(__ballot(valid && key == T));
    });
    uint32_t* wsum = lh;  // LDS words free again: [0..NW) above, [NW..2NW) equal
    __syncthreads();
    if (lane == 0) { wsum[wave] = gt_w; wsum[NW + wave] = eq_w; }
    __syncthreads();
    uint32_t gt_run = 0, eq_run = 0, gt_blk = 0, eq_blk = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) {
        if (i < wave) { gt_run += wsum[i]; eq_run += wsum[NW + i]; }
        gt_blk += wsum[i];
        eq_blk += wsum[NW + i];
    }
    if (threadIdx.x == 0) {
        st_agent(&w.blk_above[(uint64_t)b * kGroups + grp], gt_blk);
        st_agent(&w.blk_eq[(uint64_t)b * kGroups + grp], eq_blk);
    }
    if (!bucket_barrier(st + S_BARF + 3, fg.ng, &L.flag, limit_ticks)) return false;
    {
        static_assert(kGroups <= kBlock, "one thread per group of the bucket");
        const uint32_t vg = threadIdx.x < grp ? ld_agent(&w.blk_above[(uint64_t)b * kGroups + threadIdx.x]) : 0u;
        const uint32_t ve = threadIdx.x < grp ? ld_agent(&w.blk_eq[(uint64_t)b * kGroups + threadIdx.x]) : 0u;
        uint32_t gt_before, eq_before;
        block_exclusive_scan(vg, L.scratch, &gt_before);
        block_exclusive_scan(ve, L.scratch, &eq_before);
        gt_run += gt_before;
        eq_run += eq_before;
    }
    // 4: this wavefront's picks, in index order
    uint32_t* out = bucket_wire(g, bk, b);
    walk([&](uint64_t i, uint32_t v, bool valid) {
        const uint32_t key = v & 0x7FFFFFFFu;
        const bool is_gt = valid && key > T, is_eq = valid && key == T;
        const uint64_t mg = __ballot(is_gt), me = __ballot(is_eq);
        const uint32_t gt_b = gt_run + (uint32_t)__popcll(mg & below);
        const uint32_t eq_b = eq_run + (uint32_t)__popcll(me & below);
        if (is_gt || (is_eq && eq_b < need)) {
            const uint32_t pos = gt_b + (eq_b < need ? eq_b : need);
            out[1 + 2 * (uint64_t)pos] = (uint32_t)i;
            out[2 + 2 * (uint64_t)pos] = v;
            rp[i] = 0.0f;
        }
        gt_run += (uint32_t)__popcll(mg);
        eq_run += (uint32_t)__popcll(me);
    });
    if (grp == 0 && threadIdx.x == 0) {
        st[S_T] = T;
        st[S_NEED] = need;
    }
    return true;
}


// ---- the select launch ----------------------------------------------------------------------
// blockIdx.x = group, blockIdx.y = bucket - first_bucket.  Everything the streaming launch
// left behind is read with plain loads; only the exact fallback talks across blocks.
__global__ __launch_bounds__(kBlock, 4) void k_topk_select(Buckets, Geometry g, Workspace w, uint32_t first_bucket,
                                                           uint64_t limit_ticks) {
    const BucketsArg bk = buckets_arg();
    __shared__ SelectLds L;
    const uint32_t b = first_bucket + blockIdx.y, grp = blockIdx.x;
    const FusedGeo fg = fused_geo(g, bk, b);
    if (grp >= fg.ng) return;
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    uint32_t* out = bucket_wire(g, bk, b);
    // Every load of the first round trip is issued before the first value is looked at, the small
    // ones first: loads complete in order, and the threshold bin is found (and its list requested)
    // while the group's slots are still arriving.
    const u4a win = *(const u4a*)(st + S_LO_KEY);
    const uint32_t gave_up = st[S_TIMEOUT];
    static_assert(kBinsPerLane == 2, "a lane owns two neighbouring bins");
    // scanned from the top bin downwards: lane l looks at bins 127 - 2 l (tot[1]) and 126 - 2 l (tot[0])
    const u2a tot = *(const u2a*)(w.bin_fill + (uint64_t)b * kCoarse + kCoarse - 2 - 2 * (threadIdx.x & (kWave - 1)));
    GroupTiles<false> G;
    G.load(g, w, b, grp, fg);
    if (gave_up) return;  // the streaming launch gave the bucket up: its payload header says so
    if (grp == 0 && threadIdx.x == 0) st[S_READY] = 0u;  // a replay of a captured launch carries the same epoch
    const uint32_t lo = win[0], that_key = win[2], wmul = window_mul(win[0], win[1]);
    const uint32_t k = fg.k;
    const uint64_t bn = fg.bn;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint64_t below = (1ull << lane) - 1ull;
    float* rp = bucket_residual(g, bk, b);

    bool failed = false;
    do {
    // ---- 3: threshold bin from the bucket's counts ------------------------------------------
    const uint32_t inc = wave_inclusive_scan(tot[0] + tot[1]);
    const uint64_t reach = __ballot(inc >= k);
    if (!reach) {  // fewer than k candidates
        failed = true;
        break;
    }
    const int lstar = __ffsll((long long)reach) - 1;
    const uint32_t pair_hi = (uint32_t)__shfl((int)tot[1], lstar, kWave), pair_lo = (uint32_t)__shfl((int)tot[0], lstar, kWave);
    const uint32_t above_pair = (uint32_t)__shfl((int)inc, lstar, kWave) - pair_hi - pair_lo;  // candidates in the bins above the pair
    const bool in_hi = above_pair + pair_hi >= k;                                     // the upper bin of the pair reaches k
    const uint32_t jstar = (uint32_t)(kCoarse - 1 - 2 * lstar) - (in_hi ? 0u : 1u);
    if (jstar == (uint32_t)(kCoarse - 1)) {  // the threshold lies at or above the window's upper end
        failed = true;
        break;
    }
    const uint32_t n2 = in_hi ? pair_hi : pair_lo;                     // candidates in the threshold bin
    const uint32_t above_total = above_pair + (in_hi ? 0u : pair_hi);
    const uint32_t need = k - above_total;                              // picks inside the bin, 1..n2
    // certain picks (bins above the threshold bin) in the groups before this one: requested now,
    // summed when the bin's list has been requested as well
    const uint32_t ab = threadIdx.x < grp ? w.gsuf[((uint64_t)b * kCoarse + jstar) * kGroups + threadIdx.x] : 0u;
    if (n2 > g.lcapb) {  // more keys in the threshold bin than its list holds (heavy ties, clustered values)
        failed = true;
        break;
    }

    // ---- 4: exact threshold from the bin's list ---------------------------------------------
    const uint64_t* l2 = w.blist + ((uint64_t)b * (kCoarse - 1) + jstar) * g.lcapb;
    // the first 4096 entries stay in registers (a bin of the expected width holds about 3500)
    constexpr int kL2Regs = 16;
    uint64_t ent[kL2Regs];
#pragma unroll
    for (int j = 0; j < kL2Regs; j++) {
        const uint32_t i = (uint32_t)j * kBlock + threadIdx.x;
        ent[j] = i < n2 ? l2[i] : 0ull;
    }
    auto for_list2 = [&](auto&& body) {
#pragma unroll
        for (int j = 0; j < kL2Regs; j++)
            if ((uint32_t)j * kBlock + threadIdx.x < n2) body((uint32_t)ent[j], key64(ent[j]));
#pragma unroll 1
        for (uint32_t i = kL2Regs * kBlock + threadIdx.x; i < n2; i += kBlock) {
            const uint64_t e = l2[i];
            body((uint32_t)e, key64(e));
        }
    };
    uint32_t above_before;
    block_exclusive_scan(ab, L.scratch, &above_before);
    uint32_t* lh = L.lh;
    const uint32_t bin_lo = window_bin_lo(lo, wmul, jstar);  // smallest key of the threshold bin
    const uint32_t bin_span = window_bin_lo(lo, wmul, jstar + 1) - bin_lo;  // jstar <= kCoarse - 2
    uint32_t vprefix = 0, want = need;              // key - bin_lo: up to 30 bits, selected as 10 + 10 + 10
    // rounds whose digits lie wholly above the bin's span are skipped
    const int first_round = bin_span <= (1u << 10) ? 2 : (bin_span <= (1u << 20) ? 1 : 0);
#pragma unroll 1
    for (int r = first_round; r < 3; r++) {
        const int sh = 20 - 10 * r;
        const int hs = sh + 10;
        for (int i = threadIdx.x; i < kBinsR; i += kBlock) lh[i] = 0;
        __syncthreads();
        for_list2([&](uint32_t, uint32_t key) {
            const uint32_t v = key - bin_lo;
            if ((v >> hs) == (vprefix >> hs)) atomicAdd(&lh[(v >> sh) & (kBinsR - 1)], 1u);
        });
        __syncthreads();
        {
            const uint32_t* const hists[1] = {lh};
            const uint32_t wants[1] = {want};
            sample_pick<kBinsR, 1>(hists, wants, L.wsum, L.res);
        }
        const uint32_t bin = L.res[0][0], left = L.res[0][1];
        __syncthreads();  // res is rewritten by the next round
        if (bin >= (uint32_t)kBinsR) {  // the list holds fewer matching keys than the counts promised
            failed = true;
            break;
        }
        vprefix |= bin << sh;
        want = left;
    }
    if (failed) break;
    const uint32_t T = bin_lo + vprefix;
    const uint32_t need2 = want;
    const uint32_t ties = lh[vprefix & (kBinsR - 1)];
    __syncthreads();
    // when only some keys equal to T are taken, they are the need2 lowest indices
    const uint32_t istar = ties != need2 ? resolve_ties64(for_list2, T, need2, lh, L.scratch) : 0xFFFFFFFFu;
    auto is_pick = [&](bool valid, uint32_t key, uint32_t idx) {
        return valid && (key > T || (key == T && idx <= istar));
    };
    // the threshold bin's picks at indices below this group's first element
    uint32_t mine_before = 0, mine_all = 0;
    const uint64_t first_elem = (uint64_t)G.t0 * kFTile;
    for_list2([&](uint32_t idx, uint32_t key) {
        if (is_pick(true, key, idx)) {
            mine_all++;
            mine_before += (uint64_t)idx < first_elem ? 1u : 0u;
        }
    });
    uint32_t l2_before, l2_total;
    block_exclusive_scan(mine_before, L.scratch, &l2_before);
    block_exclusive_scan(mine_all, L.scratch, &l2_total);
    if (above_total + l2_total != k) {  // cannot happen with consistent lists
        failed = true;
        break;
    }
    // ---- 5: payload, in index order -----------------------------------------------------------
    // picks per tile first: the register-held tiles' into rcnt, the others' into the total
    uint32_t w_total = 0;
    G.sweep([&](uint32_t h, uint32_t, uint32_t cnt, uint64_t a0, uint64_t a1) {
              const uint32_t c = (uint32_t)__popcll(__ballot(is_pick((uint32_t)lane < cnt, key64(a0), (uint32_t)a0))) +
                                 (uint32_t)__popcll(__ballot(is_pick((uint32_t)(kWave + lane) < cnt, key64(a1), (uint32_t)a1)));
              if (h != ~0u) L.rcnt[wave][h] = c;
              w_total += c;
          },
          [&](uint32_t h, uint32_t t) {
              uint32_t c = 0;
              dense_tile_walk<false>(rp, bn, t, L.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                  c += (uint32_t)__popcll(__ballot(is_pick(in && (v & 0x7FFFFFFFu) >= lo, v & 0x7FFFFFFFu, i)));
              });
              if (h != ~0u) L.rcnt[wave][h] = c;
              w_total += c;
          });
    if (lane == 0) L.wtot[wave] = w_total;
    __syncthreads();
    uint32_t wave_off = above_before + l2_before;
    for (int i = 0; i < wave; i++) wave_off += L.wtot[i];
    auto emit_half = [&](bool valid, uint64_t e, uint32_t pos) {
        const uint32_t key = key64(e), idx = (uint32_t)e, bitsv = (uint32_t)(e >> 32);
        const bool pick = is_pick(valid, key, idx);
        const uint64_t m = __ballot(pick);
        if (pick) {
            const u2a pr = {idx, bitsv};
            *(u2a4*)(out + 1 + 2 * (uint64_t)(pos + (uint32_t)__popcll(m & below))) = pr;
        }
        // the streaming block stored 0.0f for key >= predicted threshold; repair where the prediction was wrong
        if (valid && pick != (key >= that_key)) rp[idx] = pick ? 0.0f : u2f(bitsv);
        return pos + (uint32_t)__popcll(m);
    };
    auto emit_dense = [&](uint32_t t, uint32_t pos) {
        // a dense tile's residual holds plain sums (nothing was stored as zero)
        dense_tile_walk<false>(rp, bn, t, L.dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
            const bool pick = is_pick(in && (v & 0x7FFFFFFFu) >= lo, v & 0x7FFFFFFFu, i);
            const uint64_t m = __ballot(pick);
            if (pick) {
                const uint32_t p = pos + (uint32_t)__popcll(m & below);
                out[1 + 2 * (uint64_t)p] = i;
                out[2 + 2 * (uint64_t)p] = v;
                rp[i] = 0.0f;
            }
            pos += (uint32_t)__popcll(m);
        });
        return pos;
    };
    {
        uint32_t pos = wave_off;
#pragma unroll
        for (int h = 0; h < kHeld; h++) {
            if (G.wt0 + h < G.wt1) {
                if (G.cnt[h] != kDense) {
                    pos = emit_half((uint32_t)lane < G.cnt[h], G.e0[h], pos);
                    pos = emit_half((uint32_t)(kWave + lane) < G.cnt[h], G.e1[h], pos);
                } else {
                    pos += L.rcnt[wave][h];  // written out by the loop below
                }
            }
        }
    }
    if (G.more) {
        uint32_t pos = wave_off;
#pragma unroll 1
        for (uint32_t t = G.wt0; t < G.wt1; t++) {
            const uint32_t cnt = (uint32_t)__builtin_amdgcn_readfirstlane((int)G.tcnt[t]);
            if (cnt == kDense) {
                pos = emit_dense(t, pos);
            } else if (t - G.wt0 < (uint32_t)kHeld) {
                pos += L.rcnt[wave][t - G.wt0];
            } else {
                const uint64_t a0 = G.slots[(uint64_t)t * kTileSlots + lane];
                const uint64_t a1 = G.slots[(uint64_t)t * kTileSlots + kWave + lane];
                pos = emit_half((uint32_t)lane < cnt, a0, pos);
                pos = emit_half((uint32_t)(kWave + lane) < cnt, a1, pos);
            }
        }
    }
    if (grp == 0 && threadIdx.x == 0) {
        st[S_T] = T;
        st[S_NEED] = need2;
        st[S_ISTAR] = istar;
        st[S_OK] = 1u;
    }
    } while (false);
    // the exact selection for a bucket the window could not finish (S_OK stays 0)
    if (failed) {
        if (!select_exact_group(bk, g, w, b, grp, fg, that_key, G, L, limit_ticks)) {
            fused_give_up(w, st, out);
            return;
        }
    }
    if (grp == 0 && threadIdx.x == 0 && !ld_agent(st + S_TIMEOUT)) out[0] = k;
}

// ================================ host side =======================================

uint64_t align4(uint64_t words) { return (words + 3) & ~uint64_t(3); }

uint64_t zeroed_words(const Geometry& g) {
    return align4((uint64_t)g.nbuckets * kHistWords) + align4((uint64_t)g.nbuckets * kStateWords);
}

uint64_t workspace_words(const Geometry& g) {
    return zeroed_words(g) + 2 * align4((uint64_t)g.nbuckets * g.tiles) + 2 * align4((uint64_t)g.nbuckets * kGroups) +
           align4((uint64_t)g.nbuckets * g.ftiles) + align4((uint64_t)g.nbuckets * g.ftiles * kTileSlots * 2) +
           align4((uint64_t)g.nbuckets * kGroups * kCntStride) + align4((uint64_t)g.nbuckets * kCoarse * kGroups) +
           align4((uint64_t)g.nbuckets * kCoarse) + align4((uint64_t)g.nbuckets * (kCoarse - 1) * g.lcapb * 2);
}

Workspace carve(void* base, const Geometry& g) {
    Workspace w;
    uint32_t* p = (uint32_t*)base;
    w.hist = p;        p += align4((uint64_t)g.nbuckets * kHistWords);
    w.state = p;       p += align4((uint64_t)g.nbuckets * kStateWords);
    w.tile_gt = p;     p += align4((uint64_t)g.nbuckets * g.tiles);
    w.tile_eq = p;     p += align4((uint64_t)g.nbuckets * g.tiles);
    w.blk_above = p;   p += align4((uint64_t)g.nbuckets * kGroups);
    w.blk_eq = p;      p += align4((uint64_t)g.nbuckets * kGroups);
    w.tile_cnt = p;    p += align4((uint64_t)g.nbuckets * g.ftiles);
    w.slots = (uint64_t*)p;  p += align4((uint64_t)g.nbuckets * g.ftiles * kTileSlots * 2);
    w.grp_cnt = p;     p += align4((uint64_t)g.nbuckets * kGroups * kCntStride);
    w.gsuf = p;       p += align4((uint64_t)g.nbuckets * kGroups * kCoarse);
    w.bin_fill = p;    p += align4((uint64_t)g.nbuckets * kCoarse);
    w.blist = (uint64_t*)p;
    w.status = nullptr;
    return w;
}

bool make_geometry(uint64_t n_total, uint64_t bucket_elems, double ratio, Geometry* g) {
    if (n_total == 0 || bucket_elems == 0 || n_total > MCCL_HIP_MAX_ELEMS) return false;
    if (bucket_elems > n_total) bucket_elems = n_total;
    if (bucket_elems > 0xFFFFFFFFull) return false;  // indices are 32-bit
    const uint64_t nb = (n_total + bucket_elems - 1) / bucket_elems;
    if (nb > 65535) return false;
    g->n_total = n_total;
    g->bucket_elems = bucket_elems;
    g->nbuckets = (uint32_t)nb;
    g->tiles = (uint32_t)((bucket_elems + kTile - 1) / kTile);
    g->k_full = mccl_hip_topk_k(bucket_elems, ratio);
    g->k_last = mccl_hip_topk_k(n_total - (nb - 1) * bucket_elems, ratio);
    g->listed = 0;
    g->ftiles = (uint32_t)((bucket_elems + kFTile - 1) / kFTile);
    // a coarse bin holds about k / 80 candidates when the window is as wide as a sample of 8192
    // leaves it, the bins at the window's lower end three times that; k / 10 + 2048 entries
    // leave room for more uneven ones
    uint64_t capb = (uint64_t)g->k_full / 10 + 2048;
    if (capb > bucket_elems) capb = bucket_elems;
    g->lcapb = (uint32_t)capb;
    return true;
}

// Every call of the single-pass path carries a number of its own; a bucket's window counts
// as published when its S_READY word shows that number (whatever a workspace held before,
// it is not this call's number; zero is what a finished call leaves behind).
std::atomic<uint32_t> g_epoch{0x5EED0001u};

// The two launches of the single-pass path.  False when the grid would not fit.
bool launch_single_pass(const Buckets& bk, const Geometry& g, const Workspace& w, hipStream_t st) {
    // the streaming launch: a sample block per bucket, then per bucket its tiles and 64 bin blocks
    const uint64_t blocks = (uint64_t)g.nbuckets * ((uint64_t)g.ftiles + kGroups + 1) + kGroups;
    if (blocks >= 0x7FFFFFFFull) return false;
    uint32_t epoch = ++g_epoch;
    if (epoch == 0) epoch = ++g_epoch;
    // 100 MHz ticks a block may wait before it gives up
    const uint64_t lim = (uint64_t)tuning().topk_barrier_ms * 100000ull;
    // blocks that are resident from the start of the launch: they wait for the sample blocks
    static const int per_cu = [] {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k_topk_stream, kBlock, 0) != hipSuccess || n < 1) n = 6;
        return n;
    }();
    const uint32_t first_wave = g.nbuckets + (uint32_t)device_info().num_cus * (uint32_t)per_cu;
    // (tests of the give-up path: the sample blocks publish a number nobody waits for)
    const uint32_t published = tuning().topk_stall_test ? ~epoch : epoch;
    k_topk_stream<<<(uint32_t)blocks, kBlock, 0, st>>>(bk, g, w, epoch, published, first_wave, lim);
    // the select launch, at most kSelBuckets buckets at a time: all its blocks are resident
    // together, whatever the order in which the hardware dispatches them
    for (uint32_t b0 = 0; b0 < g.nbuckets; b0 += kSelBuckets) {
        const uint32_t nb = g.nbuckets - b0 < (uint32_t)kSelBuckets ? g.nbuckets - b0 : (uint32_t)kSelBuckets;
        k_topk_select<<<dim3(kGroups, nb), kBlock, 0, st>>>(bk, g, w, b0, lim);
    }
    return true;
}

}  // namespace
}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

uint32_t mccl_hip_topk_k(uint64_t count, double ratio) {
    uint32_t k = static_cast<uint32_t>(static_cast<double>(count) * ratio);
    return k < 1u ? 1u : k;
}

uint64_t mccl_hip_topk_max_compressed_size(uint64_t nbytes, double ratio) {
    const uint64_t count = nbytes / 4;
    const uint32_t k = static_cast<uint32_t>(static_cast<double>(count) * ratio) + 1u;
    return 4u + (uint64_t)k * 8u;
}

uint64_t mccl_hip_topk_workspace_bytes(uint64_t n_total, uint64_t bucket_elems, double ratio) {
    Geometry g;
    if (!(ratio > 0.0 && ratio <= 1.0)) return 0;
    if (!make_geometry(n_total, bucket_elems, ratio, &g)) return 0;
    return workspace_words(g) * 4 + 256;
}

int mccl_hip_topk_compress(const float* grad, float* residual, uint64_t n_total,
                           uint64_t bucket_elems, double ratio, void* wire,
                           uint64_t wire_stride, void* workspace, uint64_t workspace_bytes,
                           int* status, void* stream) {
    if (!grad || !residual || !wire || !workspace) return MCCL_HIP_ERR_ARG;
    if (!(ratio > 0.0 && ratio <= 1.0)) return MCCL_HIP_ERR_ARG;
    Geometry g;
    if (!make_geometry(n_total, bucket_elems, ratio, &g)) return MCCL_HIP_ERR_ARG;
    if ((wire_stride & 3) || ((uintptr_t)wire & 3)) return MCCL_HIP_ERR_ARG;
    const uint32_t kmax = g.k_full > g.k_last ? g.k_full : g.k_last;
    if (wire_stride < 4 + 8 * (uint64_t)kmax) return MCCL_HIP_ERR_CAPACITY;
    if (workspace_bytes < workspace_words(g) * 4 + 16) return MCCL_HIP_ERR_WORKSPACE;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    // the carved arrays are 16-byte aligned inside the caller's buffer
    void* aligned = (void*)(((uintptr_t)workspace + 15) & ~(uintptr_t)15);
    Workspace w = carve(aligned, g);
    w.status = status;
    const int path = tuning().topk_path;  // 0 auto, 1 exact path only, 2 single-pass path at any size
    bool fast = path == 2 || (path == 0 && g.bucket_elems >= kFastMinBucket);

    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    const uint64_t nvec = g.bucket_elems / 4;
    const uint64_t bx = (cap + g.nbuckets - 1) / g.nbuckets;
    const uint64_t need_r = (nvec + kBlock * 4 - 1) / (kBlock * 4);
    const uint32_t bx_r = clamp_u32(bx < need_r ? bx : need_r, 1, 65535);
    const uint32_t bx_t = clamp_u32(bx < g.tiles ? bx : g.tiles, 1, 65535);
    if (fast) {
        Buckets bk = {};
        bk.grad = grad;
        bk.residual = residual;
        bk.wire = (uint8_t*)wire;
        bk.wire_stride = wire_stride;
        fast = launch_single_pass(bk, g, w, st);
    }
    if (!fast) {
        const uint64_t zw = zeroed_words(g);
        k_zero_words<<<clamp_u32((zw / 4 + kBlock - 1) / kBlock, 1, cap), kBlock, 0, st>>>(w.hist, zw);
        const uint64_t need_a = (nvec + kBlock * 2 - 1) / (kBlock * 2);
        const uint32_t bx_a = clamp_u32(bx < need_a ? bx : need_a, 1, 65535);
        k_topk_pass_a<<<dim3(bx_a, g.nbuckets), kBlock, 0, st>>>(grad, residual, g, w);
        k_topk_refine<<<dim3(bx_r, g.nbuckets), kBlock, 0, st>>>(residual, g, w, 1, 0);
        k_topk_refine<<<dim3(bx_r, g.nbuckets), kBlock, 0, st>>>(residual, g, w, 2, 0);
        k_topk_count<<<dim3(bx_t, g.nbuckets), kBlock, 0, st>>>(residual, g, w, 0);
        k_topk_emit<<<dim3(bx_t, g.nbuckets), kBlock, 0, st>>>(residual, g, w, (uint8_t*)wire, wire_stride, 0);
    }
    return launch_status();
}

uint64_t mccl_hip_topk_list_workspace_bytes(const uint64_t* host_counts, uint32_t nbuckets, double ratio) {
    if (!host_counts || nbuckets == 0 || nbuckets > kMaxListed) return 0;
    uint64_t longest = 0;
    for (uint32_t b = 0; b < nbuckets; b++) {
        if (host_counts[b] == 0) return 0;
        longest = host_counts[b] > longest ? host_counts[b] : longest;
    }
    return mccl_hip_topk_workspace_bytes(longest * nbuckets, longest, ratio);
}

int mccl_hip_topk_compress_list(const float* const* host_grads, float* const* host_residuals,
                                const uint64_t* host_counts, void* const* host_wires,
                                const uint64_t* host_wire_capacities, uint32_t nbuckets, double ratio,
                                void* workspace, uint64_t workspace_bytes, int* status, void* stream) {
    if (!host_grads || !host_residuals || !host_counts || !host_wires || !host_wire_capacities || !workspace)
        return MCCL_HIP_ERR_ARG;
    if (nbuckets == 0 || nbuckets > kMaxListed || !(ratio > 0.0 && ratio <= 1.0)) return MCCL_HIP_ERR_ARG;
    Buckets bk = {};
    uint64_t longest = 0;
    for (uint32_t b = 0; b < nbuckets; b++) {
        if (!host_grads[b] || !host_residuals[b] || !host_wires[b] || ((uintptr_t)host_wires[b] & 3))
            return MCCL_HIP_ERR_ARG;
        if (host_counts[b] == 0 || host_counts[b] > 0xFFFFFFFFull) return MCCL_HIP_ERR_ARG;  // indices are 32-bit
        const uint32_t k = mccl_hip_topk_k(host_counts[b], ratio);
        if (host_wire_capacities[b] < 4 + 8 * (uint64_t)k) return MCCL_HIP_ERR_CAPACITY;
        bk.lgrad[b] = host_grads[b];
        bk.lresidual[b] = host_residuals[b];
        bk.lwire[b] = (uint8_t*)host_wires[b];
        bk.lcount[b] = (uint32_t)host_counts[b];
        bk.lk[b] = k;
        longest = host_counts[b] > longest ? host_counts[b] : longest;
    }
    Geometry g;
    if (!make_geometry(longest * nbuckets, longest, ratio, &g)) return MCCL_HIP_ERR_ARG;
    g.listed = 1;
    if (workspace_bytes < workspace_words(g) * 4 + 16) return MCCL_HIP_ERR_WORKSPACE;
    int rc = mccl_hip_init();
    if (rc) return rc;
    void* aligned = (void*)(((uintptr_t)workspace + 15) & ~(uintptr_t)15);
    Workspace w = carve(aligned, g);
    w.status = status;
    if (!launch_single_pass(bk, g, w, (hipStream_t)stream)) return MCCL_HIP_ERR_ARG;
    return launch_status();
}


int mccl_hip_topk_path_report(const void* workspace, uint64_t n_total, uint64_t bucket_elems, double ratio,
                              uint32_t* host_single_pass_buckets, uint32_t* host_buckets, void* stream) {
    if (!workspace || !host_single_pass_buckets || !host_buckets) return MCCL_HIP_ERR_ARG;
    Geometry g;
    if (!(ratio > 0.0 && ratio <= 1.0) || !make_geometry(n_total, bucket_elems, ratio, &g)) return MCCL_HIP_ERR_ARG;
    void* aligned = (void*)(((uintptr_t)workspace + 15) & ~(uintptr_t)15);
    Workspace w = carve(aligned, g);
    std::vector<uint32_t> st((size_t)g.nbuckets * kStateWords);
    MCCLHIP_TRY(hipMemcpyAsync(st.data(), w.state, st.size() * 4, hipMemcpyDeviceToHost, (hipStream_t)stream));
    MCCLHIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    uint32_t ok = 0;
    for (uint32_t b = 0; b < g.nbuckets; b++) {
        if (st[(size_t)b * kStateWords + S_TIMEOUT]) return MCCL_HIP_ERR_TIMEOUT;  // the payload is invalid
        ok += st[(size_t)b * kStateWords + S_OK] ? 1u : 0u;
    }
    *host_single_pass_buckets = ok;
    *host_buckets = g.nbuckets;
    return MCCL_HIP_OK;
}

}  // extern "C"

