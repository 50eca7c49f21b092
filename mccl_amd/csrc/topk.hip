// Top-k gradient sparsifier with error feedback for gfx950.
//
// Semantics (csrc/compression/TopKCompression.cpp:38-120): per bucket,
// adjusted = grad + residual; the k elements of largest |adjusted| go on the
// wire in ascending index order as [u32 k][k x {u32 index, f32 value}];
// residual = adjusted everywhere except 0.0f at the picks.  Ties at the
// threshold magnitude go to the lower index.
//
// For non-NaN floats, ordering by fabs() is ordering of the 31-bit pattern
// `key = bits & 0x7FFFFFFF`, so selection is an exact radix select on that key.
// All buckets of a gradient run in the same launches (blockIdx.y = bucket).
//
// FAST PATH (one pass over the gradient, 12 B/element of HBM traffic, three launches):
//   sample     one block per bucket loads 12,288 evenly spread elements (keys
//              stay in registers) and radix-selects three of their keys: `lo`,
//              which with 6 sigma of margin lies below the k-th largest key of
//              the bucket, `hi`, which with the same margin lies above it, and
//              the predicted threshold itself
//   pass A     residual <- grad + residual in one streaming pass, except that
//              elements at or above the predicted threshold are stored as 0.0f
//              at once; elements with key >= lo ("candidates", about 1.7 k) go,
//              in index order, to the 64 slots of their region (the 2048
//              elements one wavefront streams): no atomics, no shared lists.
//              A region with more than 64 candidates is marked dense and later
//              read from the residual itself
//   selection  (k_topk_tail) 64 blocks per bucket that meet at two counter
//              barriers; every wavefront keeps the slots of its regions in
//              registers throughout.
//              1: 256-bin histogram of the candidates, linear in the key over
//                 [lo, hi)                                          -- barrier --
//              2: the bin that holds the k-th largest key; per block the count
//                 of candidates in higher bins (picks for certain); the
//                 threshold bin's candidates (a few hundred) to list2
//                                                                   -- barrier --
//              3: every block finishes the radix select on list2: exact threshold
//                 key T, how many keys equal to T are taken and - when not all of
//                 them are - the largest index still taken
//              4: an ordered filter: each block writes its regions' picks at its
//                 offset in the payload (scan of the 64 blocks' counts) and
//                 repairs the residual where the predicted threshold and T
//                 disagree (zero a missed pick, restore a non-pick)
//              A threshold outside the window, a list2 overflow or an
//              inconsistent count hands the bucket to the exact fallback: its
//              64 blocks put the pre-zeroed values back and run the radix
//              select over the whole bucket together (three more barriers).
// EXACT PATH (any input; small buckets and topk_path = 1):
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
#include <mutex>
#include <unordered_map>
#include <vector>

namespace mcclhip {

namespace {

constexpr int kTile = 4096;    // exact path: elements per compaction tile
constexpr int kBins0 = 2048;   // key[30:20]
constexpr int kBinsR = 1024;   // key[19:10], key[9:0]
constexpr int kWinBins = 256;  // fast path: bins of the candidate window histogram
constexpr int kHistWords = kBins0 + 2 * kBinsR;
constexpr int kStateWords = 32;
constexpr int kATile = 8192;   // fast path: elements per pass-A block
constexpr int kRegion = 2048;  // fast path: elements per candidate region (one wavefront of a pass-A block)
constexpr int kRegSlots = 64;  // fast path: candidate slots per region, one per lane of the wavefront that reads it
static_assert(kATile == kRegion * (kBlock / kWave), "one region per wavefront");
static_assert(kRegSlots == kWave, "a wavefront reads a region's slots in one go");
constexpr uint32_t kDense = 0xFFFFFFFFu;  // region count: more candidates than slots, read the residual range itself
constexpr int kNSub = 64;      // fast path: blocks per bucket in the kernels that walk the regions
constexpr int kSampleThreads = 1024;  // sample kernel (256 threads measured slower: 21 vs 15.5 us)
constexpr uint64_t kFastMinBucket = 1u << 18;
constexpr int kSample = 12288;  // fast path: sampled elements per bucket (12 per select thread)

// per-bucket state words
enum {
    S_P0 = 0, S_R0 = 1,   // key prefix / picks still to place after round 0
    S_P1 = 2, S_R1 = 3,   // after round 1
    S_T = 4, S_NEED = 5,  // exact threshold key, number of keys == T that are taken
    S_LO_KEY = 6,         // fast path: candidates have key >= this
    S_HI_KEY = 11,        // fast path: keys >= this fall into the top bin of the window histogram
    S_SHIFT = 12,         // fast path: window bin = (key - lo) >> shift
    S_OK = 7,             // fast path: 1 when select succeeded for this bucket
    S_ISTAR = 8,          // fast path: ties are taken while index <= this
    S_EXACT_HIST = 9,     // 1 when hist round 0 holds the full histogram
    S_N2 = 10,            // fast path: entries in list2
    S_THAT = 13,          // fast path: predicted threshold key; pass A stores 0 for keys >= this
    S_BAR1 = 14,          // fused tail: blocks of the bucket that have flushed their histogram
    S_BAR2 = 15,          // fused tail: blocks that have published their certain picks and list2 share
    S_TIMEOUT = 16,       // fused tail: a block gave up waiting at a barrier (result invalid)
    // The window words (S_LO_KEY, S_HI_KEY, S_SHIFT, S_THAT) and the next three survive from
    // call to call: after every call they hold the window predicted for the next one.
    S_DLO = 17,           // predicted threshold minus lower window end, in key units (from the last sample)
    S_DHI = 18,           // upper window end minus predicted threshold
    S_WARM = 19,          // 1 once a call has left a prediction behind
    S_BARF = 20,          // 20..23: barriers of the in-kernel exact selection
    S_READY = 24          // one-launch path: holds the launch's epoch number once the bucket's window is published
};

// The shared description of a bucket's window, and the rule every kernel applies to
// whatever the state words hold (they may be stale or arbitrary when a caller hands
// in a workspace with foreign contents): elements are only ever stored as zero when
// they are also listed, i.e. the predicted threshold is never below the window.
struct Window {
    uint32_t lo, hi, shift, that;
    bool sound;  // bins fit the histogram; otherwise the bucket takes the exact selection
};
__device__ __forceinline__ Window load_window(const uint32_t* st) {
    Window wn;
    wn.lo = st[S_LO_KEY];
    wn.hi = st[S_HI_KEY];
    wn.shift = st[S_SHIFT];
    wn.that = st[S_THAT] < wn.lo ? wn.lo : st[S_THAT];
    wn.sound = wn.shift < 32u && wn.hi >= wn.lo && ((wn.hi - wn.lo) >> (wn.shift & 31u)) < (uint32_t)(kWinBins - 1);
    wn.shift &= 31u;
    return wn;
}
// Block (0, b) of a call's last kernel: the window for the next call, centred on this call's
// exact threshold with the widths the last sample found.
__device__ __forceinline__ void predict_next_window(uint32_t* st, uint32_t T) {
    const uint32_t dlo = st[S_DLO], dhi = st[S_DHI];
    const uint32_t lo = T > dlo ? T - dlo : 0u;
    uint32_t hi = dhi < 0x7FFFFFFFu - T ? T + dhi : 0x7FFFFFFFu;
    if (hi < lo) hi = lo;
    uint32_t shift = 0;
    while (((hi - lo) >> shift) >= (uint32_t)(kWinBins - 1)) shift++;
    st[S_LO_KEY] = lo;
    st[S_HI_KEY] = hi;
    st[S_SHIFT] = shift;
    st[S_THAT] = T < lo ? lo : T;
    st[S_WARM] = 1u;
}

struct Geometry {
    uint64_t n_total;
    uint64_t bucket_elems;
    uint32_t nbuckets;
    uint32_t tiles;    // exact-path tiles per (full) bucket
    uint32_t k_full;   // k of a bucket with bucket_elems elements
    uint32_t k_last;   // k of the last bucket
    uint32_t regions;  // fast path: candidate regions allotted per bucket
    uint32_t lcap2;    // fast path: capacity of a bucket's list2 (entries)
    uint32_t listed;   // fast path: 1 when the buckets are separate buffers (see Buckets)
    uint32_t ftiles;   // one-launch path: streaming tiles allotted per bucket
    uint32_t lcapb;    // one-launch path: capacity of one coarse bin's list (entries)
};

struct Workspace {
    // zeroed at the start of every exact-path call; the single-pass path zeroes what it uses itself
    uint32_t* hist;         // [nbuckets][kHistWords]
    uint32_t* hist_w;       // [nbuckets][kWinBins] candidates: window histogram, last bin = above the window
    uint32_t* state;        // [nbuckets][kStateWords]
    // scratch, written before read
    uint32_t* tile_gt;      // [nbuckets][tiles]
    uint32_t* tile_eq;      // [nbuckets][tiles]
    uint32_t* reg_cnt;      // [nbuckets][regions] candidates in the region's slots, or kDense
    uint32_t* list;         // [nbuckets][regions][kRegSlots][2]  (index, bits), index order
    uint32_t* list2;        // [nbuckets][lcap2][2] candidates of the threshold bin (index, key)
    uint32_t* blk_above;    // [nbuckets][kNSub] fused tail: picks above the threshold bin per block
    uint32_t* blk_eq;       // [nbuckets][kNSub] in-kernel exact selection: keys equal to the threshold per block
    // one-launch path
    uint32_t* tile_cnt;     // [nbuckets][ftiles] candidates in the tile's slots, or kDense
    uint64_t* slots;        // [nbuckets][ftiles][128] (bits << 32) | index, index order
    uint32_t* grp_cnt;      // [nbuckets][64][kCntStride] finished tiles per group (first word of each 256 bytes)
    uint32_t* ghist;        // [nbuckets][64 groups][64 bins] candidates per group and coarse window bin
    uint32_t* bin_fill;     // [nbuckets][64] entries in each coarse bin's list
    uint64_t* blist;        // [nbuckets][63][lcapb] the window's candidates by coarse bin, any order
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

// ================================= fast path ======================================

// Window bin of a candidate key: linear in the key over [lo, hi), everything
// at or above hi in bin kWinBins - 1.
__device__ __forceinline__ uint32_t window_bin(uint32_t key, uint32_t lo, uint32_t hi, uint32_t shift) {
    return key >= hi ? (uint32_t)(kWinBins - 1) : (key - lo) >> shift;
}

// One block per bucket.  Loads kSample evenly spread elements of grad + residual
// (their keys stay in registers, 12 per thread) and radix-selects (11 + 10 key
// bits, all ranks in the same sweeps) the keys of sample ranks
//     r_hi = ks - 6 sqrt(ks) - 16,   r_lo = ks + 6 sqrt(ks) + 16   and   ks,
// ks = k * S / n being the expected number of sampled elements among the top k:
// the two ends of the candidate window and the predicted threshold.
__global__ __launch_bounds__(kSampleThreads) void k_topk_sample(Buckets, Geometry g, Workspace w) {
    const BucketsArg bk = buckets_arg();
    __shared__ uint32_t lh[3][kBinsR];
    __shared__ uint32_t scratch[3 * (kSampleThreads / kWave + 2)];
    const uint32_t b = blockIdx.x;
    const uint64_t bn = bucket_count(g, bk, b);
    const float* gp = bucket_grad(g, bk, b);
    const float* rp = bucket_residual(g, bk, b);
    const uint64_t nvec = bn / 4;
    constexpr int SV = kSample / 4;               // sampled vectors
    constexpr int PV = SV / kSampleThreads;       // vectors per thread; their 4 * PV keys stay in registers
    // sampled in runs of 8 vectors (one 128-byte line per array), runs evenly spread
    const uint32_t nsv = nvec < (uint64_t)SV ? (uint32_t)(nvec & ~7ull) : (uint32_t)SV;
    const uint64_t stride = nsv ? (nvec / (nsv / 8)) : 8;  // vectors between run starts (>= 8)
    u4a gv[PV], rv[PV];
#pragma unroll
    for (int j = 0; j < PV; j++) {
        const uint32_t i = (uint32_t)j * kSampleThreads + threadIdx.x;
        const uint32_t ii = i < nsv ? i : 0;
        const uint64_t v = (uint64_t)(ii >> 3) * stride + (ii & 7);
        gv[j] = nsv ? *(const u4u4*)(gp + v * 4) : u4a{0u, 0u, 0u, 0u};
        rv[j] = nsv ? *(const u4u4*)(rp + v * 4) : u4a{0u, 0u, 0u, 0u};
    }
    // the histogram is cleared while the loads are under way
    for (int i = threadIdx.x; i < 3 * kBinsR; i += kSampleThreads) (&lh[0][0])[i] = 0;
    uint32_t key[PV][4];
    bool have[PV];
#pragma unroll
    for (int j = 0; j < PV; j++) {
        have[j] = (uint32_t)j * kSampleThreads + threadIdx.x < nsv;
#pragma unroll
        for (int q = 0; q < 4; q++) key[j][q] = key_of(u2f(gv[j][q]) + u2f(rv[j][q]));
    }
    const uint32_t S = nsv * 4;
    const float ks = (float)bucket_k(g, bk, b) * (float)S / (float)bn;
    const float margin = 6.0f * sqrtf(ks) + 16.0f;
    // ranks: 0 upper end of the window, 1 lower end, 2 the predicted threshold itself
    constexpr int NR = 3;
    uint32_t rank[NR];
    rank[0] = ks - margin >= 1.0f ? (uint32_t)(ks - margin) : 0u;  // 0: no upper end
    rank[1] = (uint32_t)(ks + margin) + 1u;                       // > S: no lower end
    rank[2] = ks >= 1.0f ? (uint32_t)ks : 1u;
    uint32_t prefix[NR] = {0u, 0u, 0u}, want[NR] = {rank[0], rank[1], rank[2]};
    const bool active[NR] = {rank[0] >= 1u && rank[0] <= S, rank[1] <= S, rank[2] <= S};
    // Two rounds, 11 + 10 key bits: the selected keys are exact to 2^-13 of their value,
    // far finer than the sampling noise the window margins allow for.  The ten low bits
    // are filled so that the window only widens.
    __syncthreads();
    for (int r = 0; r < 2; r++) {
        // round 0 uses 2048 bins: lh[0] and lh[1] are adjacent, one histogram serves all ranks
        uint32_t* h0 = &lh[0][0];
        if (r == 1) {
            for (int i = threadIdx.x; i < NR * kBinsR; i += kSampleThreads) h0[i] = 0;
            __syncthreads();
        }
#pragma unroll
        for (int j = 0; j < PV; j++) {
            if (!have[j]) continue;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t kq = key[j][q];
                if (r == 0) {
                    atomicAdd(&h0[kq >> 20], 1u);
                } else {
#pragma unroll
                    for (int z = 0; z < NR; z++)
                        if (active[z] && (kq >> 20) == (prefix[z] >> 20)) atomicAdd(&lh[z][(kq >> 10) & (kBinsR - 1)], 1u);
                }
            }
        }
        __syncthreads();
        uint32_t rem[NR], bin[NR], left[NR];
#pragma unroll
        for (int z = 0; z < NR; z++) rem[z] = active[z] ? want[z] : 0u;
        if (r == 0) {
            const uint32_t* const hs[NR] = {h0, h0, h0};
            pick_bins<kBins0, kSampleThreads, NR>(hs, rem, bin, left, scratch);
        } else {
            const uint32_t* const hs[NR] = {lh[0], lh[1], lh[2]};
            pick_bins<kBinsR, kSampleThreads, NR>(hs, rem, bin, left, scratch);
        }
#pragma unroll
        for (int z = 0; z < NR; z++) {
            if (!active[z]) continue;
            prefix[z] |= bin[z] << (r == 0 ? 20 : 10);
            want[z] = left[z];
        }
    }
    prefix[0] |= 0x3FFu;  // upper end of the window: rounded up
    prefix[2] |= 0x200u;  // predicted threshold: middle of its 1024-key cell
    if (threadIdx.x == 0) {
        const uint32_t lo = active[1] ? prefix[1] : 0u;
        uint32_t hi = active[0] ? prefix[0] : 0x7FFFFFFFu;
        if (hi < lo) hi = lo;
        uint32_t shift = 0;
        while (((hi - lo) >> shift) >= (uint32_t)(kWinBins - 1)) shift++;
        uint32_t* st = w.state + (uint64_t)b * kStateWords;
        st[S_LO_KEY] = lo;
        st[S_HI_KEY] = hi;
        st[S_SHIFT] = shift;
        // never below lo: every pre-zeroed element must be a listed candidate
        uint32_t that = active[2] ? prefix[2] : 0x7FFFFFFFu;
        if (that < lo) that = lo;
        st[S_THAT] = that;
        // widths for the predictions that follow this call
        st[S_DLO] = that - lo;
        st[S_DHI] = hi > that ? hi - that : 0u;
        st[S_WARM] = 1u;
    }
}

// ---- candidate regions ------------------------------------------------------------
// A region is the kRegion consecutive elements one wavefront of a pass-A block
// streams.  Its candidates land, in index order, in the region's kRegSlots slots
// of `list` (slot = lane of the wave that later reads it) and their number in
// reg_cnt.  A region with more candidates than slots is marked kDense: readers
// then take every element of the region's residual range as a candidate.  No
// atomics and no shared capacity are involved, so nothing can overflow.

// The regions [r0, r1) of bucket b that block s of kNSub works on.
__device__ __forceinline__ void block_regions(const Geometry& g, BucketsArg bk, uint32_t b, uint32_t s,
                                              uint32_t* r0, uint32_t* r1) {
    const uint32_t nreg = (uint32_t)((bucket_count(g, bk, b) + kRegion - 1) / kRegion);
    const uint32_t per = (nreg + kNSub - 1) / kNSub;
    *r0 = s * per < nreg ? s * per : nreg;
    *r1 = *r0 + per < nreg ? *r0 + per : nreg;
}

// residual <- grad + residual; candidates (key >= lo) are written to their
// region.  One 8192-element tile per block, tiles in address order, one region
// per wavefront.  Elements at or above the predicted threshold are stored as
// 0.0f straight away (their values are in the region's list): a million
// scattered 4-byte stores after the selection cost more than a tenth of the
// whole compress, while the streaming store here is free; emit only repairs
// the few elements between the predicted and the true threshold.  A region
// that turns out dense puts its values back and stores plain sums from then on.
// Nothing else happens here: returning atomics and histogram flushes in these
// 12,000 streaming blocks each cost 7-15 % of the kernel's time when they were
// tried.
constexpr int kAWaves = kATile / kRegion;  // wavefronts (= regions) per streaming block; 1, 2 and 8 measured the same or worse
constexpr int kAThreads = kAWaves * kWave;
__global__ __launch_bounds__(kAThreads) void k_topk_pass_a_fast(Buckets, Geometry g, Workspace w) {
    const BucketsArg bk = buckets_arg();
    __shared__ __attribute__((aligned(16))) uint32_t stage[kAWaves][kRegSlots][2];
    const uint32_t b = blockIdx.y, t = blockIdx.x;
    const uint64_t bn = bucket_count(g, bk, b);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint64_t w0 = (uint64_t)t * kATile + (uint64_t)wave * kRegion;  // first element of this wave's region
    if (t == 0) {
        // the words the selection kernel accumulates into start every call at zero
        for (int i = threadIdx.x; i < kWinBins; i += kAThreads) w.hist_w[(uint64_t)b * kWinBins + i] = 0;
        if (threadIdx.x == 0) {
            uint32_t* st = w.state + (uint64_t)b * kStateWords;
            st[S_BAR1] = 0; st[S_BAR2] = 0; st[S_N2] = 0; st[S_OK] = 0; st[S_TIMEOUT] = 0;
            st[S_BARF] = 0; st[S_BARF + 1] = 0; st[S_BARF + 2] = 0; st[S_BARF + 3] = 0;
        }
        for (int i = threadIdx.x; i < kHistWords; i += kAThreads) w.hist[(uint64_t)b * kHistWords + i] = 0;
    }
    if (w0 >= bn) return;  // whole wavefront; the kernel has no barriers
    const float* gp = bucket_grad(g, bk, b) + w0;
    float* rp = bucket_residual(g, bk, b) + w0;
    constexpr int U = 2;
    constexpr int ROUNDS = kRegion / (kWave * 4 * U);
    const uint32_t len = (uint32_t)((bn - w0) < (uint64_t)kRegion ? (bn - w0) : (uint64_t)kRegion);
    const uint32_t nfull = len / 4;  // full vectors in this region
    // The streaming loads of a round are issued one round ahead: round 0's before
    // the bucket parameters are read, round r+1's before round r is processed.
    u4a gv[ROUNDS][U], rv[ROUNDS][U];
    auto issue = [&](int round) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t vi = (uint32_t)(round * U + u) * kWave + lane;
            if (vi < nfull) {
                gv[round][u] = __builtin_nontemporal_load((const u4u4*)(gp + vi * 4));
                rv[round][u] = __builtin_nontemporal_load((const u4u4*)(rp + vi * 4));
            }
        }
    };
    issue(0);
    const Window wn = load_window(w.state + (uint64_t)b * kStateWords);
    const uint32_t lo_key = wn.lo, that_key = wn.that;
    // both the same in every lane, and kept in scalar registers by saying so at every update
    uint32_t staged = 0;  // candidates of the region so far
    uint32_t dense = 0;   // 1: more candidates than slots
    u2a* const slots = (u2a*)&stage[wave][0][0];
    // lanes of `m` below this one
    auto lanes_below = [&](uint64_t m) {
        return (uint32_t)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
    };
    auto pick = [](const u4a& a, uint32_t q) {
        uint32_t v = a[0];
        v = q == 1 ? a[1] : v;
        v = q == 2 ? a[2] : v;
        return q == 3 ? a[3] : v;
    };

    // Appends the lanes' candidates (mask4: which of a lane's four elements) in
    // index order: lane-major, element-minor.  Nearly every call finds a few lanes
    // with one candidate each: one ballot, one 8-byte LDS store.  Lanes with
    // several candidates (about one call in ten has one) take the branch that
    // counts them level by level and stores the rest in a loop.
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
        if (staged + total > (uint32_t)kRegSlots) {
            // the region goes dense: its earlier candidates were stored as zeros where
            // they reached the predicted threshold; put those values back
            dense = 1u;
            if ((uint32_t)lane < staged && (stage[wave][lane][1] & 0x7FFFFFFFu) >= that_key)
                bucket_residual(g, bk, b)[stage[wave][lane][0]] = u2f(stage[wave][lane][1]);
            return;
        }
        if (mask4) {
            uint32_t pos = staged + before;
            const uint32_t q = (uint32_t)__ffs((int)mask4) - 1u;
            slots[pos] = u2a{first_idx + q, pick(a, q)};
            uint32_t rest = mask4 & (mask4 - 1u);
            while (rest) {
                const uint32_t q2 = (uint32_t)__ffs((int)rest) - 1u;
                slots[++pos] = u2a{first_idx + q2, pick(a, q2)};
                rest &= rest - 1u;
            }
        }
        staged = (uint32_t)__builtin_amdgcn_readfirstlane((int)(staged + total));
    };

#pragma unroll
    for (int round = 0; round < ROUNDS; round++) {
        if (round + 1 < ROUNDS) issue(round + 1);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t vi = (uint32_t)(round * U + u) * kWave + lane;
            u4a a = {0u, 0u, 0u, 0u}, z = {0u, 0u, 0u, 0u};
            uint32_t mask4 = 0;
            if (vi < nfull) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float adj = u2f(gv[round][u][q]) + u2f(rv[round][u][q]);
                    a[q] = f2u(adj);
                    z[q] = key_of(adj) >= that_key ? 0u : a[q];
                    mask4 |= (key_of(adj) >= lo_key ? 1u : 0u) << q;
                }
            }
            append(mask4, a, (uint32_t)w0 + vi * 4);  // may turn the region dense
            if (vi < nfull) __builtin_nontemporal_store(dense ? a : z, (u4u4*)(rp + vi * 4));
        }
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
                rp[nfull * 4 + q] = (!dense && (a[q] & 0x7FFFFFFFu) >= that_key) ? 0.0f : u2f(a[q]);
        }
    }
    const uint32_t region = (uint32_t)(w0 / kRegion);
    if (!dense && (uint32_t)lane < staged) {
        const u2a e = slots[lane];
        *(u2a*)(w.list + (((uint64_t)b * g.regions + region) * kRegSlots + lane) * 2) = e;
    }
    if (lane == 0) w.reg_cnt[(uint64_t)b * g.regions + region] = dense ? kDense : staged;
}

// ================================ fused tail ======================================
// Everything after the streaming pass in one launch: window histogram, threshold
// bin, exact threshold, tie-break, payload offsets and the payload itself.  The
// kNSub blocks that work on one bucket meet at two barriers (the histogram is
// complete; the threshold bin's candidates and the blocks' certain-pick counts
// are published); nothing else crosses blocks.  Each wavefront owns a contiguous
// run of regions and keeps their slots in registers across the phases, so the
// candidate lists are read from memory once.
//
// Barrier: a per-bucket arrival counter in the state words (zero at kernel
// start).  A block's 64 partners are the blocks next to it in dispatch order, so
// they are resident or about to be; the wait is bounded all the same: a block
// that waits longer than `limit_ticks` of the 100 MHz wall clock records
// S_TIMEOUT and leaves, and the call's result for that bucket is then invalid
// (mccl_hip_topk_path_report returns an error).

constexpr int kTailRegs = 14;  // regions per wavefront whose slots stay in registers

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

// Dense regions (more candidates than slots) are rare.  Every sweep of the tail
// kernel handles them in a compact loop of its own after the unrolled sweep over
// the wavefront's register-held regions, so the common path stays small.
// Calls f(index, bits, in_range) for every element of dense region r, 64 elements
// per step, every lane of the wavefront taking part in every step; the loads of
// 16 steps are in flight together and parked in LDS, so the code stays a loop.
template <class F>
__device__ __forceinline__ void dense_walk(const float* rp, uint64_t bn, uint32_t r, uint32_t* buf /* 1024 words of LDS per wavefront */,
                                           F&& f) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t e0 = (uint64_t)r * kRegion;
    const uint64_t e1 = e0 + kRegion < bn ? e0 + kRegion : bn;
    constexpr int B = 16;
#pragma unroll 1
    for (uint64_t base = e0; base < e1; base += (uint64_t)B * kWave) {
        uint32_t v[B];
#pragma unroll
        for (int j = 0; j < B; j++) {
            const uint64_t i = base + (uint64_t)j * kWave + lane;
            v[j] = i < e1 ? f2u(rp[i]) : 0u;
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

// The need-th smallest index among list2's entries with key == T (ties at the
// threshold go to the lower index): radix select over the index, 11 + 11 + 10 bits.
// Called by all threads of the block.
__device__ __forceinline__ uint32_t resolve_ties(const uint32_t* l2, uint32_t count2, uint32_t T, uint32_t need,
                                              uint32_t* lh /* kBins0 words */, uint32_t* scratch) {
    uint32_t iwant = need, iprefix = 0;
    const int shifts[3] = {21, 10, 0};
    const int widths[3] = {11, 11, 10};
    for (int r = 0; r < 3; r++) {
        const int bins = 1 << widths[r];
        for (int i = threadIdx.x; i < kBins0; i += kBlock) lh[i] = 0;
        __syncthreads();
        const int hs = shifts[r] + widths[r];
        for (uint32_t i = threadIdx.x; i < count2; i += kBlock) {
            const uint32_t idx = ld_agent(&l2[2 * (uint64_t)i]), key = ld_agent(&l2[2 * (uint64_t)i + 1]);
            const bool match = hs >= 32 ? true : ((idx >> hs) == (iprefix >> hs));
            // bins stored reversed, so that pick_bin's top-down scan runs over ascending indices
            if (key == T && match) atomicAdd(&lh[(bins - 1) - ((idx >> shifts[r]) & (bins - 1))], 1u);
        }
        __syncthreads();
        uint32_t left;
        // a 1024-bin round leaves the upper half of the 2048 bins empty: one scan serves both widths
        const uint32_t rb = pick_bin<kBins0, kBlock>(lh, iwant, 0, &left, scratch);
        iprefix |= ((uint32_t)(bins - 1) - (rb - (uint32_t)(kBins0 - bins))) << shifts[r];
        iwant = left;
    }
    return iprefix;
}

// The exact selection of one bucket by the kNSub blocks that work on it: the
// fallback for a bucket whose window could not finish the selection (too few
// candidates, threshold outside the window, a threshold bin with more keys than
// list2 holds).  No extra launch; every block of the bucket enters it together.
//   1  each block puts back, in its own regions, what the streaming pass stored as 0.0f
//   2  three radix rounds over the key (11 + 10 + 10 bits): a block histograms its
//      own slice of the bucket in LDS and adds it to the bucket's histogram; after
//      a barrier every block scans that histogram and gets the same digit
//   3  a block counts the keys above and at the threshold in its slice; after a
//      barrier every block knows how many picks precede its slice
//   4  a block writes its slice's picks in index order and zeroes them
// A block only ever reads the residual range it restored itself, so the residual
// needs no exchange between blocks.  lh: kBins0 words, scratch: kBlock / kWave + 2
// words, flag: one word of LDS.  Returns false when a barrier wait timed out;
// *T_out receives the exact threshold key.
__device__ __forceinline__ bool bucket_exact_group(BucketsArg bk, const Geometry& g, const Workspace& w,
                                                   uint32_t b, uint32_t s, const Window& wn, uint32_t* lh,
                                                   uint32_t* scratch, uint32_t* flag, uint64_t limit_ticks,
                                                   uint32_t* T_out) {
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const uint64_t bn = bucket_count(g, bk, b);
    float* rp = bucket_residual(g, bk, b);
    uint32_t r0, r1;
    block_regions(g, bk, b, s, &r0, &r1);
    const uint64_t e0 = (uint64_t)r0 * kRegion;
    const uint64_t e1 = (uint64_t)r1 * kRegion < bn ? (uint64_t)r1 * kRegion : bn;
    // 1: this block's regions
    {
        const uint32_t* rc = w.reg_cnt + (uint64_t)b * g.regions;
        const uint32_t* lb = w.list + (uint64_t)b * g.regions * kRegSlots * 2;
        for (uint32_t slot = r0 * kRegSlots + threadIdx.x; slot < r1 * kRegSlots; slot += kBlock) {
            const uint32_t cnt = rc[slot / kRegSlots];
            if (cnt == kDense || (slot % kRegSlots) >= cnt) continue;
            const uint32_t idx = lb[2 * (uint64_t)slot], bitsv = lb[2 * (uint64_t)slot + 1];
            if ((bitsv & 0x7FFFFFFFu) >= wn.that) rp[idx] = u2f(bitsv);
        }
        __syncthreads();
    }
    // 2: radix select.  Every wavefront walks a contiguous quarter of the block's slice,
    // 64 elements per step with the loads of eight steps in flight; f(i, bits, valid) is
    // called by all lanes of the wavefront for every step.
    constexpr int NW = kBlock / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
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
    uint32_t* gh = w.hist + (uint64_t)b * kHistWords;  // zero at kernel start
    uint32_t prefix = 0, remaining = bucket_k(g, bk, b);
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
        if (!bucket_barrier(st + S_BARF + round, kNSub, flag, limit_ticks)) return false;
        for (int i = threadIdx.x; i < bins; i += kBlock) lh[i] = ld_agent(&ghr[i]);
        __syncthreads();
        uint32_t left, bin;
        if (round == 0) bin = pick_bin<kBins0, kBlock>(lh, remaining, 0, &left, scratch);
        else bin = pick_bin<kBinsR, kBlock>(lh, remaining, 0, &left, scratch);
        prefix |= bin << shift;
        remaining = left;
    }
    const uint32_t T = prefix, need = remaining;
    // 3: keys above and at the threshold per wavefront range, per block, and in the slices before
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
        st_agent(&w.blk_above[(uint64_t)b * kNSub + s], gt_blk);
        st_agent(&w.blk_eq[(uint64_t)b * kNSub + s], eq_blk);
    }
    if (!bucket_barrier(st + S_BARF + 3, kNSub, flag, limit_ticks)) return false;
    {
        static_assert(kNSub <= kBlock, "one thread per block of the bucket");
        const uint32_t vg = threadIdx.x < s ? ld_agent(&w.blk_above[(uint64_t)b * kNSub + threadIdx.x]) : 0u;
        const uint32_t ve = threadIdx.x < s ? ld_agent(&w.blk_eq[(uint64_t)b * kNSub + threadIdx.x]) : 0u;
        uint32_t gt_before, eq_before;
        block_exclusive_scan(vg, scratch, &gt_before);
        block_exclusive_scan(ve, scratch, &eq_before);
        gt_run += gt_before;
        eq_run += eq_before;
    }
    // 4: this wavefront's picks, in index order: an element lands at (keys above T before it)
    // + min(keys equal to T before it, need); ties are taken while fewer than need came before
    uint32_t* out = bucket_wire(g, bk, b);
    if (s == 0 && threadIdx.x == 0) out[0] = bucket_k(g, bk, b);
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
    *T_out = T;
    return true;
}

__global__ __launch_bounds__(kBlock, 4) void k_topk_tail(Buckets, Geometry g, Workspace w, uint64_t limit_ticks) {
    const BucketsArg bk = buckets_arg();
    constexpr int NW = kBlock / kWave;
    __shared__ uint32_t lh[kBins0];
    __shared__ uint32_t scratch[NW + 2];
    __shared__ uint32_t sh_a[NW], sh_b[NW], sh_x[2];
    __shared__ uint32_t rcnt[NW][kTailRegs];  // phase 4: picks per register-held region
    __shared__ uint32_t dbuf[NW][16 * kWave];  // dense_walk's staging area, one per wavefront
    const uint32_t b = blockIdx.y, s = blockIdx.x;
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const Window wn = load_window(st);
    const uint32_t lo = wn.lo, hi = wn.hi, shift = wn.shift, that_key = wn.that;
    const uint32_t k = bucket_k(g, bk, b);
    const uint64_t bn = bucket_count(g, bk, b);
    uint32_t r0, r1;
    block_regions(g, bk, b, s, &r0, &r1);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
    // this wavefront's regions: a contiguous quarter of the block's
    const uint32_t pw = (r1 - r0 + NW - 1) / NW;
    const uint32_t wr0 = r0 + wave * pw < r1 ? r0 + wave * pw : r1;
    const uint32_t wr1 = wr0 + pw < r1 ? wr0 + pw : r1;
    const uint32_t* rc = w.reg_cnt + (uint64_t)b * g.regions;
    const uint32_t* lb = w.list + (uint64_t)b * g.regions * kRegSlots * 2;
    float* rp = bucket_residual(g, bk, b);
    uint32_t* hw = w.hist_w + (uint64_t)b * kWinBins;
    uint32_t* l2 = w.list2 + (uint64_t)b * g.lcap2 * 2;
    uint32_t* above_of = w.blk_above + (uint64_t)b * kNSub;
    uint32_t* out = bucket_wire(g, bk, b);

    // ---- slots of the first kTailRegs regions into registers, every load issued at once
    uint32_t ccnt[kTailRegs], cidx[kTailRegs], cbits[kTailRegs];
#pragma unroll
    for (int q = 0; q < kTailRegs; q++) {
        const uint32_t r = wr0 + q < wr1 ? wr0 + q : (wr1 > wr0 ? wr1 - 1 : 0);  // stays inside the bucket's lists
        ccnt[q] = rc[r];
        const u2a e = *(const u2a*)(lb + 2 * ((uint64_t)r * kRegSlots + lane));  // slots past the count: ignored below
        cidx[q] = e[0];
        cbits[q] = e[1];
    }
    bool any_dense = false;  // wave-uniform: one of the register-held regions is dense
#pragma unroll
    for (int q = 0; q < kTailRegs; q++) any_dense |= wr0 + q < wr1 && ccnt[q] == kDense;

    // A sweep = nd(q, r, cnt, idx, bits) for every ordinary region (q < kTailRegs: register-held,
    // else ~0u), dn(q, r) for every dense one.  Order: register-held ordinary regions first, then
    // the dense ones and those past the register window, in index order.
    const bool more = any_dense || wr1 > wr0 + kTailRegs;  // wave-uniform
    auto sweep = [&](auto&& nd, auto&& dn) {
#pragma unroll
        for (int q = 0; q < kTailRegs; q++)
            if (wr0 + q < wr1 && ccnt[q] != kDense) nd((uint32_t)q, wr0 + q, ccnt[q], cidx[q], cbits[q]);
        if (more) {
#pragma unroll 1
            for (uint32_t r = wr0; r < wr1; r++) {
                const uint32_t q = r - wr0 < (uint32_t)kTailRegs ? r - wr0 : ~0u;
                const uint32_t cnt = rc[r];
                if (cnt == kDense) {
                    dn(q, r);
                } else if (q == ~0u) {
                    const u2a e = *(const u2a*)(lb + 2 * ((uint64_t)r * kRegSlots + lane));
                    nd(q, r, cnt, e[0], e[1]);
                }
            }
        }
    };
    // Reasons to hand the bucket to the exact selection are collected in `failed`
    // (block-uniform, and the same in every block of the bucket); the one call sits
    // at the end of the kernel.
    bool failed = false;

    // ---- phase 1: window histogram -------------------------------------------------
    // (A window that does not fit the histogram - only possible when the state words hold
    // foreign contents - skips the work but not the barrier: a block that reaches the end
    // of the kernel may rewrite the window, so every block must have read it by then.)
    for (int i = threadIdx.x; i < kWinBins; i += kBlock) lh[i] = 0;
    __syncthreads();
    if (wn.sound)
    sweep([&](uint32_t, uint32_t, uint32_t cnt, uint32_t, uint32_t bitsv) {
              if ((uint32_t)lane < cnt) atomicAdd(&lh[window_bin(bitsv & 0x7FFFFFFFu, lo, hi, shift)], 1u);
          },
          [&](uint32_t, uint32_t r) {
              dense_walk(rp, bn, r, dbuf[wave], [&](uint32_t, uint32_t v, bool in) {
                  const uint32_t key = v & 0x7FFFFFFFu;
                  const bool cand = in && key >= lo;
                  wave_hist_add(lh, cand, cand ? window_bin(key, lo, hi, shift) : 0u);
              });
          });
    __syncthreads();
    for (int i = threadIdx.x; i < kWinBins; i += kBlock) {
        const uint32_t c = lh[i];
        if (c) __hip_atomic_fetch_add(&hw[i], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!bucket_barrier(st + S_BAR1, kNSub, &sh_x[0], limit_ticks)) {
        if (threadIdx.x == 0) st_agent(st + S_TIMEOUT, 1u);
        return;
    }

    do {
    if (!wn.sound) {
        failed = true;
        break;
    }
    // ---- phase 2: threshold bin; certain picks per block; the bin's candidates to list2
    for (int i = threadIdx.x; i < kWinBins; i += kBlock) lh[i] = ld_agent(&hw[i]);
    __syncthreads();
    uint32_t need;
    const uint32_t jstar = pick_bin<kWinBins, kBlock>(lh, k, 0, &need, scratch);
    if (jstar >= (uint32_t)(kWinBins - 1)) {  // fewer than k candidates, or the threshold lies above the window
        failed = true;
        break;
    }
    uint32_t w_above = 0, w_hits = 0;
    sweep([&](uint32_t, uint32_t, uint32_t cnt, uint32_t, uint32_t bitsv) {
              const bool valid = (uint32_t)lane < cnt;
              const uint32_t bin = valid ? window_bin(bitsv & 0x7FFFFFFFu, lo, hi, shift) : 0u;
              w_above += (uint32_t)__popcll(__ballot(valid && bin > jstar));
              w_hits += (uint32_t)__popcll(__ballot(valid && bin == jstar));
          },
          [&](uint32_t, uint32_t r) {
              dense_walk(rp, bn, r, dbuf[wave], [&](uint32_t, uint32_t v, bool in) {
                  const uint32_t key = v & 0x7FFFFFFFu;
                  const bool cand = in && key >= lo;
                  const uint32_t bin = cand ? window_bin(key, lo, hi, shift) : 0u;
                  w_above += (uint32_t)__popcll(__ballot(cand && bin > jstar));
                  w_hits += (uint32_t)__popcll(__ballot(cand && bin == jstar));
              });
          });
    if (lane == 0) { sh_a[wave] = w_above; sh_b[wave] = w_hits; }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t ta = 0, th = 0;
#pragma unroll
        for (int i = 0; i < NW; i++) { ta += sh_a[i]; th += sh_b[i]; }
        st_agent(&above_of[s], ta);
        sh_x[1] = th ? __hip_atomic_fetch_add(st + S_N2, th, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    }
    __syncthreads();
    if (w_hits) {  // wave-uniform; list2's order does not matter
        uint32_t pos = sh_x[1];
        for (int i = 0; i < wave; i++) pos += sh_b[i];
        auto put = [&](bool hit, uint32_t idx, uint32_t key) {
            const uint64_t m = __ballot(hit);
            if (hit) {
                const uint32_t p = pos + (uint32_t)__popcll(m & below);
                if (p < g.lcap2) {
                    st_agent(&l2[2 * (uint64_t)p], idx);
                    st_agent(&l2[2 * (uint64_t)p + 1], key);
                }
            }
            pos += (uint32_t)__popcll(m);
        };
        sweep([&](uint32_t, uint32_t, uint32_t cnt, uint32_t idx, uint32_t bitsv) {
                  const uint32_t key = bitsv & 0x7FFFFFFFu;
                  put((uint32_t)lane < cnt && window_bin(key, lo, hi, shift) == jstar, idx, key);
              },
              [&](uint32_t, uint32_t r) {
                  dense_walk(rp, bn, r, dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                      const uint32_t key = v & 0x7FFFFFFFu;
                      put(in && key >= lo && window_bin(key, lo, hi, shift) == jstar, i, key);
                  });
              });
    }
    if (!bucket_barrier(st + S_BAR2, kNSub, &sh_x[0], limit_ticks)) {
        if (threadIdx.x == 0) st_agent(st + S_TIMEOUT, 1u);
        return;
    }

    // ---- phase 3: exact threshold from list2 (every block, redundantly) -----------------
    // every load of this phase is issued at once: the entries do not wait for their count
    // (slots past it hold leftovers and are masked below)
    constexpr int kL2Regs = 4;  // list2 entries per thread kept in registers (1024 per block)
    uint32_t eidx[kL2Regs], ekey[kL2Regs];
#pragma unroll
    for (int j = 0; j < kL2Regs; j++) {
        const uint32_t i = (uint32_t)j * kBlock + threadIdx.x;
        eidx[j] = i < g.lcap2 ? ld_agent(&l2[2 * (uint64_t)i]) : 0u;
        ekey[j] = i < g.lcap2 ? ld_agent(&l2[2 * (uint64_t)i + 1]) : 0u;
    }
    const uint32_t above_mine = threadIdx.x < (uint32_t)kNSub ? ld_agent(&above_of[threadIdx.x]) : 0u;
    const uint32_t count2 = ld_agent(st + S_N2);
    if (count2 > g.lcap2) {  // more keys in the threshold bin than list2 holds (heavy ties)
        failed = true;
        break;
    }
    auto for_list2 = [&](auto&& body) {
#pragma unroll
        for (int j = 0; j < kL2Regs; j++)
            if ((uint32_t)j * kBlock + threadIdx.x < count2) body(eidx[j], ekey[j]);
#pragma unroll 1
        for (uint32_t i = kL2Regs * kBlock + threadIdx.x; i < count2; i += kBlock)
            body(ld_agent(&l2[2 * (uint64_t)i]), ld_agent(&l2[2 * (uint64_t)i + 1]));
    };
    const uint32_t bin_lo = lo + (jstar << shift);  // smallest key of the threshold bin
    uint32_t vprefix = 0, want = need;              // key - bin_lo: up to 30 bits, selected as 10 + 10 + 10
    // a window bin spans 2^shift keys: rounds whose digits lie wholly above that are skipped
    const int first_round = shift <= 10 ? 2 : (shift <= 20 ? 1 : 0);
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
        uint32_t left;
        const uint32_t bin = pick_bin<kBinsR, kBlock>(lh, want, 0, &left, scratch);
        vprefix |= bin << sh;
        want = left;
    }
    const uint32_t T = bin_lo + vprefix;
    const uint32_t need2 = want;
    const uint32_t ties = lh[vprefix & (kBinsR - 1)];
    __syncthreads();
    // when only some keys equal to T are taken, they are the need2 lowest indices
    const uint32_t istar = ties != need2 ? resolve_ties(l2, count2, T, need2, lh, scratch) : 0xFFFFFFFFu;
    auto is_pick = [&](bool valid, uint32_t key, uint32_t idx) {
        return valid && (key > T || (key == T && idx <= istar));
    };
    // picks before this block's first element: the earlier blocks' certain picks and the
    // threshold bin's picks at lower indices
    uint32_t mine_before = 0, mine_all = 0;
    const uint64_t first_elem = (uint64_t)r0 * kRegion;
    for_list2([&](uint32_t idx, uint32_t key) {
        if (is_pick(true, key, idx)) {
            mine_all++;
            mine_before += (uint64_t)idx < first_elem ? 1u : 0u;
        }
    });
    uint32_t l2_before, l2_total, above_before, above_total;
    block_exclusive_scan(mine_before, scratch, &l2_before);
    block_exclusive_scan(mine_all, scratch, &l2_total);
    block_exclusive_scan(threadIdx.x < s ? above_mine : 0u, scratch, &above_before);
    block_exclusive_scan(above_mine, scratch, &above_total);
    if (above_total + l2_total != k) {  // cannot happen with consistent lists
        failed = true;
        break;
    }

    // ---- phase 4: payload, in index order -----------------------------------------------
    // picks per region first: the register-held regions' into rcnt, the others' into a total
    uint32_t w_total = 0;
    sweep([&](uint32_t q, uint32_t, uint32_t cnt, uint32_t idx, uint32_t bitsv) {
              const uint32_t c = (uint32_t)__popcll(__ballot(is_pick((uint32_t)lane < cnt, bitsv & 0x7FFFFFFFu, idx)));
              if (q != ~0u) rcnt[wave][q] = c;
              w_total += c;
          },
          [&](uint32_t q, uint32_t r) {
              uint32_t c = 0;
              dense_walk(rp, bn, r, dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
                  c += (uint32_t)__popcll(__ballot(is_pick(in, v & 0x7FFFFFFFu, i)));
              });
              if (q != ~0u) rcnt[wave][q] = c;
              w_total += c;
          });
    if (lane == 0) sh_a[wave] = w_total;
    __syncthreads();
    uint32_t wave_off = above_before + l2_before;
    for (int i = 0; i < wave; i++) wave_off += sh_a[i];
    auto emit_dense = [&](uint32_t r, uint32_t pos) {
        dense_walk(rp, bn, r, dbuf[wave], [&](uint32_t i, uint32_t v, bool in) {
            const bool pick = is_pick(in, v & 0x7FFFFFFFu, i);
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
    auto emit_region = [&](uint32_t cnt, uint32_t idx, uint32_t bitsv, uint32_t pos) {
        const bool valid = (uint32_t)lane < cnt;
        const uint32_t key = bitsv & 0x7FFFFFFFu;
        const bool pick = is_pick(valid, key, idx);
        const uint64_t m = __ballot(pick);
        if (pick) {
            const u2a e = {idx, bitsv};
            *(u2a4*)(out + 1 + 2 * (uint64_t)(pos + (uint32_t)__popcll(m & below))) = e;
        }
        // pass A stored 0.0f for key >= predicted threshold; repair where the prediction was wrong
        if (valid && pick != (key >= that_key)) rp[idx] = pick ? 0.0f : u2f(bitsv);
        return pos + (uint32_t)__popcll(m);
    };
    {
        uint32_t pos = wave_off;
#pragma unroll
        for (int q = 0; q < kTailRegs; q++) {
            if (wr0 + q < wr1) {
                if (ccnt[q] != kDense) pos = emit_region(ccnt[q], cidx[q], cbits[q], pos);
                else pos += rcnt[wave][q];  // written out by the loop below
            }
        }
    }
    if (more) {
        uint32_t pos = wave_off;
#pragma unroll 1
        for (uint32_t r = wr0; r < wr1; r++) {
            const uint32_t cnt = rc[r];
            if (cnt == kDense) {
                pos = emit_dense(r, pos);
            } else if (r - wr0 < (uint32_t)kTailRegs) {
                pos += rcnt[wave][r - wr0];
            } else {
                const u2a e = *(const u2a*)(lb + 2 * ((uint64_t)r * kRegSlots + lane));
                pos = emit_region(cnt, e[0], e[1], pos);
            }
        }
    }
    if (s == 0 && threadIdx.x == 0) {
        out[0] = k;
        st[S_T] = T;
        st[S_NEED] = need2;
        st[S_ISTAR] = istar;
        st[S_OK] = 1u;
        predict_next_window(st, T);
    }
    } while (false);
    // the exact selection for a bucket the window could not finish (S_OK stays 0)
    if (failed) {
        uint32_t T;
        if (!bucket_exact_group(bk, g, w, b, s, wn, lh, scratch, &sh_x[0], limit_ticks, &T)) {
            if (threadIdx.x == 0) st_agent(st + S_TIMEOUT, 1u);
            return;
        }
        if (s == 0 && threadIdx.x == 0) predict_next_window(st, T);
    }
}

#include "topk_fused.hip.h"

// ================================ host side =======================================

uint64_t align4(uint64_t words) { return (words + 3) & ~uint64_t(3); }

uint64_t zeroed_words(const Geometry& g) {
    return align4((uint64_t)g.nbuckets * kHistWords) + align4((uint64_t)g.nbuckets * kWinBins) +
           align4((uint64_t)g.nbuckets * kStateWords);
}

uint64_t workspace_words(const Geometry& g) {
    return zeroed_words(g) + 2 * align4((uint64_t)g.nbuckets * g.tiles) +
           align4((uint64_t)g.nbuckets * g.regions) +
           align4((uint64_t)g.nbuckets * g.regions * kRegSlots * 2) + align4((uint64_t)g.nbuckets * g.lcap2 * 2) +
           2 * align4((uint64_t)g.nbuckets * kNSub) +
           align4((uint64_t)g.nbuckets * g.ftiles) + align4((uint64_t)g.nbuckets * g.ftiles * kTileSlots * 2) +
           align4((uint64_t)g.nbuckets * kGroups * kCntStride) + align4((uint64_t)g.nbuckets * kGroups * kCoarse) +
           align4((uint64_t)g.nbuckets * kCoarse) + align4((uint64_t)g.nbuckets * (kCoarse - 1) * g.lcapb * 2);
}

Workspace carve(void* base, const Geometry& g) {
    Workspace w;
    uint32_t* p = (uint32_t*)base;
    w.hist = p;        p += align4((uint64_t)g.nbuckets * kHistWords);
    w.hist_w = p;      p += align4((uint64_t)g.nbuckets * kWinBins);
    w.state = p;       p += align4((uint64_t)g.nbuckets * kStateWords);
    w.tile_gt = p;     p += align4((uint64_t)g.nbuckets * g.tiles);
    w.tile_eq = p;     p += align4((uint64_t)g.nbuckets * g.tiles);
    w.reg_cnt = p;     p += align4((uint64_t)g.nbuckets * g.regions);
    w.list = p;        p += align4((uint64_t)g.nbuckets * g.regions * kRegSlots * 2);
    w.list2 = p;       p += align4((uint64_t)g.nbuckets * g.lcap2 * 2);
    w.blk_above = p;   p += align4((uint64_t)g.nbuckets * kNSub);
    w.blk_eq = p;      p += align4((uint64_t)g.nbuckets * kNSub);
    w.tile_cnt = p;    p += align4((uint64_t)g.nbuckets * g.ftiles);
    w.slots = (uint64_t*)p;  p += align4((uint64_t)g.nbuckets * g.ftiles * kTileSlots * 2);
    w.grp_cnt = p;     p += align4((uint64_t)g.nbuckets * kGroups * kCntStride);
    w.ghist = p;       p += align4((uint64_t)g.nbuckets * kGroups * kCoarse);
    w.bin_fill = p;    p += align4((uint64_t)g.nbuckets * kCoarse);
    w.blist = (uint64_t*)p;
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
    g->regions = (uint32_t)((bucket_elems + kATile - 1) / kATile) * (kATile / kRegion);
    // list2 holds the candidates of one window bin (1/256 of about 1.7 k in the expected
    // case); 2 k + 4096 entries leave room for heavy ties, never more than the bucket
    uint64_t cap = 2 * (uint64_t)g->k_full + 4096;
    if (cap > bucket_elems) cap = bucket_elems;
    g->lcap2 = (uint32_t)cap;
    g->listed = 0;
    g->ftiles = (uint32_t)((bucket_elems + kFTile - 1) / kFTile);
    // a coarse bin holds about k / 40 candidates when the window is as wide as a sample of
    // 8192 leaves it; k / 8 + 2048 entries leave room for uneven bins
    uint64_t capb = (uint64_t)g->k_full / 8 + 2048;
    if (capb > bucket_elems) capb = bucket_elems;
    g->lcapb = (uint32_t)capb;
    return true;
}

std::atomic<uint32_t> g_epoch{0x5EED0001u};

// The three launches of the single-pass path, or the one launch that does the same.
void launch_single_pass(const Buckets& bk, const Geometry& g, const Workspace& w, bool warm, hipStream_t st) {
    // the streaming launch: a sample block per bucket, then per bucket its tiles and 64 bin blocks
    const uint64_t blocks = (uint64_t)g.nbuckets * ((uint64_t)g.ftiles + kGroups + 1) + kGroups;
    if (tuning().topk_fused && blocks < 0x7FFFFFFFull) {
        uint32_t epoch = ++g_epoch;
        if (epoch == 0) epoch = ++g_epoch;  // zero is what a finished call leaves in S_READY
        // 100 MHz ticks a block may wait before it gives up
        const uint64_t lim = (uint64_t)tuning().topk_barrier_ms * 100000ull;
        // blocks that are resident from the start of the launch: they wait for the sample blocks
        static const int per_cu = [] {
            int n = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k_topk_stream, kBlock, 0) != hipSuccess || n < 1) n = 5;
            return n;
        }();
        const uint32_t first_wave = g.nbuckets + (uint32_t)device_info().num_cus * (uint32_t)per_cu;
        k_topk_stream<<<(uint32_t)blocks, kBlock, 0, st>>>(bk, g, w, epoch, first_wave, lim);
        // the select launch, at most kSelBuckets buckets at a time: all its blocks are resident
        // together, whatever the order in which the hardware dispatches them
        for (uint32_t b0 = 0; b0 < g.nbuckets; b0 += kSelBuckets) {
            const uint32_t nb = g.nbuckets - b0 < (uint32_t)kSelBuckets ? g.nbuckets - b0 : (uint32_t)kSelBuckets;
            k_topk_select<<<dim3(kGroups, nb), kBlock, 0, st>>>(bk, g, w, b0, lim);
        }
        return;
    }
    // the window comes from the previous call's exact threshold when there was one
    if (!warm) k_topk_sample<<<g.nbuckets, kSampleThreads, 0, st>>>(bk, g, w);
    const uint32_t atiles = (uint32_t)((g.bucket_elems + kATile - 1) / kATile);
    k_topk_pass_a_fast<<<dim3(atiles, g.nbuckets), kAThreads, 0, st>>>(bk, g, w);
    // 100 MHz ticks a block may wait at a barrier before it gives up
    const uint64_t limit = (uint64_t)tuning().topk_barrier_ms * 100000ull;
    k_topk_tail<<<dim3(kNSub, g.nbuckets), kBlock, 0, st>>>(bk, g, w, limit);
}

// Workspaces whose state words hold a window prediction: address -> shape of the last
// single-pass call that used it.  A call finds its workspace here with the same shape
// and skips the sample kernel; anything else (first use, another shape, the exact path
// in between, mccl_hip_topk_workspace_forget) starts from a fresh sample.
struct WarmShape {
    uint64_t n_total, bucket_elems;
    double ratio;
    int device;
};
std::mutex g_warm_mu;
std::unordered_map<uintptr_t, WarmShape> g_warm;

bool take_warm(void* workspace, const Geometry& g, double ratio, bool single_pass) {
    std::lock_guard<std::mutex> lock(g_warm_mu);
    const uintptr_t key = (uintptr_t)workspace;
    if (!single_pass) {
        g_warm.erase(key);
        return false;
    }
    const WarmShape now = {g.n_total, g.bucket_elems, ratio, device_info().device};
    auto it = g_warm.find(key);
    const bool warm = it != g_warm.end() && it->second.n_total == now.n_total &&
                      it->second.bucket_elems == now.bucket_elems && it->second.ratio == now.ratio &&
                      it->second.device == now.device;
    if (g_warm.size() > 4096 && it == g_warm.end()) g_warm.clear();
    g_warm[key] = now;
    return warm;
}

}  // namespace
}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

int mccl_hip_topk_workspace_forget(void* workspace) {
    if (!workspace) return MCCL_HIP_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_warm_mu);
    g_warm.erase((uintptr_t)workspace);
    return MCCL_HIP_OK;
}

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
                           void* stream) {
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
    const int path = tuning().topk_path;  // 0 auto, 1 exact path only, 2 fast path at any size
    const bool fast = path == 2 || (path == 0 && g.bucket_elems >= kFastMinBucket);

    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    const uint64_t nvec = g.bucket_elems / 4;
    const uint64_t bx = (cap + g.nbuckets - 1) / g.nbuckets;
    const uint64_t need_r = (nvec + kBlock * 4 - 1) / (kBlock * 4);
    const uint32_t bx_r = clamp_u32(bx < need_r ? bx : need_r, 1, 65535);
    const uint32_t bx_t = clamp_u32(bx < g.tiles ? bx : g.tiles, 1, 65535);
    const bool warm = take_warm(workspace, g, ratio, fast) && tuning().topk_warm != 0;
    if (fast) {
        Buckets bk = {};
        bk.grad = grad;
        bk.residual = residual;
        bk.wire = (uint8_t*)wire;
        bk.wire_stride = wire_stride;
        launch_single_pass(bk, g, w, warm, st);
    } else {
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
                                void* workspace, uint64_t workspace_bytes, void* stream) {
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
    // a list changes from call to call: every call samples
    mccl_hip_topk_workspace_forget(workspace);
    launch_single_pass(bk, g, w, false, (hipStream_t)stream);
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
