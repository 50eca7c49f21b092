// Decompress and rank-ordered sparse accumulate of top-k payloads for gfx950.
//
// Payload layout (csrc/compression/TopKCompression.cpp:93-113):
//   [u32 k][k x {u32 index, f32 value}], little endian, indices ascending.
//
// decompress: dense = 0, dense[index] = value (TopKCompression.cpp:122-152).
//
// sparse accumulate: the reference decompresses every peer's payload into a
// dense buffer and folds the dense buffers in ascending rank order
// (csrc/backend/ProcessGroupMCCL.cpp:1692-1709,:2272-2296).  Here the output is
// cut into tiles that live in LDS, start at +0.0, receive rank 0's, rank 1's, ...
// pairs that fall inside them, and are written once, scaled.  Two kernel
// families do that:
//   runs of tiles (up to 8 ranks, payloads of the usual density, a workspace):
//     one wavefront per run of 2048-element tiles, every rank's pairs held in
//     registers, rank order kept by the LDS's in-order execution of one
//     wavefront's adds; a small table says near which pair (to the nearest 80) of each
//     payload a run begins.
//   tile kernels (everything else): one block per 8192-element tile with a
//     barrier between ranks, ranges from a bounds table or by binary search.
// HBM traffic is close to the algorithmic minimum: every payload read once (plus
// one index in 80 for the table), every output element written once.
#include "common.hip.h"
#include "runtime.h"

namespace mcclhip {

namespace {

constexpr int kAccThreads = 512;  // threads per block of the accumulate kernel with bounds
constexpr int kAccTile = 8192;  // output elements per block, accumulated in LDS (32 KiB)

__global__ __launch_bounds__(kBlock) void k_fill_zero(float* p, uint64_t n) {
    // 16-byte stores over the aligned body, scalars at both ends
    uint64_t head = ((16 - ((uintptr_t)p & 15)) & 15) / 4;
    if (head > n) head = n;
    const uint64_t nvec = (n - head) / 4;
    u4a* v = (u4a*)(p + head);
    const u4a z = {0u, 0u, 0u, 0u};
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (uint64_t)gridDim.x * kBlock)
        v[i] = z;
    const uint64_t g = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (g < head) p[g] = 0.0f;
    const uint64_t tail = head + nvec * 4;
    if (g < 4 && tail + g < n) p[tail + g] = 0.0f;
}

__global__ __launch_bounds__(kBlock) void k_scatter(const uint32_t* wire, uint32_t expected_k, float* dense,
                                                    uint64_t count, int* status) {
    const uint32_t k = wire[0];
    if (k != expected_k) {
        if (status && blockIdx.x == 0 && threadIdx.x == 0) *status = MCCL_HIP_ERR_SIZE;
        return;
    }
    for (uint64_t p = (uint64_t)blockIdx.x * kBlock + threadIdx.x; p < k; p += (uint64_t)gridDim.x * kBlock) {
        const uint32_t idx = wire[1 + 2 * p];
        const uint32_t val = wire[2 + 2 * p];
        if (idx < count) dense[idx] = u2f(val);
        else if (status) *status = MCCL_HIP_ERR_INDEX;
    }
}

struct WirePtrs {
    const uint8_t* w[MCCL_HIP_MAX_WORLD];
};

// Scratch of mccl_hip_sparse_accumulate_static: the position table lives in
// this file-scope device array instead of a caller workspace, so the call
// allocates nothing.  Every GPU holds its own copy at its own address; host
// code only ever uses the address hipGetSymbolAddress returned for the device
// (g_static_ptr), never the array's name.
constexpr uint64_t kStaticWords = MCCL_HIP_SPARSE_STATIC_BYTES / 4;
static __device__ __align__(256) uint32_t scratch[kStaticWords];
constexpr int kMaxDevices = 64;
uint32_t* g_static_ptr[kMaxDevices];

// First pair position in [0, k) whose index is >= target (k if none).
__device__ __forceinline__ uint32_t lower_bound_idx(const uint32_t* pairs, uint32_t k, uint32_t target) {
    uint32_t lo = 0, hi = k;
    while (lo < hi) {
        const uint32_t mid = lo + ((hi - lo) >> 1);
        if (pairs[2 * (uint64_t)mid] < target) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(kBlock) void k_sparse_accumulate(float* acc, uint64_t n_total,
                                                              uint64_t bucket_elems, WirePtrs wires, int ws,
                                                              uint64_t wire_stride, int apply_scale,
                                                              float scale, int* status) {
    __shared__ float tile[kAccTile];
    __shared__ uint32_t lo_s[MCCL_HIP_MAX_WORLD], hi_s[MCCL_HIP_MAX_WORLD];
    const uint32_t b = blockIdx.y, t = blockIdx.x;
    const uint64_t bstart = (uint64_t)b * bucket_elems;
    const uint64_t bn = (n_total - bstart) < bucket_elems ? (n_total - bstart) : bucket_elems;
    const uint64_t tstart = (uint64_t)t * kAccTile;
    if (tstart >= bn) return;
    const uint32_t tlen = (uint32_t)((bn - tstart) < kAccTile ? (bn - tstart) : kAccTile);
    const uint32_t kmax = (uint32_t)((wire_stride - 4) / 8);

    for (int i = threadIdx.x; i < kAccTile; i += kBlock) tile[i] = 0.0f;
    // range of every rank's pairs inside this tile: thread r -> lower end, thread ws + r -> upper end
    if (threadIdx.x < 2 * ws) {
        const int r = threadIdx.x < ws ? threadIdx.x : threadIdx.x - ws;
        const uint32_t* wp = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride);
        uint32_t k = wp[0];
        if (k > kmax) {
            if (status) *status = MCCL_HIP_ERR_SIZE;
            k = 0;
        }
        if (threadIdx.x < ws) {
            lo_s[r] = lower_bound_idx(wp + 1, k, (uint32_t)tstart);
        } else {
            hi_s[r] = lower_bound_idx(wp + 1, k, (uint32_t)(tstart + tlen));
            // the block that owns the bucket's last tile also checks the largest index
            if (tstart + tlen == bn && k > 0 && wp[1 + 2 * (uint64_t)(k - 1)] >= bn && status)
                *status = MCCL_HIP_ERR_INDEX;
        }
    }
    __syncthreads();
    for (int r = 0; r < ws; r++) {
        const uint32_t* pairs = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride) + 1;
        const uint32_t lo = lo_s[r], hi = hi_s[r];
        for (uint32_t p = lo + threadIdx.x; p < hi; p += kBlock) {
            const uint32_t off = pairs[2 * (uint64_t)p] - (uint32_t)tstart;
            const float v = u2f(pairs[2 * (uint64_t)p + 1]);
            if (off < tlen) tile[off] = tile[off] + v;
            else if (status) *status = MCCL_HIP_ERR_INDEX;  // unsorted payload
        }
        __syncthreads();
    }
    float* out = acc + bstart + tstart;
    if (tlen == kAccTile && (((uintptr_t)out & 15) == 0)) {
        for (int i = threadIdx.x; i < kAccTile / 4; i += kBlock) {
            u4a v;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float x = tile[4 * i + q];
                v[q] = f2u(apply_scale ? x * scale : x);
            }
            ((u4a*)out)[i] = v;
        }
    } else {
        for (uint32_t i = threadIdx.x; i < tlen; i += kBlock) {
            const float x = tile[i];
            out[i] = apply_scale ? x * scale : x;
        }
    }
}

// ---- tile bounds pre-pass ------------------------------------------------------
// start[(b * ws + r) * (tiles + 1) + t] = first pair of rank r's bucket-b payload
// whose index lies in tile t or later; entry t = tiles holds k.  A rank's entries
// are contiguous: interleaving the ranks put the entries that eight different
// blocks write into one 32-byte sector and made this kernel 40 % slower.  One
// thread per pair: pair p writes the
// entry of every tile that begins between pair p-1 and pair p (usually none), so
// each entry is written exactly once for a sorted payload.  A thread takes eight
// consecutive pairs.  The pair loads do not wait for k: they stay inside the
// payload's stride and are masked afterwards.
__global__ __launch_bounds__(kBlock) void k_sparse_bounds(WirePtrs wires, int ws, uint64_t wire_stride,
                                                          uint64_t n_total, uint64_t bucket_elems, uint32_t tiles,
                                                          uint32_t* start, int* status) {
    const uint32_t b = blockIdx.y / (uint32_t)ws, r = blockIdx.y % (uint32_t)ws;
    const uint64_t bstart = (uint64_t)b * bucket_elems;
    const uint64_t bn = (n_total - bstart) < bucket_elems ? (n_total - bstart) : bucket_elems;
    const uint32_t* wp = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride);
    const uint32_t kmax = (uint32_t)((wire_stride - 4) / 8);
    constexpr int PP = 8;  // consecutive pairs per thread: four 16-byte loads, issued before the first use
    const uint32_t p0 = (blockIdx.x * kBlock + threadIdx.x) * PP;
    const u4u4* pv = (const u4u4*)(wp + 1);  // two (index, value) pairs per vector
    u4a v[PP / 2];
    uint32_t before = 0;  // index of pair p0 - 1
    if (p0 + PP <= kmax) {
#pragma unroll
        for (int j = 0; j < PP / 2; j++) v[j] = pv[p0 / 2 + j];
        if (p0 > 0) before = wp[1 + 2 * (uint64_t)(p0 - 1)];
    } else {
#pragma unroll
        for (int j = 0; j < PP / 2; j++) {
            v[j][0] = p0 + 2 * j < kmax ? wp[1 + 2 * (uint64_t)(p0 + 2 * j)] : 0u;
            v[j][2] = p0 + 2 * j + 1 < kmax ? wp[1 + 2 * (uint64_t)(p0 + 2 * j + 1)] : 0u;
        }
        if (p0 > 0 && p0 - 1 < kmax) before = wp[1 + 2 * (uint64_t)(p0 - 1)];
    }
    uint32_t k = wp[0];
    if (k > kmax) {
        if (status) *status = MCCL_HIP_ERR_SIZE;
        k = 0;
    }
    uint32_t* st = start + ((uint64_t)b * ws + r) * (tiles + 1);  // entry of tile t at st[t]
    if (k == 0) {
        for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t <= tiles; t += gridDim.x * kBlock) st[t] = 0;
        return;
    }
    uint32_t prev = before;
#pragma unroll
    for (int j = 0; j < PP; j++) {
        const uint32_t p = p0 + (uint32_t)j;
        const uint32_t idx = v[j / 2][(j & 1) * 2];
        if (p < k) {
            if (idx >= bn && status) *status = MCCL_HIP_ERR_INDEX;
            uint32_t t_hi = idx / kAccTile;  // tiles (t_prev, t_hi] begin at pair p
            if (t_hi > tiles) t_hi = tiles;
            int64_t t_prev = -1;
            if (p > 0) {
                if (prev >= idx && status) *status = MCCL_HIP_ERR_INDEX;  // not ascending
                t_prev = prev / kAccTile;
            }
            for (int64_t t = t_prev + 1; t <= (int64_t)t_hi; t++) st[t] = p;
            if (p == k - 1)
                for (uint32_t t = t_hi + 1; t <= tiles; t++) st[t] = k;
        }
        prev = idx;
    }
}

// Accumulate with precomputed bounds: every block reads its 2 * ws bounds with one
// load per lane, then issues the loads of all its pairs (every rank) before the
// first LDS add; the adds run rank by rank.
__global__ __launch_bounds__(kAccThreads) void k_sparse_accumulate_b(float* acc, uint64_t n_total,
                                                                uint64_t bucket_elems, WirePtrs wires, int ws,
                                                                uint64_t wire_stride, uint32_t tiles,
                                                                const uint32_t* start, int apply_scale,
                                                                float scale, int* status) {
    __shared__ float tile[kAccTile];
    __shared__ uint32_t lo_s[MCCL_HIP_MAX_WORLD], hi_s[MCCL_HIP_MAX_WORLD];
    const uint32_t b = blockIdx.y, t = blockIdx.x;
    const uint64_t bstart = (uint64_t)b * bucket_elems;
    const uint64_t bn = (n_total - bstart) < bucket_elems ? (n_total - bstart) : bucket_elems;
    const uint64_t tstart = (uint64_t)t * kAccTile;
    if (tstart >= bn) return;
    const uint32_t tlen = (uint32_t)((bn - tstart) < kAccTile ? (bn - tstart) : kAccTile);
    const uint32_t kmax = (uint32_t)((wire_stride - 4) / 8);
    if (threadIdx.x < 2 * ws) {
        const int r = threadIdx.x < ws ? threadIdx.x : threadIdx.x - ws;
        uint32_t v = start[((uint64_t)b * ws + r) * (tiles + 1) + t + (threadIdx.x < ws ? 0 : 1)];
        if (v > kmax) v = kmax;  // stale bound of a malformed payload: stay inside the buffer
        if (threadIdx.x < ws) lo_s[r] = v; else hi_s[r] = v;
    }
    for (int i = threadIdx.x; i < kAccTile; i += kAccThreads) tile[i] = 0.0f;
    __syncthreads();
    constexpr int RB = 8;  // ranks whose pairs are in flight together
    for (int r0 = 0; r0 < ws; r0 += RB) {
        uint32_t off[RB], val[RB];
        bool have[RB];
#pragma unroll
        for (int j = 0; j < RB; j++) {
            const int r = r0 + j;
            have[j] = false;
            if (r < ws) {
                const uint32_t lo = lo_s[r], hi = hi_s[r];
                const uint32_t p = lo + threadIdx.x;
                if (p < hi) {
                    const uint32_t* pairs = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride) + 1;
                    off[j] = pairs[2 * (uint64_t)p] - (uint32_t)tstart;
                    val[j] = pairs[2 * (uint64_t)p + 1];
                    have[j] = true;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < RB; j++) {
            const int r = r0 + j;
            if (r < ws) {
                if (have[j]) {
                    if (off[j] < tlen) tile[off[j]] = tile[off[j]] + u2f(val[j]);
                    else if (status) *status = MCCL_HIP_ERR_INDEX;
                }
                // a barrier between ranks keeps the adds to one element in rank order
                __syncthreads();
                // dense tiles (more than kAccThreads pairs of this rank): the rest, still in rank order
                if (hi_s[r] > lo_s[r] + kAccThreads) {  // block-uniform
                    const uint32_t lo = lo_s[r], hi = hi_s[r];
                    const uint32_t* pairs = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride) + 1;
                    for (uint32_t p = lo + kAccThreads + threadIdx.x; p < hi; p += kAccThreads) {
                        const uint32_t o = pairs[2 * (uint64_t)p] - (uint32_t)tstart;
                        if (o < tlen) tile[o] = tile[o] + u2f(pairs[2 * (uint64_t)p + 1]);
                        else if (status) *status = MCCL_HIP_ERR_INDEX;
                    }
                    __syncthreads();
                }
            }
        }
    }
    float* out = acc + bstart + tstart;
    if (tlen == kAccTile && (((uintptr_t)out & 15) == 0)) {
        for (int i = threadIdx.x; i < kAccTile / 4; i += kAccThreads) {
            u4a v;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float x = tile[4 * i + q];
                v[q] = f2u(apply_scale ? x * scale : x);
            }
            __builtin_nontemporal_store(v, (u4a*)out + i);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < tlen; i += kAccThreads) {
            const float x = tile[i];
            out[i] = apply_scale ? x * scale : x;
        }
    }
}

// ---- runs of tiles, one wavefront each ------------------------------------------
// The kernels above pay for finding where a tile's pairs begin: a table that a
// pre-pass builds from a second read of every payload.  Here a wavefront owns a
// run of consecutive 2048-element tiles of one bucket (four tiles at 1 %
// density) and needs a position only where its run begins, and only to the
// nearest 80 pairs.  For each rank it requests three windows of 64 consecutive
// pairs (one pair per lane) when the run begins, all ranks at once, and keeps
// them in registers: every load of the run is issued before its first store
// (a load after stores would wait for their acknowledgements).  A pair belongs
// to the current tile exactly when its index lies inside it; pairs of earlier
// tiles are behind, pairs of later tiles wait in their window.  When the
// window's last index is below the tile's end the next window shifts in and is
// looked at for the same tile; a run denser than its three windows fetches
// further windows one at a time.  The tile sits in LDS (8 KiB per wavefront),
// ranks add in ascending order (the LDS executes one wavefront's operations in
// order, so no barrier is involved), and the tile goes out once, scaled, in
// 16-byte stores.  Everything that decides control flow (tile bounds, window
// ends, counts) lives in scalar registers.
//
// Where a run begins: k_sparse_starts reads every 80th index (one 128-byte line
// in five) and writes, for every run w, the window that holds the last sampled
// index below the run's first element; every pair before that window belongs to
// an earlier run.
constexpr int kRunL = 2048;    // elements per tile of a wavefront (1024 and 4096 measured 4-5 % slower)
constexpr int kRunWaves = 8;   // wavefronts (= runs) per block: 64 KiB of LDS, two blocks per CU (4 measured 3 % slower, 2 slower still)
constexpr int kRunRanks = 8;   // ranks a wavefront holds windows for; larger worlds use the tile kernels
constexpr int kWin = kWave;    // pairs per window
constexpr int kStride = 80;    // pairs between two sampled indices of the position table: five 128-byte lines,
                               // so a run begins with at most 79 pairs of an earlier run in its first window
constexpr int kRunWins = 3;    // windows of a rank a wavefront requests when its run begins
constexpr int kXcds = 8;       // accelerator dies of an MI355X; block B runs on die B mod 8

constexpr int kStartThreads = 1024;
constexpr uint32_t kStartSamples = 8192;  // samples of one payload the block keeps in LDS (32 KiB)

// One block per (bucket, rank).  The samples (every 80th index) are requested before k is known
// (inside the payload's capacity, masked afterwards), so the kernel is one round trip: samples
// into LDS, then every run finds by binary search how many samples lie below its first element.
__global__ __launch_bounds__(kStartThreads) void k_sparse_starts(WirePtrs wires, int ws, uint64_t wire_stride,
                                                                 uint32_t run_elems, uint32_t runs, uint32_t* start,
                                                                 int* status) {
    __shared__ uint32_t samp[kStartSamples];
    const uint32_t b = blockIdx.x / (uint32_t)ws, r = blockIdx.x % (uint32_t)ws;
    const uint32_t* wp = (const uint32_t*)(wires.w[r] + (uint64_t)b * wire_stride);
    const uint32_t kmax = (uint32_t)((wire_stride - 4) / 8);
    const uint32_t cap = (kmax + kStride - 1) / kStride;  // samples the payload can hold (at most kStartSamples)
    constexpr int kPer = kStartSamples / kStartThreads;
    uint32_t v[kPer];
#pragma unroll
    for (int i = 0; i < kPer; i++) {
        const uint32_t j = (uint32_t)i * kStartThreads + threadIdx.x;
        v[i] = j < cap ? wp[1 + 2 * (uint64_t)kStride * j] : 0u;
    }
    uint32_t k = wp[0];
    if (k > kmax) {
        if (status) *status = MCCL_HIP_ERR_SIZE;
        k = 0;
    }
    const uint32_t nsamp = (k + kStride - 1) / kStride;
#pragma unroll
    for (int i = 0; i < kPer; i++) {
        const uint32_t j = (uint32_t)i * kStartThreads + threadIdx.x;
        if (j < cap) samp[j] = v[i];
    }
    __syncthreads();
    uint32_t* st = start + ((uint64_t)b * ws + r) * runs;
    for (uint32_t w = threadIdx.x; w < runs; w += kStartThreads) {
        // samples below the run's first element; the last of them names the window to begin in.
        // (Unsorted samples give some window or other; the accumulate kernel trusts no entry.)
        const uint64_t first = (uint64_t)w * run_elems;
        uint32_t lo = 0, hi = nsamp;
        while (lo < hi) {
            const uint32_t mid = lo + ((hi - lo) >> 1);
            if (samp[mid] < first) lo = mid + 1;
            else hi = mid;
        }
        st[w] = lo ? (lo - 1) * kStride : 0u;
    }
}

typedef const __attribute__((address_space(1))) uint32_t* GlobalWords;  // loads compile to global_load, not flat_load

// One window of a rank's pairs: lane l asks for pair base + l.  The load is unconditional (no
// branch, so the loads of all ranks and windows are in flight together): positions past the
// payload's capacity are clamped to its last pair (kmax >= 1) and sorted out by window_index.
__device__ __forceinline__ u2a4 load_window(GlobalWords pairs, uint32_t base, uint32_t kmax, int lane) {
    uint32_t pos = base + (uint32_t)lane;
    if (pos > kmax - 1) pos = kmax - 1;
    return *(const __attribute__((address_space(1))) u2a4*)(pairs + 2 * (uint64_t)pos);
}

// The index a lane holds: lanes at or past k hold 0xFFFFFFFF, which lies in no tile.
__device__ __forceinline__ uint32_t window_index(u2a4 v, uint32_t base, uint32_t k, int lane) {
    return base + (uint32_t)lane < k ? v[0] : 0xFFFFFFFFu;
}

// The value the lane below holds (lane 0: `first`): one DPP move, no LDS traffic.
__device__ __forceinline__ uint32_t from_lane_below(uint32_t v, uint32_t first) {
    // wave_shr:1 - lane l reads lane l - 1 across the whole wavefront; lane 0 keeps `first`
    return (uint32_t)__builtin_amdgcn_update_dpp((int)first, (int)v, 0x138, 0xf, 0xf, false);
}

// Lanes (as a mask) whose pair breaks the rule: indices of a window ascend, continue the pair
// before the window (`before`), and stay inside the bucket.  `idx` is what was loaded, before
// the lanes past k are marked.
__device__ __forceinline__ uint64_t bad_lanes(uint32_t idx, uint32_t base, uint32_t k, uint32_t before, uint32_t bn) {
    const uint32_t up = from_lane_below(idx, before);
    uint64_t m = __ballot(up >= idx);
    if (base == 0) m &= ~1ull;  // the payload's first pair follows nothing
    m |= __ballot(idx >= bn);
    const uint32_t live = k > base ? k - base : 0u;  // lanes that hold a pair of the payload
    return live >= (uint32_t)kWin ? m : m & ((1ull << live) - 1);
}

// tile[off] += v as one LDS instruction that returns nothing.  The LDS adds in IEEE single
// precision, round to nearest even, subnormals kept, and executes one wavefront's instructions in
// the order they were issued, so successive ranks' adds to one element happen in rank order
// with no wait between them.
__device__ __forceinline__ void lds_add(float* p, float v) {
    (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}

__device__ __forceinline__ uint32_t lane_value(uint32_t v, int l) {
    return (uint32_t)__builtin_amdgcn_readlane((int)v, l);
}


// NR: ranks the code is unrolled for (ws <= NR; the ranks past ws read rank 0's payload as if
// its k were 0).  wire_stride holds at least one pair.
template <int NR>
__global__ __launch_bounds__(kRunWaves * kWave, 4) void k_sparse_accumulate_runs(
    float* acc, uint64_t n_total, uint64_t bucket_elems, WirePtrs wires, int ws, uint64_t wire_stride,
    uint32_t run_steps, uint32_t runs, uint32_t nbuckets, uint32_t blocks_per_xcd, const uint32_t* start,
    int apply_scale, float scale, int* status) {
    __shared__ __attribute__((aligned(16))) float tiles[kRunWaves][kRunL];
    const int lane = threadIdx.x & (kWave - 1);
    // the same in every lane; saying so keeps everything derived from it (the run, its tiles,
    // the window tests) in scalar registers and on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    // blocks go to the XCDs in turn: block B runs on XCD B mod 8.  Each XCD takes one contiguous
    // eighth of the runs, in order, so the windows that neighbouring runs share are found in
    // that XCD's L2 and its stores move through memory in one direction.
    const uint32_t vblock = (blockIdx.x % kXcds) * blocks_per_xcd + blockIdx.x / kXcds;
    const uint64_t grun = (uint64_t)vblock * kRunWaves + (uint32_t)wave;
    if (grun >= (uint64_t)runs * nbuckets) return;  // whole wavefront; the kernel has no block barriers
    const uint32_t b = (uint32_t)(grun / runs), run = (uint32_t)(grun % runs);
    const uint64_t bstart = (uint64_t)b * bucket_elems;
    const uint32_t bn = (uint32_t)((n_total - bstart) < bucket_elems ? (n_total - bstart) : bucket_elems);
    const uint64_t e0 = (uint64_t)run * run_steps * kRunL;
    if (e0 >= bn) return;
    const uint64_t e1w = e0 + (uint64_t)run_steps * kRunL;
    const uint32_t e1 = e1w < bn ? (uint32_t)e1w : bn;  // end of this run
    const uint32_t kmax = (uint32_t)((wire_stride - 4) / 8);
    float* tile = tiles[wave];
    {
        const u4a z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < kRunL / (4 * kWave); i++) ((u4a*)tile)[i * kWave + lane] = z;
    }

    uint64_t bad = 0;       // lanes that saw a pair out of order or out of range, reported once
    bool oversize = false;  // a k beyond the payload's capacity
    // first round trip: every rank's k and the window its pairs of this run begin in
    uint32_t kk[NR], wnext[NR];
    GlobalWords pairs[NR];
    {
        uint32_t kraw[NR], craw[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const int rr = r < ws ? r : 0;
            GlobalWords wp = (GlobalWords)(wires.w[rr] + (uint64_t)b * wire_stride);
            pairs[r] = wp + 1;
            kraw[r] = wp[0];
            craw[r] = ((GlobalWords)start)[((uint64_t)b * ws + rr) * runs + run];
        }
#pragma unroll
        for (int r = 0; r < NR; r++) {
            uint32_t k = kraw[r], c = craw[r];
            if (k > kmax) {
                oversize = true;
                k = 0;
            }
            if (r >= ws) k = 0;
            if (c >= k) c = k ? k - 1 : 0u;  // a table entry is never trusted
            kk[r] = __builtin_amdgcn_readfirstlane(k);
            wnext[r] = __builtin_amdgcn_readfirstlane(c);
        }
    }
    // second round trip: kRunWins windows of every rank at once; a run of the usual density needs
    // no other load
    u2a4 raw[NR][kRunWins];
    uint32_t before[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
        before[r] = pairs[r][2 * (uint64_t)(wnext[r] ? wnext[r] - 1 : 0u)];  // only used when the window is not the first
#pragma unroll
        for (int i = 0; i < kRunWins; i++) raw[r][i] = load_window(pairs[r], wnext[r] + (uint32_t)i * kWin, kmax, lane);
    }
    // wlast[r][i]: last index of window i, in a scalar register: whether a tile is done with a
    // window is decided without vector work
    uint32_t widx[NR][kRunWins], wval[NR][kRunWins], wlast[NR][kRunWins];
    int nreg[NR];  // windows of the rank still in registers
#pragma unroll
    for (int r = 0; r < NR; r++) {
        uint32_t prev = lane_value(before[r], 0);
        // The pair in front of the first window must lie before this run: a position-table entry
        // that points past the run's first pair (a table left by another call racing on shared
        // scratch, or sampled from a payload that is not ascending) would drop pairs silently.
        if (wnext[r] > 0 && kk[r] > 0 && prev >= (uint32_t)e0) bad |= 1ull;
#pragma unroll
        for (int i = 0; i < kRunWins; i++) {
            const uint32_t base = wnext[r] + (uint32_t)i * kWin;
            bad |= bad_lanes(raw[r][i][0], base, kk[r], prev, bn);
            widx[r][i] = window_index(raw[r][i], base, kk[r], lane);
            wval[r][i] = raw[r][i][1];
            prev = lane_value(widx[r][i], kWin - 1);  // 0xFFFFFFFF once the payload's end is in the window
            wlast[r][i] = prev;
        }
        wnext[r] += kRunWins * kWin;  // the first window not in registers
        nreg[r] = kRunWins;
    }

    for (uint64_t ts64 = e0; ts64 < e1; ts64 += kRunL) {  // 64-bit: the last tile of a 2^32-element bucket ends past 32 bits
        const uint32_t ts = (uint32_t)ts64;
        const uint32_t tlen = (e1 - ts) < (uint32_t)kRunL ? (e1 - ts) : (uint32_t)kRunL;
        const uint32_t tend = ts + tlen;
#pragma unroll
        for (int r = 0; r < NR; r++) {
            // slot 0 is the window the run has reached; the others wait behind it
            for (;;) {
                const uint32_t off = widx[r][0] - ts;
                if (off < tlen) lds_add(&tile[off], u2f(wval[r][0]));
                if (wlast[r][0] >= tend) break;  // the rest of the window belongs to later tiles
                // the window ends inside this tile: the next one may begin in it
                if (nreg[r] > 1) {
#pragma unroll
                    for (int i = 0; i + 1 < kRunWins; i++) {
                        widx[r][i] = widx[r][i + 1];
                        wval[r][i] = wval[r][i + 1];
                        wlast[r][i] = wlast[r][i + 1];
                    }
                    nreg[r]--;
                } else if (wnext[r] < kk[r]) {
                    // a dense stretch used up the windows requested at the start: further windows
                    // come one at a time, each waited for
                    const u2a4 v = load_window(pairs[r], wnext[r], kmax, lane);
                    bad |= bad_lanes(v[0], wnext[r], kk[r], wlast[r][0], bn);
                    widx[r][0] = window_index(v, wnext[r], kk[r], lane);
                    wval[r][0] = v[1];
                    wlast[r][0] = lane_value(widx[r][0], kWin - 1);
                    wnext[r] += kWin;
                } else {
                    wlast[r][0] = 0xFFFFFFFFu;  // the payload is finished
                    widx[r][0] = 0xFFFFFFFFu;
                    break;
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        float* out = acc + bstart + ts;
        if (tlen == (uint32_t)kRunL && (((uintptr_t)out & 15) == 0)) {
            // all LDS reads first, so that one wait covers them; then the tile is cleared for the
            // next round and the stores go out
            constexpr int kVecs = kRunL / (4 * kWave);
            u4a v[kVecs];
#pragma unroll
            for (int i = 0; i < kVecs; i++) v[i] = ((u4a*)tile)[i * kWave + lane];
            const u4a z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < kVecs; i++) ((u4a*)tile)[i * kWave + lane] = z;
            if (apply_scale) {
#pragma unroll
                for (int i = 0; i < kVecs; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) v[i][q] = f2u(u2f(v[i][q]) * scale);
            }
#pragma unroll
            for (int i = 0; i < kVecs; i++) {
                __builtin_nontemporal_store(v[i], (u4a*)out + i * kWave + lane);
            }
        } else {
            for (uint32_t i = (uint32_t)lane; i < tlen; i += kWave) {
                const float x = tile[i];
                tile[i] = 0.0f;
                out[i] = apply_scale ? x * scale : x;
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (status) {
        if (bad) *status = MCCL_HIP_ERR_INDEX;
        if (oversize) *status = MCCL_HIP_ERR_SIZE;
    }
}

// Validates the arguments and enqueues the kernels; `workspace` (may be null:
// scratch-free kernel) is known to be large enough.
int accumulate(float* acc, uint64_t n_total, uint64_t bucket_elems, const void* const* host_wires, int ws,
               uint64_t wire_stride, int apply_scale, float scale, int* status, void* workspace,
               void* stream) {
    if (!acc || !host_wires || ws < 1 || ws > MCCL_HIP_MAX_WORLD) return MCCL_HIP_ERR_ARG;
    if (n_total == 0 || n_total > MCCL_HIP_MAX_ELEMS || bucket_elems == 0) return MCCL_HIP_ERR_ARG;
    if (wire_stride < 4 || (wire_stride & 3)) return MCCL_HIP_ERR_ARG;
    if (bucket_elems > n_total) bucket_elems = n_total;
    if (bucket_elems > 0xFFFFFFFFull) return MCCL_HIP_ERR_ARG;
    const uint64_t nb = (n_total + bucket_elems - 1) / bucket_elems;
    if (nb * (uint64_t)ws > 65535) return MCCL_HIP_ERR_ARG;
    WirePtrs wp;
    for (int r = 0; r < MCCL_HIP_MAX_WORLD; r++) wp.w[r] = nullptr;
    for (int r = 0; r < ws; r++) {
        if (!host_wires[r] || ((uintptr_t)host_wires[r] & 3)) return MCCL_HIP_ERR_ARG;
        wp.w[r] = (const uint8_t*)host_wires[r];
    }
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const uint32_t tiles = (uint32_t)((bucket_elems + kAccTile - 1) / kAccTile);
    if (!workspace) {
        // no scratch: every block finds its ranges by binary search
        k_sparse_accumulate<<<dim3(tiles, (uint32_t)nb), kBlock, 0, st>>>(acc, n_total, bucket_elems, wp, ws,
                                                                           wire_stride, apply_scale, scale, status);
        return launch_status();
    }
    uint32_t* start = (uint32_t*)(((uintptr_t)workspace + 15) & ~(uintptr_t)15);
    const uint64_t kmax = (wire_stride - 4) / 8;
    // pairs of one rank in a 2048-element tile when the payload is full
    const uint64_t steps_bucket = (bucket_elems + kRunL - 1) / kRunL;
    const uint64_t per_tile = (kmax + steps_bucket - 1) / steps_bucket;
    if (ws <= kRunRanks && tuning().sparse_path != 1 && per_tile <= 96 && kmax >= 1 &&
        (kmax + kStride - 1) / kStride <= kStartSamples) {
        // a run is as many tiles as bring about 96 pairs of a rank: with up to 79 pairs of the run
        // before it in the first window, the three windows requested at its start (192 pairs) hold a
        // run of the usual density whole, and it never loads again
        uint64_t run_steps = (uint64_t)tuning().sparse_run_steps;
        if (run_steps == 0) run_steps = per_tile ? 96 / per_tile : 8;
        if (run_steps > 8 && tuning().sparse_run_steps == 0) run_steps = 8;
        if (run_steps < 1) run_steps = 1;
        if (run_steps > steps_bucket) run_steps = steps_bucket;
        const uint32_t runs = (uint32_t)((steps_bucket + run_steps - 1) / run_steps);
        k_sparse_starts<<<(uint32_t)(nb * ws), kStartThreads, 0, st>>>(wp, ws, wire_stride,
                                                                        (uint32_t)(run_steps * kRunL), runs, start, status);
        const uint64_t blocks = ((uint64_t)runs * nb + kRunWaves - 1) / kRunWaves;
        const uint32_t per_xcd = (uint32_t)((blocks + kXcds - 1) / kXcds);
#define MCCLHIP_RUNS(NR)                                                                               \
    k_sparse_accumulate_runs<NR><<<per_xcd * kXcds, kRunWaves * kWave, 0, st>>>(                        \
        acc, n_total, bucket_elems, wp, ws, wire_stride, (uint32_t)run_steps, runs, (uint32_t)nb, per_xcd, \
        start, apply_scale, scale, status)
        if (ws == 1) MCCLHIP_RUNS(1);
        else if (ws == 2) MCCLHIP_RUNS(2);
        else if (ws <= 4) MCCLHIP_RUNS(4);
        else MCCLHIP_RUNS(8);
#undef MCCLHIP_RUNS
        return launch_status();
    }
    const uint32_t bx = clamp_u32((kmax + kBlock * 8 - 1) / (kBlock * 8), 1, 0x7FFFFFFF);
    k_sparse_bounds<<<dim3(bx, (uint32_t)(nb * ws)), kBlock, 0, st>>>(wp, ws, wire_stride, n_total, bucket_elems,
                                                                        tiles, start, status);
    k_sparse_accumulate_b<<<dim3(tiles, (uint32_t)nb), kAccThreads, 0, st>>>(acc, n_total, bucket_elems, wp, ws,
                                                                         wire_stride, tiles, start, apply_scale,
                                                                         scale, status);
    return launch_status();
}

}  // namespace

// Called by mccl_hip_init with `device` current, once per device: looks up the
// address of that device's copy of the static scratch array.
int sparse_static_setup(int device) {
    if (device < 0 || device >= kMaxDevices) return MCCL_HIP_OK;  // the static entry point reports it
    if (g_static_ptr[device]) return MCCL_HIP_OK;
    uint32_t* p = nullptr;
    MCCLHIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    g_static_ptr[device] = p;
    return MCCL_HIP_OK;
}

}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

int mccl_hip_topk_decompress(const void* wire, uint64_t wire_bytes, float* dense, uint64_t count,
                             int* status, void* stream) {
    if (!wire || (!dense && count) || ((uintptr_t)wire & 3)) return MCCL_HIP_ERR_ARG;
    if (count > 0xFFFFFFFFull) return MCCL_HIP_ERR_ARG;
    if (wire_bytes < 4 || ((wire_bytes - 4) & 7)) return MCCL_HIP_ERR_SIZE;
    const uint64_t k64 = (wire_bytes - 4) / 8;
    if (k64 > 0xFFFFFFFFull) return MCCL_HIP_ERR_SIZE;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    if (count) {
        k_fill_zero<<<clamp_u32((count / 4 + kBlock - 1) / kBlock, 1, cap), kBlock, 0, st>>>(dense, count);
    }
    k_scatter<<<clamp_u32((k64 + kBlock - 1) / kBlock, 1, cap), kBlock, 0, st>>>(
        (const uint32_t*)wire, (uint32_t)k64, dense, count, status);
    return launch_status();
}

uint64_t mccl_hip_sparse_accumulate_workspace_bytes(uint64_t n_total, uint64_t bucket_elems, int ws) {
    if (n_total == 0 || bucket_elems == 0 || ws < 1 || ws > MCCL_HIP_MAX_WORLD) return 0;
    if (bucket_elems > n_total) bucket_elems = n_total;
    const uint64_t nb = (n_total + bucket_elems - 1) / bucket_elems;
    // one entry per 2048-element tile: room for the table of either kernel pair
    const uint64_t tiles = (bucket_elems + kRunL - 1) / kRunL;
    return nb * (uint64_t)ws * (tiles + 1) * 4 + 64;
}

int mccl_hip_sparse_accumulate(float* acc, uint64_t n_total, uint64_t bucket_elems,
                               const void* const* host_wires, int ws, uint64_t wire_stride,
                               int apply_scale, float scale, int* status, void* workspace,
                               uint64_t workspace_bytes, void* stream) {
    if (workspace && workspace_bytes < mccl_hip_sparse_accumulate_workspace_bytes(n_total, bucket_elems, ws))
        return MCCL_HIP_ERR_WORKSPACE;
    return accumulate(acc, n_total, bucket_elems, host_wires, ws, wire_stride, apply_scale, scale, status,
                      workspace, stream);
}

int mccl_hip_sparse_accumulate_static(float* acc, uint64_t n_total, uint64_t bucket_elems,
                                      const void* const* host_wires, int ws, uint64_t wire_stride,
                                      int apply_scale, float scale, int* status, void* stream) {
    const uint64_t need = mccl_hip_sparse_accumulate_workspace_bytes(n_total, bucket_elems, ws);
    if (need == 0) return MCCL_HIP_ERR_ARG;
    if (need > MCCL_HIP_SPARSE_STATIC_BYTES) return MCCL_HIP_ERR_WORKSPACE;
    int rc = mccl_hip_init();  // resolves this device's copy of the scratch array on first use
    if (rc) return rc;
    const int dev = device_info().device;
    if (dev < 0 || dev >= kMaxDevices || !g_static_ptr[dev]) return MCCL_HIP_ERR_RUNTIME;
    return accumulate(acc, n_total, bucket_elems, host_wires, ws, wire_stride, apply_scale, scale, status,
                      g_static_ptr[dev], stream);
}

}  // extern "C"
