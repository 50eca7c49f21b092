// Top-k gradient sparsifier with error feedback for gfx950.
//
// Semantics (csrc/compression/TopKCompression.cpp:38-120): per bucket,
// adjusted = grad + residual; the k elements of largest |adjusted| go on the
// wire in ascending index order as [u32 k][k x {u32 index, f32 value}];
// residual = adjusted everywhere except 0.0f at the picks.  Ties at the
// threshold magnitude go to the lower index.
//
// For non-NaN floats, ordering by fabs() is ordering of the 31-bit pattern
// `bits & 0x7FFFFFFF`, so selection is an exact radix select on that key:
//   pass A      residual <- grad + residual, histogram of key[30:20]   (12 B/elem)
//   pick        threshold bin, how many picks remain inside it
//   refine x2   histograms of key[19:10] and key[9:0] among elements that match
//               the prefix so far                                      (4 B/elem each)
//   count       per 4096-element tile: #(key > T) and #(key == T)
//   scan        exclusive prefix over tiles
//   emit        ordered compaction: an element at index i lands at
//               gt_before(i) + min(eq_before(i), need), ties accepted while
//               eq_before(i) < need; residual[i] = 0 at every pick
// All buckets of a gradient run in the same launches (blockIdx.y = bucket).
#include "common.hip.h"
#include "runtime.h"

namespace mcclhip {

namespace {

constexpr int kTile = 4096;           // elements per compaction tile
constexpr int kBins0 = 2048;          // key[30:20]
constexpr int kBinsR = 1024;          // key[19:10], key[9:0]
constexpr int kHistWords = kBins0 + 2 * kBinsR;
constexpr int kStateWords = 16;

// per-bucket state words
enum { S_PREFIX = 0, S_REMAIN = 1, S_GT_TOTAL = 2, S_EQ_TOTAL = 3 };

struct Geometry {
    uint64_t n_total;
    uint64_t bucket_elems;
    uint32_t nbuckets;
    uint32_t tiles;   // tiles per (full) bucket
    uint32_t k_full;  // k of a bucket with bucket_elems elements
    uint32_t k_last;  // k of the last bucket
};

struct Workspace {
    uint32_t* hist;     // [nbuckets][kHistWords]
    uint32_t* state;    // [nbuckets][kStateWords]
    uint32_t* tile_gt;  // [nbuckets][tiles]
    uint32_t* tile_eq;  // [nbuckets][tiles]
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

__global__ __launch_bounds__(kBlock) void k_zero_words(uint32_t* p, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        p[i] = 0;
}

// Adds the block's LDS histogram into the bucket's global one (non-empty bins only).
__device__ __forceinline__ void flush_hist(const uint32_t* lds, uint32_t* global, int bins) {
    for (int i = threadIdx.x; i < bins; i += kBlock) {
        uint32_t c = lds[i];
        if (c) atomicAdd(&global[i], c);
    }
}

// ---- pass A ---------------------------------------------------------------------
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
    flush_hist(lh, w.hist + (uint64_t)b * kHistWords, kBins0);
}

// ---- pick: one block per bucket ---------------------------------------------------
// Finds the bin where the running count from the top bin downwards reaches the
// number of picks still to place, narrows the key prefix to it, and keeps the
// number of picks that fall inside it.
template <int BINS>
__global__ __launch_bounds__(kBlock) void k_topk_pick(Geometry g, Workspace w, int round) {
    __shared__ uint32_t scan_smem[kBlock / kWave + 1];
    constexpr int PER = BINS / kBlock;
    const uint32_t b = blockIdx.x;
    const int hist_off = round == 0 ? 0 : (round == 1 ? kBins0 : kBins0 + kBinsR);
    const int shift = round == 0 ? 20 : (round == 1 ? 10 : 0);
    const uint32_t* h = w.hist + (uint64_t)b * kHistWords + hist_off;
    uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const uint32_t remaining = round == 0 ? bucket_k(g, b) : st[S_REMAIN];
    const uint32_t prefix = round == 0 ? 0u : st[S_PREFIX];
    // thread t owns bins descending from BINS-1 - t*PER
    uint32_t c[PER];
    uint32_t sum = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        c[j] = h[BINS - 1 - (threadIdx.x * PER + j)];
        sum += c[j];
    }
    uint32_t total;
    uint32_t above = block_exclusive_scan(sum, scan_smem, &total);
#pragma unroll
    for (int j = 0; j < PER; j++) {
        if (above < remaining && remaining <= above + c[j]) {
            const uint32_t bin = BINS - 1 - (threadIdx.x * PER + j);
            st[S_PREFIX] = prefix | (bin << shift);
            st[S_REMAIN] = remaining - above;
        }
        above += c[j];
    }
}

// ---- refine: histogram of the next key bits among prefix matches -------------------
__global__ __launch_bounds__(kBlock) void k_topk_refine(const float* residual, Geometry g, Workspace w,
                                                        int round) {
    __shared__ uint32_t lh[kBinsR];
    for (int i = threadIdx.x; i < kBinsR; i += kBlock) lh[i] = 0;
    __syncthreads();
    const uint32_t b = blockIdx.y;
    const uint64_t bn = bucket_count(g, b);
    const float* rp = residual + (uint64_t)b * g.bucket_elems;
    const int shift = round == 1 ? 10 : 0;
    const int hi_shift = shift + 10;
    const uint32_t want = w.state[(uint64_t)b * kStateWords + S_PREFIX] >> hi_shift;
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
                    if ((key >> hi_shift) == want) atomicAdd(&lh[(key >> shift) & (kBinsR - 1)], 1u);
                }
            }
        }
    }
    const uint64_t gtid = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (gtid < 4 && nvec * 4 + gtid < bn) {
        const uint32_t key = key_of(rp[nvec * 4 + gtid]);
        if ((key >> hi_shift) == want) atomicAdd(&lh[(key >> shift) & (kBinsR - 1)], 1u);
    }
    __syncthreads();
    flush_hist(lh, w.hist + (uint64_t)b * kHistWords + (round == 1 ? kBins0 : kBins0 + kBinsR), kBinsR);
}

// ---- tiles ---------------------------------------------------------------------------
// Loads the four keys of tile `t`, sub-tile `it`, lane slot; elements past the
// bucket end read as "not selected" (valid = false).
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

__global__ __launch_bounds__(kBlock) void k_topk_count(const float* residual, Geometry g, Workspace w) {
    __shared__ uint32_t red[kBlock / kWave + 1];
    const uint32_t b = blockIdx.y, t = blockIdx.x;
    const uint64_t bn = bucket_count(g, b);
    if ((uint64_t)t * kTile >= bn) {
        if (threadIdx.x == 0) {
            w.tile_gt[(uint64_t)b * g.tiles + t] = 0;
            w.tile_eq[(uint64_t)b * g.tiles + t] = 0;
        }
        return;
    }
    const float* rp = residual + (uint64_t)b * g.bucket_elems;
    const uint32_t T = w.state[(uint64_t)b * kStateWords + S_PREFIX];
    uint32_t packed = 0;  // gt in the low half, eq in the high half (each <= 4096)
#pragma unroll
    for (int it = 0; it < kTile / (kBlock * 4); it++) {
        Quad q = load_quad(rp, bn, t, it);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t key = q.bits[j] & 0x7FFFFFFFu;
            if (q.valid[j]) packed += (key > T ? 1u : 0u) + (key == T ? 0x10000u : 0u);
        }
    }
    uint32_t total;
    block_exclusive_scan(packed, red, &total);
    if (threadIdx.x == 0) {
        w.tile_gt[(uint64_t)b * g.tiles + t] = total & 0xFFFFu;
        w.tile_eq[(uint64_t)b * g.tiles + t] = total >> 16;
    }
}

// One block per bucket: in-place exclusive scan of the tile counts.
__global__ __launch_bounds__(kBlock) void k_topk_scan(Geometry g, Workspace w) {
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const uint32_t b = blockIdx.x;
    uint32_t* gt = w.tile_gt + (uint64_t)b * g.tiles;
    uint32_t* eq = w.tile_eq + (uint64_t)b * g.tiles;
    uint32_t carry_gt = 0, carry_eq = 0;
    for (uint32_t base = 0; base < g.tiles; base += kBlock) {
        const uint32_t i = base + threadIdx.x;
        const uint32_t a = i < g.tiles ? gt[i] : 0u;
        const uint32_t e = i < g.tiles ? eq[i] : 0u;
        uint32_t ta, te;
        const uint32_t xa = block_exclusive_scan(a, smem, &ta);
        const uint32_t xe = block_exclusive_scan(e, smem, &te);
        if (i < g.tiles) {
            gt[i] = carry_gt + xa;
            eq[i] = carry_eq + xe;
        }
        carry_gt += ta;
        carry_eq += te;
    }
    if (threadIdx.x == 0) {
        w.state[(uint64_t)b * kStateWords + S_GT_TOTAL] = carry_gt;
        w.state[(uint64_t)b * kStateWords + S_EQ_TOTAL] = carry_eq;
    }
}

__global__ __launch_bounds__(kBlock) void k_topk_emit(float* residual, Geometry g, Workspace w,
                                                      uint8_t* wire, uint64_t wire_stride) {
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const uint32_t b = blockIdx.y, t = blockIdx.x;
    const uint64_t bn = bucket_count(g, b);
    uint32_t* out = (uint32_t*)(wire + (uint64_t)b * wire_stride);
    if (t == 0 && threadIdx.x == 0) out[0] = bucket_k(g, b);
    if ((uint64_t)t * kTile >= bn) return;
    float* rp = residual + (uint64_t)b * g.bucket_elems;
    const uint32_t* st = w.state + (uint64_t)b * kStateWords;
    const uint32_t T = st[S_PREFIX];
    const uint32_t need = st[S_REMAIN];
    uint32_t gt_run = w.tile_gt[(uint64_t)b * g.tiles + t];
    uint32_t eq_run = w.tile_eq[(uint64_t)b * g.tiles + t];
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

Workspace carve(void* base, const Geometry& g) {
    Workspace w;
    uint32_t* p = (uint32_t*)base;
    w.hist = p;
    p += (uint64_t)g.nbuckets * kHistWords;
    w.state = p;
    p += (uint64_t)g.nbuckets * kStateWords;
    w.tile_gt = p;
    p += (uint64_t)g.nbuckets * g.tiles;
    w.tile_eq = p;
    return w;
}

uint64_t workspace_words(uint64_t nbuckets, uint64_t tiles) {
    return nbuckets * (kHistWords + kStateWords + 2 * tiles);
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

uint64_t mccl_hip_topk_workspace_bytes(uint64_t n_total, uint64_t bucket_elems) {
    Geometry g;
    if (!make_geometry(n_total, bucket_elems, 0.5, &g)) return 0;
    return workspace_words(g.nbuckets, g.tiles) * 4 + 256;
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
    if (workspace_bytes < workspace_words(g.nbuckets, g.tiles) * 4) return MCCL_HIP_ERR_WORKSPACE;
    if ((uintptr_t)workspace & 3) return MCCL_HIP_ERR_ARG;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    Workspace w = carve(workspace, g);

    const uint64_t zero_words = (uint64_t)g.nbuckets * (kHistWords + kStateWords);
    k_zero_words<<<clamp_u32((zero_words + kBlock - 1) / kBlock, 1, 1024), kBlock, 0, st>>>(w.hist, zero_words);

    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    const uint64_t nvec = g.bucket_elems / 4;
    uint64_t bx = (cap + g.nbuckets - 1) / g.nbuckets;
    const uint64_t need_a = (nvec + kBlock * 2 - 1) / (kBlock * 2);
    const uint32_t bx_a = clamp_u32(bx < need_a ? bx : need_a, 1, 65535);
    const uint64_t need_r = (nvec + kBlock * 4 - 1) / (kBlock * 4);
    const uint32_t bx_r = clamp_u32(bx < need_r ? bx : need_r, 1, 65535);

    k_topk_pass_a<<<dim3(bx_a, g.nbuckets), kBlock, 0, st>>>(grad, residual, g, w);
    k_topk_pick<kBins0><<<g.nbuckets, kBlock, 0, st>>>(g, w, 0);
    k_topk_refine<<<dim3(bx_r, g.nbuckets), kBlock, 0, st>>>(residual, g, w, 1);
    k_topk_pick<kBinsR><<<g.nbuckets, kBlock, 0, st>>>(g, w, 1);
    k_topk_refine<<<dim3(bx_r, g.nbuckets), kBlock, 0, st>>>(residual, g, w, 2);
    k_topk_pick<kBinsR><<<g.nbuckets, kBlock, 0, st>>>(g, w, 2);
    k_topk_count<<<dim3(g.tiles, g.nbuckets), kBlock, 0, st>>>(residual, g, w);
    k_topk_scan<<<g.nbuckets, kBlock, 0, st>>>(g, w);
    k_topk_emit<<<dim3(g.tiles, g.nbuckets), kBlock, 0, st>>>(residual, g, w, (uint8_t*)wire, wire_stride);
    return launch_status();
}

}  // extern "C"
