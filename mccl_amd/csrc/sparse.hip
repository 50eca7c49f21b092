// Decompress and rank-ordered sparse accumulate of top-k payloads for gfx950.
//
// Payload layout (csrc/compression/TopKCompression.cpp:93-113):
//   [u32 k][k x {u32 index, f32 value}], little endian, indices ascending.
//
// decompress: dense = 0, dense[index] = value (TopKCompression.cpp:122-152).
//
// sparse accumulate: the reference decompresses every peer's payload into a
// dense buffer and folds the dense buffers in ascending rank order
// (csrc/backend/ProcessGroupMCCL.cpp:1692-1709,:2272-2296).  Here each block
// owns one 8192-element tile of the output, keeps it in LDS starting at +0.0,
// and for rank 0, 1, ... adds that rank's pairs that fall inside the tile
// (found by binary search in the sorted payload; indices are unique within a
// rank, so a rank's adds never collide), then writes the tile once, scaled.
// HBM traffic is the algorithmic minimum: every payload read once, every output
// element written once.
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

// Scratch of mccl_hip_sparse_accumulate_static: the tile-bounds table lives in
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
    const uint64_t tiles = (bucket_elems + kAccTile - 1) / kAccTile;
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
