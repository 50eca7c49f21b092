// Chunk-fold kernels for gfx950: the reduction a ring allreduce / reduce-scatter
// applies to every inbound chunk, the AVG scale, the fused add+scale, and the
// W-way fold in ring-step order.
//
// All of them are HBM-bound streaming kernels: 256-thread blocks, every lane
// moves 16 bytes per access (global_load/store_dwordx4), a few independent
// accesses per operand are issued before the first use, and the grid is sized
// to keep every CU's wave slots full.  The destination is peeled to 16-byte
// alignment; sources are read with element alignment only, because chunk views
// start at arbitrary element offsets (csrc/backend/ProcessGroupMCCL.cpp:1735-1741).
//
// Arithmetic follows the reference's CPU folds (csrc/metal/AccelerateOps.mm):
// one IEEE fp32 operation per element and step, never an FMA (this file is
// compiled with -ffp-contract=off); fp16/bf16 are widened, operated on in fp32
// and narrowed once with round-to-nearest-even.
#include "common.hip.h"
#include "runtime.h"

#include <type_traits>

namespace mcclhip {

namespace {

// Vectors in flight per thread and operand.  Measured on MI355X over 96.5 M elements (fraction
// of the 8 TB/s peak): the binary folds are fastest with one (fold 0.81 against 0.78 with four,
// scale 0.86 against 0.77: a 1024-element tile per block keeps the set of tiles in flight one
// narrow address front); the ring fold with one for three ranks (0.76 against 0.73), eight for
// six and seven ranks (0.71 against 0.70) and four otherwise.
constexpr int kUnroll = 1;
constexpr int ring_unroll(int ws) { return ws == 3 ? 1 : ((ws == 6 || ws == 7) ? 8 : 4); }

template <bool NT>
__device__ __forceinline__ u4a load_vec_a(const u4a* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}
template <int ES, bool NT>
__device__ __forceinline__ u4a load_vec_u(const void* p) {
    if constexpr (ES == 4) {
        if constexpr (NT) return __builtin_nontemporal_load((const u4u4*)p);
        else return *(const u4u4*)p;
    } else {
        if constexpr (NT) return __builtin_nontemporal_load((const u4u2*)p);
        else return *(const u4u2*)p;
    }
}
template <bool NT>
__device__ __forceinline__ void store_vec_a(u4a* p, u4a v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// ---- one element / one dword -------------------------------------------------

// KIND: 0 dst (op) src, 1 (dst + src) * scale, 2 dst * scale (src unused)
template <int DT, int OP, int KIND>
__device__ __forceinline__ float fold_f32(float d, float s, float scale) {
    if constexpr (KIND == 0) return op_f32<OP>(d, s);
    else if constexpr (KIND == 1) return (d + s) * scale;  // two roundings: no contraction
    else return d * scale;
}

template <int DT, int OP, int KIND>
__device__ __forceinline__ uint32_t fold_dword(uint32_t d, uint32_t s, float scale) {
    if constexpr (DT == MCCL_HIP_F32) {
        return f2u(fold_f32<DT, OP, KIND>(u2f(d), u2f(s), scale));
    } else {
        float lo = fold_f32<DT, OP, KIND>(widen16<DT>(d & 0xFFFFu), widen16<DT>(s & 0xFFFFu), scale);
        float hi = fold_f32<DT, OP, KIND>(widen16<DT>(d >> 16), widen16<DT>(s >> 16), scale);
        return narrow16<DT>(lo) | (narrow16<DT>(hi) << 16);
    }
}

template <int DT, int OP, int KIND>
__device__ __forceinline__ void fold_elem(void* dst, const void* src, uint64_t i, float scale) {
    if constexpr (DT == MCCL_HIP_F32) {
        float* d = (float*)dst;
        float s = KIND == 2 ? 0.0f : ((const float*)src)[i];
        d[i] = fold_f32<DT, OP, KIND>(d[i], s, scale);
    } else {
        uint16_t* d = (uint16_t*)dst;
        float s = KIND == 2 ? 0.0f : widen16<DT>(((const uint16_t*)src)[i]);
        d[i] = (uint16_t)narrow16<DT>(fold_f32<DT, OP, KIND>(widen16<DT>(d[i]), s, scale));
    }
}

// ---- binary fold / scale / fused ----------------------------------------------
// Layout: [head scalars][nvec 16-byte vectors][tail scalars]; head makes the
// destination 16-byte aligned.
// block `block` of `nblocks` takes its share of one fold
template <int DT, int OP, int KIND, bool NT>
__device__ __forceinline__ void fold2_block(void* dst, const void* src, uint64_t n, float scale, uint32_t head,
                                            uint64_t nvec, uint32_t block, uint32_t nblocks) {
    constexpr int ES = ElemInfo<DT>::size;
    constexpr int EPV = ElemInfo<DT>::per_vec;
    u4a* dv = (u4a*)((char*)dst + (uint64_t)head * ES);
    const char* sv = (const char*)src + (uint64_t)head * ES;
    const uint64_t tile = (uint64_t)kBlock * kUnroll;
    for (uint64_t base = (uint64_t)block * tile; base < nvec; base += (uint64_t)nblocks * tile) {
        u4a d[kUnroll], s[kUnroll];
        if (base + tile <= nvec) {
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                uint64_t idx = base + (uint64_t)u * kBlock + threadIdx.x;
                d[u] = load_vec_a<NT>(dv + idx);
                if constexpr (KIND != 2) s[u] = load_vec_u<ES, NT>(sv + idx * 16);
                else s[u] = d[u];
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                uint64_t idx = base + (uint64_t)u * kBlock + threadIdx.x;
                u4a r;
#pragma unroll
                for (int q = 0; q < 4; q++) r[q] = fold_dword<DT, OP, KIND>(d[u][q], s[u][q], scale);
                store_vec_a<NT>(dv + idx, r);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                uint64_t idx = base + (uint64_t)u * kBlock + threadIdx.x;
                if (idx < nvec) {
                    u4a dd = load_vec_a<NT>(dv + idx);
                    u4a ss = dd;
                    if constexpr (KIND != 2) ss = load_vec_u<ES, NT>(sv + idx * 16);
                    u4a r;
#pragma unroll
                    for (int q = 0; q < 4; q++) r[q] = fold_dword<DT, OP, KIND>(dd[q], ss[q], scale);
                    store_vec_a<NT>(dv + idx, r);
                }
            }
        }
    }
    // scalar head and tail (fewer than EPV elements each)
    const uint64_t g = (uint64_t)block * kBlock + threadIdx.x;
    if (g < head) fold_elem<DT, OP, KIND>(dst, src, g, scale);
    const uint64_t tail = head + nvec * EPV;
    if (g < (uint64_t)EPV && tail + g < n) fold_elem<DT, OP, KIND>(dst, src, tail + g, scale);
}

template <int DT, int OP, int KIND, bool NT>
__global__ __launch_bounds__(kBlock) void k_fold2(void* dst, const void* src, uint64_t n,
                                                  float scale, uint32_t head, uint64_t nvec) {
    fold2_block<DT, OP, KIND, NT>(dst, src, n, scale, head, nvec, blockIdx.x, gridDim.x);
}

// ---- a list of independent binary folds in one launch ---------------------------
// blockIdx.y = fold, blockIdx.x strides over that fold's vectors.  The table is read where
// the launch put it, in the kernel-argument segment, through scalar loads (indexing the
// by-value parameter would make the compiler copy it to per-lane scratch memory first): it
// is therefore the only parameter.
constexpr int kFoldBatch = 128;  // folds per launch
struct FoldBatch {
    void* dst[kFoldBatch];
    const void* src[kFoldBatch];
    uint64_t n[kFoldBatch];
};
template <int DT, int OP, bool NT>
__global__ __launch_bounds__(kBlock) void k_fold2_batch(FoldBatch) {
    typedef const __attribute__((address_space(4))) FoldBatch* Arg;
    const Arg fb = (Arg)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int ES = ElemInfo<DT>::size;
    constexpr int EPV = ElemInfo<DT>::per_vec;
    void* dst = fb->dst[blockIdx.y];
    const void* src = fb->src[blockIdx.y];
    const uint64_t n = fb->n[blockIdx.y];
    uint64_t head = ((16 - ((uintptr_t)dst & 15)) & 15) / ES;
    if (head > n) head = n;
    const uint64_t nvec = (n - head) / EPV;
    fold2_block<DT, OP, 0, NT>(dst, src, n, 1.0f, (uint32_t)head, nvec, blockIdx.x, gridDim.x);
}

// ---- integral types (DDP metadata, counters): plain grid-stride ---------------
// Wrap-around arithmetic, bool folded as raw uint8
// (csrc/metal/AccelerateOps.mm:206-236, csrc/metal/shaders.metal:554-731).
template <typename T, int OP>
__device__ __forceinline__ T fold_int(T d, T s) {
    typedef typename std::make_unsigned<T>::type UT;
    if constexpr (OP == kAdd) return (T)((UT)d + (UT)s);
    else if constexpr (OP == kMul) return (T)((UT)d * (UT)s);
    else if constexpr (OP == kMin) return s < d ? s : d;
    else return s > d ? s : d;
}
template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void k_fold2_int(T* dst, const T* src, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        dst[i] = fold_int<T, OP>(dst[i], src[i]);
}
template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void k_fold2_batch_int(FoldBatch) {
    typedef const __attribute__((address_space(4))) FoldBatch* Arg;
    const Arg fb = (Arg)__builtin_amdgcn_kernarg_segment_ptr();
    T* dst = (T*)fb->dst[blockIdx.y];
    const T* src = (const T*)fb->src[blockIdx.y];
    const uint64_t n = fb->n[blockIdx.y];
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        dst[i] = fold_int<T, OP>(dst[i], src[i]);
}

// T(float(x) * scale): int32 rounds half away from zero, int64 / uint8 truncate
// (csrc/metal/shaders.metal:622-665).
template <typename T>
__global__ __launch_bounds__(kBlock) void k_scale_int(T* buf, uint64_t n, float scale) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        float v = (float)buf[i] * scale;
        if constexpr (sizeof(T) == 4) buf[i] = (T)roundf(v);
        else buf[i] = (T)v;
    }
}

// ---- W-way fold in ring-step order --------------------------------------------
// in[i] = buffer of rank i % ws for i < 2 * ws: the ws buffers in ring order
// starting at any rank are ws consecutive entries, which a block fetches with
// one wide scalar load instead of ws dependent ones.
struct RingPtrs {
    const void* in[2 * MCCL_HIP_MAX_WORLD];
};

// blockIdx.y = bucket * nchunks + chunk.  Each block row folds one chunk of one
// bucket, so the first rank of the fold is uniform over the block.
// WSC > 0 fixes the world size at compile time, so the rank loop unrolls and
// all WSC * ring_unroll(WSC) loads of a thread are in flight together; WSC == 0 reads
// it at run time.
template <int DT, int OP, bool NT, int WSC>
__global__ __launch_bounds__(kBlock) void k_ring_fold(void* out, RingPtrs ptrs, int ws_rt,
                                                      uint64_t n_total, uint64_t bucket_elems,
                                                      int schedule, uint32_t nchunks, float scale,
                                                      int apply_scale, int stepwise) {
    constexpr int ES = ElemInfo<DT>::size;
    constexpr int EPV = ElemInfo<DT>::per_vec;
    constexpr int U = ring_unroll(WSC);
    const int ws = WSC > 0 ? WSC : ws_rt;
    const uint32_t bucket = blockIdx.y / nchunks;
    const uint32_t c = blockIdx.y - bucket * nchunks;
    const uint64_t bstart = (uint64_t)bucket * bucket_elems;
    const uint64_t bn = (n_total - bstart) < bucket_elems ? (n_total - bstart) : bucket_elems;
    const uint64_t ce = (bn + nchunks - 1) / nchunks;
    const uint64_t cstart = (uint64_t)c * ce;
    if (cstart >= bn) return;
    const uint64_t len = (bn - cstart) < ce ? (bn - cstart) : ce;
    const uint64_t e0 = bstart + cstart;  // first element of the chunk in every buffer
    const int first = (schedule == MCCL_HIP_RING_CHUNKED) ? (int)(((c + 1) >> 1) % (uint32_t)ws)
                                                          : (int)(c % (uint32_t)ws);

    char* o = (char*)out + e0 * ES;
    uint64_t head = ((16 - ((uintptr_t)o & 15)) & 15) / ES;
    if (head > len) head = len;
    const uint64_t nvec = (len - head) / EPV;
    const uint64_t voff = (e0 + head) * ES;  // byte offset of the vector body
    u4a* ov = (u4a*)((char*)out + voff);

    const uint64_t tile = (uint64_t)kBlock * U;
    const void* rp[WSC > 0 ? WSC : 1];  // rank buffers in fold order (compile-time world sizes)
    if constexpr (WSC > 0) {
#pragma unroll
        for (int j = 0; j < WSC; j++) rp[j] = ptrs.in[first + j];
    }
    auto rank_ptr = [&](int j, int r) -> const char* {
        if constexpr (WSC > 0) return (const char*)rp[j];
        else return (const char*)ptrs.in[r];
    };
    for (uint64_t base = (uint64_t)blockIdx.x * tile; base < nvec; base += (uint64_t)gridDim.x * tile) {
        if constexpr (DT == MCCL_HIP_F32) {
            float acc[U][4];
            uint64_t idx[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                idx[u] = base + (uint64_t)u * kBlock + threadIdx.x;
                if (idx[u] >= nvec) idx[u] = nvec - 1;  // clamp: recomputes a valid vector, store is guarded
            }
            {
                const char* p = rank_ptr(0, first) + voff;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    u4a v = load_vec_u<ES, NT>(p + idx[u] * 16);
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[u][q] = u2f(v[q]);
                }
            }
            int r = first;
#pragma unroll
            for (int j = 1; j < ws; j++) {
                r = (r + 1 == ws) ? 0 : r + 1;
                const char* p = rank_ptr(j, r) + voff;
                u4a v[U];
#pragma unroll
                for (int u = 0; u < U; u++) v[u] = load_vec_u<ES, NT>(p + idx[u] * 16);
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int q = 0; q < 4; q++) acc[u][q] = op_f32<OP>(u2f(v[u][q]), acc[u][q]);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                u4a rv;
#pragma unroll
                for (int q = 0; q < 4; q++) rv[q] = f2u(apply_scale ? acc[u][q] * scale : acc[u][q]);
                if (base + (uint64_t)u * kBlock + threadIdx.x < nvec) store_vec_a<NT>(ov + idx[u], rv);
            }
        } else {
            float acc[U][8];
            uint64_t idx[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                idx[u] = base + (uint64_t)u * kBlock + threadIdx.x;
                if (idx[u] >= nvec) idx[u] = nvec - 1;
            }
            {
                const char* p = rank_ptr(0, first) + voff;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    u4a v = load_vec_u<ES, NT>(p + idx[u] * 16);
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        acc[u][2 * q] = widen16<DT>(v[q] & 0xFFFFu);
                        acc[u][2 * q + 1] = widen16<DT>(v[q] >> 16);
                    }
                }
            }
            int r = first;
#pragma unroll
            for (int j = 1; j < ws; j++) {
                r = (r + 1 == ws) ? 0 : r + 1;
                const char* p = rank_ptr(j, r) + voff;
                u4a v[U];
#pragma unroll
                for (int u = 0; u < U; u++) v[u] = load_vec_u<ES, NT>(p + idx[u] * 16);
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        float lo = op_f32<OP>(widen16<DT>(v[u][q] & 0xFFFFu), acc[u][2 * q]);
                        float hi = op_f32<OP>(widen16<DT>(v[u][q] >> 16), acc[u][2 * q + 1]);
                        if (stepwise) {
                            lo = widen16<DT>(narrow16<DT>(lo));
                            hi = widen16<DT>(narrow16<DT>(hi));
                        }
                        acc[u][2 * q] = lo;
                        acc[u][2 * q + 1] = hi;
                    }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                u4a rv;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    float lo = apply_scale ? acc[u][2 * q] * scale : acc[u][2 * q];
                    float hi = apply_scale ? acc[u][2 * q + 1] * scale : acc[u][2 * q + 1];
                    rv[q] = narrow16<DT>(lo) | (narrow16<DT>(hi) << 16);
                }
                if (base + (uint64_t)u * kBlock + threadIdx.x < nvec) store_vec_a<NT>(ov + idx[u], rv);
            }
        }
    }

    // scalar head and tail of the chunk
    const uint64_t g = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t tail = head + nvec * EPV;
    uint64_t i = len;  // element (relative to the chunk) this thread folds, if any
    if (g < head) i = g;
    else if (g >= (uint64_t)EPV && g < 2u * EPV && tail + (g - EPV) < len) i = tail + (g - EPV);
    if (i < len) {
        const uint64_t e = e0 + i;
        float acc;
        if constexpr (DT == MCCL_HIP_F32) acc = ((const float*)ptrs.in[first])[e];
        else acc = widen16<DT>(((const uint16_t*)ptrs.in[first])[e]);
        int r = first;
        for (int j = 1; j < ws; j++) {
            r = (r + 1 == ws) ? 0 : r + 1;
            float x;
            if constexpr (DT == MCCL_HIP_F32) x = ((const float*)ptrs.in[r])[e];
            else x = widen16<DT>(((const uint16_t*)ptrs.in[r])[e]);
            acc = op_f32<OP>(x, acc);
            if constexpr (DT != MCCL_HIP_F32)
                if (stepwise) acc = widen16<DT>(narrow16<DT>(acc));
        }
        if (apply_scale) acc = acc * scale;
        if constexpr (DT == MCCL_HIP_F32) ((float*)out)[e] = acc;
        else ((uint16_t*)out)[e] = (uint16_t)narrow16<DT>(acc);
    }
}

// ---- launch helpers -----------------------------------------------------------

// One tile per block wherever possible: measured on MI355X, 16 K short-lived blocks
// in address order stream faster (6.38 TB/s for the binary fold) than a persistent
// grid of 2 K blocks striding through the array (6.20 TB/s).  The cap only bounds
// the grid for very large arrays; the kernels stride when it applies.
uint32_t stream_blocks(uint64_t work_tiles) {
    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    return clamp_u32(work_tiles, 1, cap);
}

template <int DT, int OP, int KIND>
int launch_fold2_t(void* dst, const void* src, uint64_t n, float scale, hipStream_t st) {
    constexpr int ES = ElemInfo<DT>::size;
    constexpr int EPV = ElemInfo<DT>::per_vec;
    uint64_t head = ((16 - ((uintptr_t)dst & 15)) & 15) / ES;
    if (head > n) head = n;
    const uint64_t nvec = (n - head) / EPV;
    const uint64_t tile = (uint64_t)kBlock * kUnroll;
    const uint32_t blocks = stream_blocks((nvec + tile - 1) / tile);
    if (tuning().nontemporal)
        k_fold2<DT, OP, KIND, true><<<blocks, kBlock, 0, st>>>(dst, src, n, scale, (uint32_t)head, nvec);
    else
        k_fold2<DT, OP, KIND, false><<<blocks, kBlock, 0, st>>>(dst, src, n, scale, (uint32_t)head, nvec);
    return launch_status();
}

template <int DT>
int launch_fold2_dt(void* dst, const void* src, uint64_t n, int opi, hipStream_t st) {
    switch (opi) {
        case kAdd: return launch_fold2_t<DT, kAdd, 0>(dst, src, n, 1.0f, st);
        case kMul: return launch_fold2_t<DT, kMul, 0>(dst, src, n, 1.0f, st);
        case kMin: return launch_fold2_t<DT, kMin, 0>(dst, src, n, 1.0f, st);
        default: return launch_fold2_t<DT, kMax, 0>(dst, src, n, 1.0f, st);
    }
}

template <typename T>
int launch_fold2_int(void* dst, const void* src, uint64_t n, int opi, hipStream_t st) {
    const uint32_t blocks = stream_blocks((n + kBlock - 1) / kBlock);
    switch (opi) {
        case kAdd: k_fold2_int<T, kAdd><<<blocks, kBlock, 0, st>>>((T*)dst, (const T*)src, n); break;
        case kMul: k_fold2_int<T, kMul><<<blocks, kBlock, 0, st>>>((T*)dst, (const T*)src, n); break;
        case kMin: k_fold2_int<T, kMin><<<blocks, kBlock, 0, st>>>((T*)dst, (const T*)src, n); break;
        default: k_fold2_int<T, kMax><<<blocks, kBlock, 0, st>>>((T*)dst, (const T*)src, n); break;
    }
    return launch_status();
}

// One launch per kFoldBatch folds.  x covers the longest fold of the launch (shorter folds' surplus
// blocks leave at once), capped so that the whole grid stays within the streaming kernels' bound.
template <class Launch>
int launch_batches(void* const* dsts, const void* const* srcs, const uint64_t* counts, uint32_t nfolds,
                   uint64_t elems_per_block, Launch&& launch) {
    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    FoldBatch fb;
    uint32_t m = 0;
    uint64_t longest = 0;
    auto flush = [&]() {
        if (m == 0) return;
        for (uint32_t i = m; i < (uint32_t)kFoldBatch; i++) { fb.dst[i] = nullptr; fb.src[i] = nullptr; fb.n[i] = 0; }
        const uint64_t want = (longest + elems_per_block - 1) / elems_per_block;
        launch(fb, dim3(clamp_u32(want, 1, cap / m > 0 ? cap / m : 1), m, 1));
        m = 0;
        longest = 0;
    };
    for (uint32_t i = 0; i < nfolds; i++) {
        if (counts[i] == 0) continue;
        fb.dst[m] = dsts[i];
        fb.src[m] = srcs[i];
        fb.n[m] = counts[i];
        longest = counts[i] > longest ? counts[i] : longest;
        if (++m == (uint32_t)kFoldBatch) flush();
    }
    flush();
    return launch_status();
}

template <int DT, int OP>
int launch_fold2_batch_t(void* const* dsts, const void* const* srcs, const uint64_t* counts, uint32_t nfolds,
                         hipStream_t st) {
    const uint64_t per_block = (uint64_t)kBlock * kUnroll * ElemInfo<DT>::per_vec;
    const bool nt = tuning().nontemporal != 0;
    return launch_batches(dsts, srcs, counts, nfolds, per_block, [&](const FoldBatch& fb, dim3 grid) {
        if (nt) k_fold2_batch<DT, OP, true><<<grid, kBlock, 0, st>>>(fb);
        else k_fold2_batch<DT, OP, false><<<grid, kBlock, 0, st>>>(fb);
    });
}
template <int DT>
int launch_fold2_batch_dt(void* const* dsts, const void* const* srcs, const uint64_t* counts, uint32_t nfolds,
                          int opi, hipStream_t st) {
    switch (opi) {
        case kAdd: return launch_fold2_batch_t<DT, kAdd>(dsts, srcs, counts, nfolds, st);
        case kMul: return launch_fold2_batch_t<DT, kMul>(dsts, srcs, counts, nfolds, st);
        case kMin: return launch_fold2_batch_t<DT, kMin>(dsts, srcs, counts, nfolds, st);
        default: return launch_fold2_batch_t<DT, kMax>(dsts, srcs, counts, nfolds, st);
    }
}
template <typename T>
int launch_fold2_batch_int(void* const* dsts, const void* const* srcs, const uint64_t* counts, uint32_t nfolds,
                           int opi, hipStream_t st) {
    return launch_batches(dsts, srcs, counts, nfolds, kBlock, [&](const FoldBatch& fb, dim3 grid) {
        switch (opi) {
            case kAdd: k_fold2_batch_int<T, kAdd><<<grid, kBlock, 0, st>>>(fb); break;
            case kMul: k_fold2_batch_int<T, kMul><<<grid, kBlock, 0, st>>>(fb); break;
            case kMin: k_fold2_batch_int<T, kMin><<<grid, kBlock, 0, st>>>(fb); break;
            default: k_fold2_batch_int<T, kMax><<<grid, kBlock, 0, st>>>(fb); break;
        }
    });
}

template <typename T>
int launch_scale_int(void* buf, uint64_t n, float scale, hipStream_t st) {
    const uint32_t blocks = stream_blocks((n + kBlock - 1) / kBlock);
    k_scale_int<T><<<blocks, kBlock, 0, st>>>((T*)buf, n, scale);
    return launch_status();
}

template <int DT, int OP>
int launch_ring_t(void* out, const RingPtrs& ptrs, int ws, uint64_t n_total, uint64_t bucket_elems,
                  int schedule, uint32_t nchunks, uint32_t nbuckets, float scale, int apply_scale,
                  int stepwise, hipStream_t st) {
    constexpr int EPV = ElemInfo<DT>::per_vec;
    const uint64_t bn = bucket_elems < n_total ? bucket_elems : n_total;
    const uint64_t ce = (bn + nchunks - 1) / nchunks;
    const uint64_t tile_vecs = (uint64_t)kBlock * ring_unroll(ws >= 2 && ws <= 8 ? ws : 0);
    const uint64_t tiles = (ce / EPV + tile_vecs - 1) / tile_vecs;
    const uint64_t rows = (uint64_t)nchunks * nbuckets;
    // One tile per block, x fastest: blocks are dispatched in address order, so
    // the set of tiles in flight is one contiguous front per rank buffer.  A
    // persistent grid looping inside each chunk row scatters the front over all
    // rows and costs about 13 % of the bandwidth on MI355X.
    uint64_t per_row = tiles < 1 ? 1 : tiles;
    if (per_row > 0x7FFFFFFFull) per_row = 0x7FFFFFFFull;
    dim3 grid((uint32_t)per_row, (uint32_t)rows, 1);
#define MCCLHIP_RING_LAUNCH(NT, WSC)                                                                  \
    k_ring_fold<DT, OP, NT, WSC><<<grid, kBlock, 0, st>>>(out, ptrs, ws, n_total, bucket_elems, schedule, \
                                                          nchunks, scale, apply_scale, stepwise)
    const bool nt = tuning().nontemporal != 0;
    switch (ws) {
        // world sizes 2..8 have an unrolled instance each: all loads of a thread are in flight
        // before the first add (the run-time loop measured 0.69 of peak at 6 ranks)
        case 2: if (nt) MCCLHIP_RING_LAUNCH(true, 2); else MCCLHIP_RING_LAUNCH(false, 2); break;
        case 3: if (nt) MCCLHIP_RING_LAUNCH(true, 3); else MCCLHIP_RING_LAUNCH(false, 3); break;
        case 4: if (nt) MCCLHIP_RING_LAUNCH(true, 4); else MCCLHIP_RING_LAUNCH(false, 4); break;
        case 5: if (nt) MCCLHIP_RING_LAUNCH(true, 5); else MCCLHIP_RING_LAUNCH(false, 5); break;
        case 6: if (nt) MCCLHIP_RING_LAUNCH(true, 6); else MCCLHIP_RING_LAUNCH(false, 6); break;
        case 7: if (nt) MCCLHIP_RING_LAUNCH(true, 7); else MCCLHIP_RING_LAUNCH(false, 7); break;
        case 8: if (nt) MCCLHIP_RING_LAUNCH(true, 8); else MCCLHIP_RING_LAUNCH(false, 8); break;
        default: if (nt) MCCLHIP_RING_LAUNCH(true, 0); else MCCLHIP_RING_LAUNCH(false, 0); break;
    }
#undef MCCLHIP_RING_LAUNCH
    return launch_status();
}

template <int DT>
int launch_ring_dt(void* out, const RingPtrs& p, int ws, uint64_t n_total, uint64_t bucket_elems,
                   int schedule, uint32_t nchunks, uint32_t nbuckets, int opi, float scale,
                   int apply_scale, int stepwise, hipStream_t st) {
    switch (opi) {
        case kAdd: return launch_ring_t<DT, kAdd>(out, p, ws, n_total, bucket_elems, schedule, nchunks, nbuckets, scale, apply_scale, stepwise, st);
        case kMul: return launch_ring_t<DT, kMul>(out, p, ws, n_total, bucket_elems, schedule, nchunks, nbuckets, scale, apply_scale, stepwise, st);
        case kMin: return launch_ring_t<DT, kMin>(out, p, ws, n_total, bucket_elems, schedule, nchunks, nbuckets, scale, apply_scale, stepwise, st);
        default: return launch_ring_t<DT, kMax>(out, p, ws, n_total, bucket_elems, schedule, nchunks, nbuckets, scale, apply_scale, stepwise, st);
    }
}

int check_common(const void* a, uint64_t n) {
    if (n == 0) return 1;  // nothing to do
    if (!a || n > MCCL_HIP_MAX_ELEMS) return MCCL_HIP_ERR_ARG;
    return 0;
}

}  // namespace
}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

int mccl_hip_fold2(void* dst, const void* src, uint64_t n, int dtype, int op, void* stream) {
    const int opi = op_index(op);
    if (opi < 0) return MCCL_HIP_ERR_OP;
    int c = check_common(dst, n);
    if (c) return c < 0 ? c : MCCL_HIP_OK;
    if (!src) return MCCL_HIP_ERR_ARG;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case MCCL_HIP_F32: return launch_fold2_dt<MCCL_HIP_F32>(dst, src, n, opi, st);
        case MCCL_HIP_F16: return launch_fold2_dt<MCCL_HIP_F16>(dst, src, n, opi, st);
        case MCCL_HIP_BF16: return launch_fold2_dt<MCCL_HIP_BF16>(dst, src, n, opi, st);
        case MCCL_HIP_I32: return launch_fold2_int<int32_t>(dst, src, n, opi, st);
        case MCCL_HIP_I64: return launch_fold2_int<int64_t>(dst, src, n, opi, st);
        case MCCL_HIP_BOOL:
        case MCCL_HIP_U8: return launch_fold2_int<uint8_t>(dst, src, n, opi, st);
        default: return MCCL_HIP_ERR_DTYPE;
    }
}

int mccl_hip_fold2_batch(void* const* host_dsts, const void* const* host_srcs, const uint64_t* host_counts,
                         uint32_t nfolds, int dtype, int op, void* stream) {
    const int opi = op_index(op);
    if (opi < 0) return MCCL_HIP_ERR_OP;
    if (nfolds == 0) return MCCL_HIP_OK;
    if (!host_dsts || !host_srcs || !host_counts) return MCCL_HIP_ERR_ARG;
    int es;
    switch (dtype) {
        case MCCL_HIP_F32: case MCCL_HIP_I32: es = 4; break;
        case MCCL_HIP_F16: case MCCL_HIP_BF16: es = 2; break;
        case MCCL_HIP_I64: es = 8; break;
        case MCCL_HIP_BOOL: case MCCL_HIP_U8: es = 1; break;
        default: return MCCL_HIP_ERR_DTYPE;
    }
    for (uint32_t i = 0; i < nfolds; i++) {
        if (host_counts[i] == 0) continue;
        if (!host_dsts[i] || !host_srcs[i] || host_counts[i] > MCCL_HIP_MAX_ELEMS) return MCCL_HIP_ERR_ARG;
    }
    // the folds of one call run in no particular order: a destination may not overlap any other
    // fold's destination or source
    for (uint32_t i = 0; i < nfolds; i++) {
        if (host_counts[i] == 0) continue;
        const uintptr_t d0 = (uintptr_t)host_dsts[i], d1 = d0 + host_counts[i] * (uint64_t)es;
        for (uint32_t j = 0; j < nfolds; j++) {
            if (j == i || host_counts[j] == 0) continue;
            const uint64_t bytes = host_counts[j] * (uint64_t)es;
            const uintptr_t a0 = (uintptr_t)host_dsts[j], b0 = (uintptr_t)host_srcs[j];
            if ((d0 < a0 + bytes && a0 < d1) || (d0 < b0 + bytes && b0 < d1)) return MCCL_HIP_ERR_ARG;
        }
    }
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case MCCL_HIP_F32: return launch_fold2_batch_dt<MCCL_HIP_F32>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
        case MCCL_HIP_F16: return launch_fold2_batch_dt<MCCL_HIP_F16>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
        case MCCL_HIP_BF16: return launch_fold2_batch_dt<MCCL_HIP_BF16>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
        case MCCL_HIP_I32: return launch_fold2_batch_int<int32_t>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
        case MCCL_HIP_I64: return launch_fold2_batch_int<int64_t>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
        default: return launch_fold2_batch_int<uint8_t>(host_dsts, host_srcs, host_counts, nfolds, opi, st);
    }
}

int mccl_hip_scale(void* buf, uint64_t n, int dtype, float scale, void* stream) {
    int c = check_common(buf, n);
    if (c) return c < 0 ? c : MCCL_HIP_OK;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case MCCL_HIP_F32: return launch_fold2_t<MCCL_HIP_F32, kAdd, 2>(buf, nullptr, n, scale, st);
        case MCCL_HIP_F16: return launch_fold2_t<MCCL_HIP_F16, kAdd, 2>(buf, nullptr, n, scale, st);
        case MCCL_HIP_BF16: return launch_fold2_t<MCCL_HIP_BF16, kAdd, 2>(buf, nullptr, n, scale, st);
        case MCCL_HIP_I32: return launch_scale_int<int32_t>(buf, n, scale, st);
        case MCCL_HIP_I64: return launch_scale_int<int64_t>(buf, n, scale, st);
        case MCCL_HIP_BOOL:
        case MCCL_HIP_U8: return launch_scale_int<uint8_t>(buf, n, scale, st);
        default: return MCCL_HIP_ERR_DTYPE;
    }
}

int mccl_hip_fold2_scale(void* dst, const void* src, uint64_t n, int dtype, float scale,
                         void* stream) {
    int c = check_common(dst, n);
    if (c) return c < 0 ? c : MCCL_HIP_OK;
    if (!src) return MCCL_HIP_ERR_ARG;
    int rc = mccl_hip_init();
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case MCCL_HIP_F32: return launch_fold2_t<MCCL_HIP_F32, kAdd, 1>(dst, src, n, scale, st);
        case MCCL_HIP_F16: return launch_fold2_t<MCCL_HIP_F16, kAdd, 1>(dst, src, n, scale, st);
        case MCCL_HIP_BF16: return launch_fold2_t<MCCL_HIP_BF16, kAdd, 1>(dst, src, n, scale, st);
        case MCCL_HIP_I32:
        case MCCL_HIP_I64:
        case MCCL_HIP_BOOL:
        case MCCL_HIP_U8:
            // Integral AVG: the add kernel then the scale kernel, as the
            // reference does (csrc/metal/MetalKernels.mm:629-635).
            rc = mccl_hip_fold2(dst, src, n, dtype, MCCL_HIP_SUM, stream);
            if (rc) return rc;
            return mccl_hip_scale(dst, n, dtype, scale, stream);
        default: return MCCL_HIP_ERR_DTYPE;
    }
}

int mccl_hip_ring_fold(void* out, const void* const* host_in, int ws, uint64_t n_total,
                       uint64_t bucket_elems, int schedule, int dtype, int op, int apply_scale,
                       float scale, int stepwise, void* stream) {
    const int opi = op_index(op);
    if (opi < 0) return MCCL_HIP_ERR_OP;
    if (dtype != MCCL_HIP_F32 && dtype != MCCL_HIP_F16 && dtype != MCCL_HIP_BF16) return MCCL_HIP_ERR_DTYPE;
    if (ws < 1 || ws > MCCL_HIP_MAX_WORLD || !host_in) return MCCL_HIP_ERR_ARG;
    if (schedule != MCCL_HIP_RING_BASIC && schedule != MCCL_HIP_RING_CHUNKED) return MCCL_HIP_ERR_ARG;
    int c = check_common(out, n_total);
    if (c) return c < 0 ? c : MCCL_HIP_OK;
    if (bucket_elems == 0) return MCCL_HIP_ERR_ARG;
    RingPtrs ptrs;
    for (int r = 0; r < 2 * MCCL_HIP_MAX_WORLD; r++) ptrs.in[r] = nullptr;
    for (int r = 0; r < ws; r++) {
        if (!host_in[r]) return MCCL_HIP_ERR_ARG;
        ptrs.in[r] = host_in[r];
        ptrs.in[ws + r] = host_in[r];
    }
    int rc = mccl_hip_init();
    if (rc) return rc;
    if (bucket_elems > n_total) bucket_elems = n_total;
    const uint64_t nbuckets64 = (n_total + bucket_elems - 1) / bucket_elems;
    const uint32_t nchunks = (uint32_t)(schedule == MCCL_HIP_RING_CHUNKED ? 2 * ws : ws);
    if (nbuckets64 * nchunks > 65535) return MCCL_HIP_ERR_ARG;  // grid rows
    const uint32_t nb = (uint32_t)nbuckets64;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case MCCL_HIP_F32: return launch_ring_dt<MCCL_HIP_F32>(out, ptrs, ws, n_total, bucket_elems, schedule, nchunks, nb, opi, scale, apply_scale, stepwise, st);
        case MCCL_HIP_F16: return launch_ring_dt<MCCL_HIP_F16>(out, ptrs, ws, n_total, bucket_elems, schedule, nchunks, nb, opi, scale, apply_scale, stepwise, st);
        default: return launch_ring_dt<MCCL_HIP_BF16>(out, ptrs, ws, n_total, bucket_elems, schedule, nchunks, nb, opi, scale, apply_scale, stepwise, st);
    }
}

}  // extern "C"
