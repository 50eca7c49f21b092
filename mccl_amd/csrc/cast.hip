// fp32 <-> fp16 transport casts of the FP16 compressor for gfx950
// (csrc/compression/FP16Compression.cpp:16-112).
//
// Semantics are those of the reference's target platform (its NEON branch):
// IEEE round-to-nearest-even with gradual underflow, overflow to infinity, and
// NaN kept NaN with the top mantissa bits and the quiet bit set
// (sign | 0x7C00 | mant >> 13 | 0x200, the rule its portable branch spells out
// at :47-51).  The portable branch (:38-73, :96-111: the one a non-ARM build of
// the reference runs) differs in two places: half subnormals are flushed to
// zero in both directions, and widening passes a NaN's mantissa bits through
// without setting the quiet bit.  The tuning key "fp16_portable" selects that
// behaviour, for bit-identical results with such a build.
//
// Both kernels stream with one tile per block in address order.  Narrowing
// handles 8 elements per lane (two 16-byte loads, one 16-byte store).
#include "common.hip.h"
#include "runtime.h"

namespace mcclhip {

namespace {

__device__ __forceinline__ uint32_t f32_to_f16_transport(uint32_t bits) {
    const float f = u2f(bits);
    _Float16 v = (_Float16)f;
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    uint32_t r = h;
    if (f != f) r = ((bits >> 16) & 0x8000u) | 0x7C00u | ((bits & 0x7FFFFFu) >> 13) | 0x200u;
    return r;
}

// The portable branch: anything below the smallest normal half becomes a signed zero, also
// what round-to-nearest would have carried up to it.
__device__ __forceinline__ uint32_t f32_to_f16_portable(uint32_t bits) {
    if (((bits >> 23) & 0xFFu) <= 112u) return (bits >> 16) & 0x8000u;
    return f32_to_f16_transport(bits);
}

__device__ __forceinline__ uint32_t f16_to_f32_portable(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0) return sign;
    if (e == 31) return sign | 0x7F800000u | (m << 13);
    return sign | ((e + 112u) << 23) | (m << 13);
}

template <bool PORTABLE>
__device__ __forceinline__ uint32_t narrow_transport(uint32_t bits) {
    return PORTABLE ? f32_to_f16_portable(bits) : f32_to_f16_transport(bits);
}

template <bool PORTABLE>
__device__ __forceinline__ uint32_t widen_transport(uint32_t h) {
    return PORTABLE ? f16_to_f32_portable(h) : f2u(widen_f16(h));
}

template <bool PORTABLE>
__global__ __launch_bounds__(kBlock) void k_cast_f32_f16(const float* __restrict__ src, uint16_t* __restrict__ dst,
                                                         uint64_t n) {
    const uint64_t ngrp = n / 8;  // groups of 8 elements
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < ngrp; i += (uint64_t)gridDim.x * kBlock) {
        const u4a a = __builtin_nontemporal_load((const u4u4*)(src + i * 8));
        const u4a b = __builtin_nontemporal_load((const u4u4*)(src + i * 8 + 4));
        u4a o;
        o[0] = narrow_transport<PORTABLE>(a[0]) | (narrow_transport<PORTABLE>(a[1]) << 16);
        o[1] = narrow_transport<PORTABLE>(a[2]) | (narrow_transport<PORTABLE>(a[3]) << 16);
        o[2] = narrow_transport<PORTABLE>(b[0]) | (narrow_transport<PORTABLE>(b[1]) << 16);
        o[3] = narrow_transport<PORTABLE>(b[2]) | (narrow_transport<PORTABLE>(b[3]) << 16);
        __builtin_nontemporal_store(o, (u4u2*)(dst + i * 8));
    }
    const uint64_t g = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (g < 8 && ngrp * 8 + g < n) dst[ngrp * 8 + g] = (uint16_t)narrow_transport<PORTABLE>(f2u(src[ngrp * 8 + g]));
}

// Widening writes twice what it reads, so the layout follows the stores: a lane
// owns 4 consecutive elements (one 8-byte load, one 16-byte store) and a wave's
// store covers 1 KiB of consecutive addresses; kWidenQuads such groups per lane,
// a block apart, keep several loads in flight (measured on the 96.5 M-element
// gradient: 1 group 6.11, 2 groups 6.24, 4 groups 5.84, 8 groups 5.50 TB/s).
constexpr int kWidenQuads = 2;

template <bool PORTABLE>
__global__ __launch_bounds__(kBlock) void k_cast_f16_f32(const uint16_t* __restrict__ src, float* __restrict__ dst,
                                                         uint64_t n) {
    const uint64_t nquad = n / 4;
    for (uint64_t base = (uint64_t)blockIdx.x * (kBlock * kWidenQuads); base < nquad;
         base += (uint64_t)gridDim.x * (kBlock * kWidenQuads)) {
        u2a h[kWidenQuads];
#pragma unroll
        for (int j = 0; j < kWidenQuads; j++) {
            const uint64_t q = base + (uint64_t)j * kBlock + threadIdx.x;
            if (q < nquad) h[j] = __builtin_nontemporal_load((const u2u2*)(src + q * 4));
        }
#pragma unroll
        for (int j = 0; j < kWidenQuads; j++) {
            const uint64_t q = base + (uint64_t)j * kBlock + threadIdx.x;
            if (q < nquad) {
                u4a o;
                o[0] = widen_transport<PORTABLE>(h[j][0] & 0xFFFFu); o[1] = widen_transport<PORTABLE>(h[j][0] >> 16);
                o[2] = widen_transport<PORTABLE>(h[j][1] & 0xFFFFu); o[3] = widen_transport<PORTABLE>(h[j][1] >> 16);
                __builtin_nontemporal_store(o, (u4u4*)(dst + q * 4));
            }
        }
    }
    const uint64_t g = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (g < 4 && nquad * 4 + g < n) dst[nquad * 4 + g] = u2f(widen_transport<PORTABLE>(src[nquad * 4 + g]));
}

uint32_t cast_blocks(uint64_t n, uint64_t per_block) {
    const uint64_t cap = (uint64_t)device_info().num_cus * (uint64_t)tuning().fold_blocks_per_cu;
    return clamp_u32((n + per_block - 1) / per_block, 1, cap);
}

}  // namespace
}  // namespace mcclhip

using namespace mcclhip;

extern "C" {

int mccl_hip_cast_f32_to_f16(const float* src, void* dst, uint64_t n, void* stream) {
    if (n == 0) return MCCL_HIP_OK;
    if (!src || !dst || n > MCCL_HIP_MAX_ELEMS || ((uintptr_t)src & 3) || ((uintptr_t)dst & 1)) return MCCL_HIP_ERR_ARG;
    int rc = mccl_hip_init();
    if (rc) return rc;
    if (tuning().fp16_portable)
        k_cast_f32_f16<true><<<cast_blocks(n, 8 * kBlock), kBlock, 0, (hipStream_t)stream>>>(src, (uint16_t*)dst, n);
    else
        k_cast_f32_f16<false><<<cast_blocks(n, 8 * kBlock), kBlock, 0, (hipStream_t)stream>>>(src, (uint16_t*)dst, n);
    return launch_status();
}

int mccl_hip_cast_f16_to_f32(const void* src, float* dst, uint64_t n, void* stream) {
    if (n == 0) return MCCL_HIP_OK;
    if (!src || !dst || n > MCCL_HIP_MAX_ELEMS || ((uintptr_t)dst & 3) || ((uintptr_t)src & 1)) return MCCL_HIP_ERR_ARG;
    int rc = mccl_hip_init();
    if (rc) return rc;
    if (tuning().fp16_portable)
        k_cast_f16_f32<true><<<cast_blocks(n, 4 * kBlock * kWidenQuads), kBlock, 0, (hipStream_t)stream>>>((const uint16_t*)src, dst, n);
    else
        k_cast_f16_f32<false><<<cast_blocks(n, 4 * kBlock * kWidenQuads), kBlock, 0, (hipStream_t)stream>>>((const uint16_t*)src, dst, n);
    return launch_status();
}

}  // extern "C"
