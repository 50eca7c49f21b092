// Shared device helpers for the gfx950 kernels: 16-byte vector types, the fp32
// op set, fp16/bf16 widen and round-to-nearest-even narrow, wave/block scans.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mccl_hip.h"

namespace mcclhip {

constexpr int kBlock = 256;  // 4 wavefronts of 64 lanes
constexpr int kWave = 64;

// Four dwords moved by one global_load/store_dwordx4.  The `u` forms only
// promise element alignment: gfx950 issues the same 16-byte access and the
// memory pipeline splits it when the address is not 16-byte aligned.
typedef uint32_t u4a __attribute__((ext_vector_type(4)));
typedef uint32_t u4u4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u4u2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u2a __attribute__((ext_vector_type(2)));
typedef uint32_t u2a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t u2u2 __attribute__((ext_vector_type(2), aligned(2)));
typedef uint32_t u4u1 __attribute__((ext_vector_type(4), aligned(1)));

enum { kAdd = 0, kMul = 1, kMin = 2, kMax = 3 };

// Maps a c10d reduce-op code to the kernel op set; -1 when unsupported.
inline int op_index(int op) {
    switch (op) {
        case MCCL_HIP_SUM:
        case MCCL_HIP_AVG: return kAdd;
        case MCCL_HIP_PRODUCT: return kMul;
        case MCCL_HIP_MIN: return kMin;
        case MCCL_HIP_MAX: return kMax;
        default: return -1;
    }
}

__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }

// dst = local value, src = incoming value: one IEEE fp32 operation.
template <int OP>
__device__ __forceinline__ float op_f32(float dst, float src) {
    if constexpr (OP == kAdd) return dst + src;
    else if constexpr (OP == kMul) return dst * src;
    else if constexpr (OP == kMin) return (src < dst) ? src : dst;
    else return (src > dst) ? src : dst;
}

// ---- fp16 / bf16 <-> fp32 ---------------------------------------------------
__device__ __forceinline__ float widen_f16(uint32_t h) {
    _Float16 v;
    uint16_t b = (uint16_t)h;
    __builtin_memcpy(&v, &b, 2);
    return (float)v;  // v_cvt_f32_f16: exact, subnormals kept, sNaN quieted
}
__device__ __forceinline__ uint32_t narrow_f16(float f) {
    // The fp32 result must exist as a rounded fp32 value before it is narrowed:
    // the empty asm keeps the compiler from folding the producing multiply into
    // a mixed-precision multiply-and-convert (one rounding instead of two).
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round to nearest even, gradual underflow
    uint16_t b;
    __builtin_memcpy(&b, &v, 2);
    uint32_t r = b;
    if (f != f) r = ((f2u(f) >> 16) & 0x8000u) | 0x7E00u;  // canonical NaN, sign kept
    return r;
}
__device__ __forceinline__ float widen_bf16(uint32_t b) { return u2f(b << 16); }
__device__ __forceinline__ uint32_t narrow_bf16(float f) {
    uint32_t u = f2u(f);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    if (f != f) r = 0x7FC0u;
    return r;
}

template <int DT>
__device__ __forceinline__ float widen16(uint32_t v) {
    if constexpr (DT == MCCL_HIP_F16) return widen_f16(v);
    else return widen_bf16(v);
}
template <int DT>
__device__ __forceinline__ uint32_t narrow16(float f) {
    if constexpr (DT == MCCL_HIP_F16) return narrow_f16(f);
    else return narrow_bf16(f);
}

template <int DT>
struct ElemInfo {
    static constexpr int size = (DT == MCCL_HIP_F32) ? 4 : 2;
    static constexpr int per_vec = 16 / size;
};

// ---- wave / block prefix sums ----------------------------------------------
// Inclusive scan of `v` across the 64 lanes of a wavefront, on the DPP data path
// (no LDS traffic): shifts by 1, 2, 4, 8 inside each row of 16 lanes, then lane
// 15 of rows 0 and 2 is added to rows 1 and 3, then lane 31 to rows 2 and 3.
// Lanes without a source, and rows masked out, read the `old` operand, 0.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, true);   // row_shr:1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, true);   // row_shr:2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, true);   // row_shr:4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, true);   // row_shr:8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, false);  // row_bcast:15 -> rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, false);  // row_bcast:31 -> rows 2, 3
    return v;
}

// Exclusive scan of one value per thread over a block of THREADS threads, in
// thread order.  `smem` holds THREADS / kWave words.  Returns the exclusive
// prefix; *total receives the block sum.  Ends with a barrier, so smem can be
// reused.
template <int THREADS>
__device__ __forceinline__ uint32_t block_exclusive_scan_n(uint32_t v, uint32_t* smem, uint32_t* total) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    uint32_t inc = wave_inclusive_scan(v);
    if (lane == kWave - 1) smem[wave] = inc;
    __syncthreads();
    uint32_t base = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < THREADS / kWave; w++) {
        uint32_t s = smem[w];
        if (w < wave) base += s;
        sum += s;
    }
    __syncthreads();
    *total = sum;
    return base + inc - v;
}

__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* smem, uint32_t* total) {
    return block_exclusive_scan_n<kBlock>(v, smem, total);
}

}  // namespace mcclhip
