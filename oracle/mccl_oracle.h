/*
 * mccl_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C CPU restatement of the reference's per-rank data-parallel compute
 * path (chunk fold, AVG scale, top-k compress with error feedback, decompress
 * and rank-ordered accumulate).  It exists to check the HIP kernels and to be
 * timed as the CPU baseline; nothing in the shipped library links or calls it.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference checkout).
 */
#ifndef MCCL_ORACLE_H
#define MCCL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Reduce-op codes: numeric values of c10d::ReduceOp::RedOpType. */
enum {
    ORC_OP_SUM = 0,
    ORC_OP_AVG = 1,
    ORC_OP_PRODUCT = 2,
    ORC_OP_MIN = 3,
    ORC_OP_MAX = 4
};

/* Element types: numeric values of at::ScalarType. */
enum {
    ORC_U8 = 0,
    ORC_I32 = 3,
    ORC_I64 = 4,
    ORC_F16 = 5,
    ORC_F32 = 6,
    ORC_BOOL = 11,
    ORC_BF16 = 15
};

/* Ring schedules whose fold order can be restated. */
enum {
    ORC_RING_BASIC = 0,   /* ws chunks of ceil(n/ws)        */
    ORC_RING_CHUNKED = 1  /* 2*ws chunks of ceil(n/(2*ws))  */
};

enum {
    ORC_OK = 0,
    ORC_ERR_OP = -1,        /* unsupported reduce op                    */
    ORC_ERR_DTYPE = -2,     /* unsupported element type                 */
    ORC_ERR_CAPACITY = -3,  /* "TopK compress: buffer too small"        */
    ORC_ERR_SIZE = -4,      /* "TopK decompress: size mismatch"         */
    ORC_ERR_INDEX = -5,     /* "TopK decompress: index out of bounds"   */
    ORC_ERR_ARG = -6
};

/* ---- 16-bit float conversions (c10::Half / c10::BFloat16 semantics) ---- */
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
float orc_bf16_to_f32(uint16_t b);
uint16_t orc_f32_to_bf16(float f);
/* Array forms: kind 0 f16->f32, 1 f32->f16, 2 bf16->f32, 3 f32->bf16,
 * 4 f32->f16 with the FP16 compressor's NaN rule. */
int orc_convert(void* dst, const void* src, int64_t n, int kind);

/* ---- FP16 compressor (csrc/compression/FP16Compression.cpp:16-165) ----
 * Follows the reference's target-platform (NEON) branch: IEEE RNE with
 * gradual underflow; NaN -> sign | 0x7C00 | mant >> 13 | 0x200 (:47-51).
 * The reference's portable branch differs only in flushing half subnormals
 * to zero (:58-59, :102-103) and in leaving signalling NaNs unquieted when
 * widening (:104-105).  dtype is ORC_F32 (cast) or ORC_F16 (passthrough).
 * compress returns the byte count or ORC_ERR_CAPACITY / ORC_ERR_DTYPE;
 * decompress returns ORC_OK or ORC_ERR_SIZE / ORC_ERR_DTYPE. */
uint16_t orc_f32_to_f16_transport(float f);
int64_t orc_fp16_compress(const void* src, int64_t nbytes, void* dst, int64_t capacity, int dtype);
int orc_fp16_decompress(const void* src, int64_t compressed_size, void* dst, int64_t nbytes, int dtype);

/* ---- binary folds, in place on dst; `threads` <= 0 picks the reference's
 *      job split (>= 1 Mi floats per job, at most 8 jobs). ---- */
int orc_fold2_f32(float* dst, const float* src, int64_t n, int op, int threads);
int orc_scale_f32(float* buf, int64_t n, float scale, int threads);
int orc_fold2_scale_f32(float* dst, const float* src, int64_t n, float scale,
                        int threads);

/* dtype = ORC_F16 / ORC_BF16: widen -> fp32 op -> one RNE narrow. */
int orc_fold2_h(uint16_t* dst, const uint16_t* src, int64_t n, int dtype, int op);
int orc_scale_h(uint16_t* buf, int64_t n, int dtype, float scale);
int orc_fold2_scale_h(uint16_t* dst, const uint16_t* src, int64_t n, int dtype,
                      float scale);

/* Integral folds / scale. scale_round_i32 != 0 selects the GPU-kernel rule
 * for int32 (round half away from zero) instead of truncation. */
int orc_fold2_int(void* dst, const void* src, int64_t n, int dtype, int op);
int orc_scale_int(void* buf, int64_t n, int dtype, float scale,
                  int scale_round_i32);

/* ---- ring fold order ---- */
/* Number of chunks and elements per chunk for a schedule. */
int orc_ring_chunks(int ws, int schedule);
int64_t orc_ring_chunk_elems(int64_t n, int ws, int schedule);
/* Rank whose local data starts the left fold of chunk c. */
int orc_ring_first_rank(int c, int ws, int schedule);

/* Closed form: out[chunk c] = ((x_s + x_{s+1}) + ...), s = first rank of c,
 * then (apply_scale) one multiply by `scale`.  dtype F32/F16/BF16.
 * stepwise != 0: 16-bit partials are rounded to the element type after every
 * step (what travels on the wire); 0: fp32 accumulate, one final rounding. */
int orc_ring_fold(void* out, const void* const* in, int ws, int64_t n,
                  int schedule, int dtype, int op, int apply_scale, float scale,
                  int stepwise);

/* Brute force: runs the reduce-scatter half of the schedule on ws private
 * rank buffers step by step (send_idx / recv_idx formulas of the reference),
 * then copies each reduced chunk from its owner.  fp32 only. */
int orc_ring_simulate_f32(float* out, const float* const* in, int ws, int64_t n,
                          int schedule, int op);

/* ---- top-k compression with error feedback ---- */
uint32_t orc_topk_k(uint64_t count, double ratio);
uint64_t orc_topk_max_compressed_size(uint64_t nbytes, double ratio);
/* residual is read (error feedback) and rewritten.  Returns bytes written
 * (4 + 8k) or a negative error. Ties at the threshold magnitude go to the
 * lower index. */
int64_t orc_topk_compress(const float* grad, float* residual, uint64_t count,
                          double ratio, void* dst, uint64_t dst_capacity);
int orc_topk_decompress(const void* src, uint64_t compressed_size, float* dst,
                        uint64_t count);
/* Dense reference form of decompress+accumulate over W ranks in rank order:
 * acc = +0; for r: tmp = decompress(wire_r); acc += tmp; then acc *= scale. */
int orc_sparse_accumulate(float* acc, uint64_t count, const void* const* wires,
                          const uint64_t* wire_bytes, int ws, int apply_scale,
                          float scale);

#ifdef __cplusplus
}
#endif
#endif
