/*
 * mccl_oracle.c -- TEST INFRASTRUCTURE ONLY (checker and timed CPU baseline).
 *
 * CPU restatement of the reference's per-rank data-parallel compute path.
 * Build with -O3 -ffp-contract=off and without any fast-math option: every
 * fold below must stay one IEEE-754 operation per element.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   16-bit conversions   torch CPU casts, exhaustively over all 65,536 encodings
 *                        and over every rounding boundary of the narrow casts
 *   folds / scale        torch CPU add/mul/min/max (independent library), the
 *                        reference tests' known answers
 *   ring fold order      orc_ring_simulate_f32 (brute-force run of the
 *                        reference's step plan) against the closed form, and
 *                        the reference tests' exact 3-rank answers
 *   top-k                brute-force lexsort on small inputs; the reference's
 *                        own TopKCompression.cpp (compiled into oracle/_ref)
 *                        on tie-free inputs; conservation invariants
 *   decompress           known answers + error cases by construction
 * Parity unpinned (reference leaves it open, recorded here on purpose):
 *   MIN/MAX on NaN or on (+0,-0) pairs -- this file uses compare-select
 *   `(src < dst) ? src : dst`; top-k on NaN input (reference: undefined).
 */
#include "mccl_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ */
/* 16-bit conversions.  The reference widens with static_cast<float>(T) and
 * narrows with static_cast<T>(float) for T = c10::Half / c10::BFloat16
 * (csrc/metal/AccelerateOps.mm:15-27).  c10 is a PyTorch dependency, not part
 * of the reference tree; its published behaviour is IEEE binary16 round to
 * nearest even with gradual underflow and NaN -> sign|0x7E00, and for
 * bfloat16 "bits + 0x7FFF + lsb, NaN -> 0x7FC0".                          */

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu) /* inf, or NaN (signalling NaNs come out quiet, as on hardware) */
        return u2f(sign | 0x7F800000u | (m << 13) | (m ? 0x00400000u : 0u));
    if (e == 0) {
        if (m == 0) return u2f(sign);
        /* subnormal: m * 2^-24, exact in fp32 */
        float v = (float)m * 5.9604644775390625e-08f;
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x = f2u(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7FFFFFFFu;
    if (x > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 -> inf */
    uint32_t e = x >> 23;
    if (e < 113u) { /* |f| < 2^-14: subnormal half or zero */
        if (e < 102u) return sign;
        uint32_t mant = (x & 0x7FFFFFu) | 0x800000u;
        uint32_t s = 126u - e; /* 14..24 */
        uint32_t q = mant >> s;
        uint32_t rem = mant & ((1u << s) - 1u);
        uint32_t half = 1u << (s - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t h = ((e - 112u) << 10) | ((x >> 13) & 0x3FFu);
    uint32_t rem = x & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

float orc_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

uint16_t orc_f32_to_bf16(float f) {
    if (f != f) return 0x7FC0u;
    uint32_t u = f2u(f);
    uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
    return (uint16_t)((u + bias) >> 16);
}

/* csrc/compression/FP16Compression.cpp:47-51: a NaN keeps its sign and top
 * mantissa bits and gets the quiet bit; everything else is plain RNE. */
uint16_t orc_f32_to_f16_transport(float f) {
    uint32_t x = f2u(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)(((x >> 16) & 0x8000u) | 0x7C00u | ((x & 0x7FFFFFu) >> 13) | 0x200u);
    return orc_f32_to_f16(f);
}

/* csrc/compression/FP16Compression.cpp:117-143 */
int64_t orc_fp16_compress(const void* src, int64_t nbytes, void* dst, int64_t capacity, int dtype) {
    if (dtype == ORC_F16) {
        if (capacity < nbytes) return ORC_ERR_CAPACITY;
        memcpy(dst, src, (size_t)nbytes);
        return nbytes;
    }
    if (dtype != ORC_F32) return ORC_ERR_DTYPE;
    int64_t count = nbytes / 4;
    if (capacity < count * 2) return ORC_ERR_CAPACITY;
    for (int64_t i = 0; i < count; i++)
        ((uint16_t*)dst)[i] = orc_f32_to_f16_transport(((const float*)src)[i]);
    return count * 2;
}

/* csrc/compression/FP16Compression.cpp:145-163 */
int orc_fp16_decompress(const void* src, int64_t compressed_size, void* dst, int64_t nbytes, int dtype) {
    if (dtype == ORC_F16) {
        if (compressed_size != nbytes) return ORC_ERR_SIZE;
        memcpy(dst, src, (size_t)nbytes);
        return ORC_OK;
    }
    if (dtype != ORC_F32) return ORC_ERR_DTYPE;
    int64_t count = nbytes / 4;
    if (compressed_size != count * 2) return ORC_ERR_SIZE;
    for (int64_t i = 0; i < count; i++) ((float*)dst)[i] = orc_f16_to_f32(((const uint16_t*)src)[i]);
    return ORC_OK;
}

/* Array forms: kind 0 f16->f32, 1 f32->f16, 2 bf16->f32, 3 f32->bf16,
 * 4 f32->f16 with the FP16 compressor's NaN rule. */
int orc_convert(void* dst, const void* src, int64_t n, int kind) {
    for (int64_t i = 0; i < n; i++) {
        switch (kind) {
            case 0: ((float*)dst)[i] = orc_f16_to_f32(((const uint16_t*)src)[i]); break;
            case 1: ((uint16_t*)dst)[i] = orc_f32_to_f16(((const float*)src)[i]); break;
            case 2: ((float*)dst)[i] = orc_bf16_to_f32(((const uint16_t*)src)[i]); break;
            case 3: ((uint16_t*)dst)[i] = orc_f32_to_bf16(((const float*)src)[i]); break;
            case 4: ((uint16_t*)dst)[i] = orc_f32_to_f16_transport(((const float*)src)[i]); break;
            default: return ORC_ERR_ARG;
        }
    }
    return ORC_OK;
}

static inline float widen(uint16_t v, int dtype) {
    return dtype == ORC_F16 ? orc_f16_to_f32(v) : orc_bf16_to_f32(v);
}
static inline uint16_t narrow(float v, int dtype) {
    return dtype == ORC_F16 ? orc_f32_to_f16(v) : orc_f32_to_bf16(v);
}

/* ------------------------------------------------------------------ */
/* One fp32 step of the op switch, dst = local value, src = incoming.
 * csrc/metal/AccelerateOps.mm:184-204 (SUM and AVG both add; AVG's scale is
 * applied by the caller afterwards), :144-154 min/max/product.            */
static inline float apply_op(float dst, float src, int op) {
    switch (op) {
        case ORC_OP_SUM:
        case ORC_OP_AVG: return dst + src;
        case ORC_OP_PRODUCT: return dst * src;
        case ORC_OP_MIN: return (src < dst) ? src : dst;
        default: /* ORC_OP_MAX */ return (src > dst) ? src : dst;
    }
}
static inline int op_ok(int op) { return op >= ORC_OP_SUM && op <= ORC_OP_MAX; }

/* Job split of the reference: below 1 Mi floats one job, else
 * min(count / 1Mi, 8) contiguous slices of ceil(count/jobs)
 * (csrc/metal/AccelerateOps.mm:67-95).                                    */
static int mt_jobs(int64_t count) {
    const int64_t thr = 1024 * 1024;
    if (count < thr) return 1;
    int64_t j = count / thr;
    return (int)(j < 8 ? j : 8);
}

typedef struct {
    float* dst;
    const float* src;
    int64_t n;
    int kind; /* 0 fold, 1 scale, 2 fold+scale */
    int op;
    float scale;
} job_t;

static void run_slice(const job_t* j) {
    float* d = j->dst;
    const float* s = j->src;
    int64_t n = j->n;
    if (j->kind == 0) {
        switch (j->op) {
            case ORC_OP_SUM:
            case ORC_OP_AVG: for (int64_t i = 0; i < n; i++) d[i] = d[i] + s[i]; break;
            case ORC_OP_PRODUCT: for (int64_t i = 0; i < n; i++) d[i] = d[i] * s[i]; break;
            case ORC_OP_MIN: for (int64_t i = 0; i < n; i++) d[i] = (s[i] < d[i]) ? s[i] : d[i]; break;
            default: for (int64_t i = 0; i < n; i++) d[i] = (s[i] > d[i]) ? s[i] : d[i]; break;
        }
    } else if (j->kind == 1) {
        /* vDSP_vsmul: one multiply (csrc/metal/AccelerateOps.mm:103-120) */
        float sc = j->scale;
        for (int64_t i = 0; i < n; i++) d[i] = d[i] * sc;
    } else {
        /* vadd pass then vsmul pass: the sum is rounded to fp32 before the
         * multiply (csrc/metal/AccelerateOps.mm:122-142) */
        float sc = j->scale;
        for (int64_t i = 0; i < n; i++) {
            float t = d[i] + s[i];
            d[i] = t * sc;
        }
    }
}

static void* job_main(void* p) { run_slice((const job_t*)p); return NULL; }

static void run_parallel(job_t whole, int threads) {
    int jobs = threads > 0 ? threads : mt_jobs(whole.n);
    if (jobs > 64) jobs = 64;
    if (jobs <= 1 || whole.n < jobs) { run_slice(&whole); return; }
    int64_t chunk = (whole.n + jobs - 1) / jobs;
    pthread_t tid[64];
    job_t js[64];
    int started = 0;
    for (int i = 0; i < jobs; i++) {
        int64_t start = (int64_t)i * chunk;
        int64_t end = start + chunk < whole.n ? start + chunk : whole.n;
        if (start >= end) break;
        js[i] = whole;
        js[i].dst = whole.dst + start;
        js[i].src = whole.src ? whole.src + start : NULL;
        js[i].n = end - start;
        if (pthread_create(&tid[i], NULL, job_main, &js[i]) != 0) {
            run_slice(&js[i]);
            tid[i] = 0;
        }
        started = i + 1;
    }
    for (int i = 0; i < started; i++)
        if (tid[i]) pthread_join(tid[i], NULL);
}

int orc_fold2_f32(float* dst, const float* src, int64_t n, int op, int threads) {
    if (!op_ok(op)) return ORC_ERR_OP;
    job_t j = {dst, src, n, 0, op, 0.0f};
    run_parallel(j, threads);
    return ORC_OK;
}

int orc_scale_f32(float* buf, int64_t n, float scale, int threads) {
    job_t j = {buf, NULL, n, 1, 0, scale};
    run_parallel(j, threads);
    return ORC_OK;
}

int orc_fold2_scale_f32(float* dst, const float* src, int64_t n, float scale,
                        int threads) {
    job_t j = {dst, src, n, 2, 0, scale};
    run_parallel(j, threads);
    return ORC_OK;
}

/* fp16 / bf16: widen both operands, fp32 op, narrow once
 * (csrc/metal/AccelerateOps.mm:29-65, exported at :156-182).               */
int orc_fold2_h(uint16_t* dst, const uint16_t* src, int64_t n, int dtype, int op) {
    if (dtype != ORC_F16 && dtype != ORC_BF16) return ORC_ERR_DTYPE;
    if (!op_ok(op)) return ORC_ERR_OP;
    for (int64_t i = 0; i < n; i++)
        dst[i] = narrow(apply_op(widen(dst[i], dtype), widen(src[i], dtype), op), dtype);
    return ORC_OK;
}

int orc_scale_h(uint16_t* buf, int64_t n, int dtype, float scale) {
    if (dtype != ORC_F16 && dtype != ORC_BF16) return ORC_ERR_DTYPE;
    for (int64_t i = 0; i < n; i++) buf[i] = narrow(widen(buf[i], dtype) * scale, dtype);
    return ORC_OK;
}

int orc_fold2_scale_h(uint16_t* dst, const uint16_t* src, int64_t n, int dtype,
                      float scale) {
    if (dtype != ORC_F16 && dtype != ORC_BF16) return ORC_ERR_DTYPE;
    for (int64_t i = 0; i < n; i++) {
        volatile float t = widen(dst[i], dtype) + widen(src[i], dtype);
        dst[i] = narrow(t * scale, dtype);
    }
    return ORC_OK;
}

/* Integral folds (csrc/metal/AccelerateOps.mm:206-276).  bool tensors are
 * folded as raw uint8 with wrap-around, exactly like integral_reduce<uint8_t>.
 * Signed overflow wraps (two's complement) as on the GPU.                  */
#define INT_FOLD(T, UT)                                                            \
    do {                                                                           \
        T* d = (T*)dst;                                                            \
        const T* s = (const T*)src;                                                \
        switch (op) {                                                              \
            case ORC_OP_SUM:                                                       \
            case ORC_OP_AVG: for (int64_t i = 0; i < n; i++) d[i] = (T)((UT)d[i] + (UT)s[i]); break; \
            case ORC_OP_PRODUCT: for (int64_t i = 0; i < n; i++) d[i] = (T)((UT)d[i] * (UT)s[i]); break; \
            case ORC_OP_MIN: for (int64_t i = 0; i < n; i++) d[i] = s[i] < d[i] ? s[i] : d[i]; break; \
            default: for (int64_t i = 0; i < n; i++) d[i] = s[i] > d[i] ? s[i] : d[i]; break; \
        }                                                                          \
    } while (0)

int orc_fold2_int(void* dst, const void* src, int64_t n, int dtype, int op) {
    if (!op_ok(op)) return ORC_ERR_OP;
    switch (dtype) {
        case ORC_BOOL:
        case ORC_U8: INT_FOLD(uint8_t, uint8_t); break;
        case ORC_I32: INT_FOLD(int32_t, uint32_t); break;
        case ORC_I64: INT_FOLD(int64_t, uint64_t); break;
        default: return ORC_ERR_DTYPE;
    }
    return ORC_OK;
}

/* buf[i] = T(float(buf[i]) * scale): truncation toward zero on the CPU path
 * (csrc/metal/AccelerateOps.mm:229-236); the GPU kernels truncate int64/uint8
 * but round int32 half away from zero (csrc/metal/shaders.metal:622-665).   */
int orc_scale_int(void* buf, int64_t n, int dtype, float scale, int scale_round_i32) {
    switch (dtype) {
        case ORC_BOOL:
        case ORC_U8: {
            uint8_t* b = (uint8_t*)buf;
            for (int64_t i = 0; i < n; i++) b[i] = (uint8_t)((float)b[i] * scale);
            break;
        }
        case ORC_I32: {
            int32_t* b = (int32_t*)buf;
            for (int64_t i = 0; i < n; i++) {
                float v = (float)b[i] * scale;
                b[i] = scale_round_i32 ? (int32_t)roundf(v) : (int32_t)v;
            }
            break;
        }
        case ORC_I64: {
            int64_t* b = (int64_t*)buf;
            for (int64_t i = 0; i < n; i++) b[i] = (int64_t)((float)b[i] * scale);
            break;
        }
        default: return ORC_ERR_DTYPE;
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* Ring fold order.
 * Basic ring: ws chunks of ceil(n/ws); step plan
 *   send_idx = (rank - step + ws) % ws, recv_idx = (rank - step - 1 + ws) % ws
 * (csrc/backend/ProcessGroupMCCL.cpp:1989-2006, :2016-2024).
 * Chunked ring: 2*ws chunks of ceil(n/(2*ws)); 2*(ws-1) reduce steps with
 *   send_idx = (2*rank - step + 2*ws) % (2*ws),
 *   recv_idx = (2*rank - step - 2 + 2*ws) % (2*ws)
 * (csrc/backend/ProcessGroupMCCL.cpp:1725-1742, :1754-1762).
 * The receive side reduces `local chunk (dst) op= incoming (src)`
 * (csrc/backend/ProcessGroupMCCL.cpp:492-512).                            */

int orc_ring_chunks(int ws, int schedule) {
    return schedule == ORC_RING_CHUNKED ? 2 * ws : ws;
}

int64_t orc_ring_chunk_elems(int64_t n, int ws, int schedule) {
    int64_t c = orc_ring_chunks(ws, schedule);
    return (n + c - 1) / c;
}

int orc_ring_first_rank(int c, int ws, int schedule) {
    if (schedule == ORC_RING_CHUNKED) return ((c + 1) / 2) % ws;
    return c % ws;
}

int orc_ring_fold(void* out, const void* const* in, int ws, int64_t n,
                  int schedule, int dtype, int op, int apply_scale, float scale,
                  int stepwise) {
    if (!op_ok(op)) return ORC_ERR_OP;
    if (dtype != ORC_F32 && dtype != ORC_F16 && dtype != ORC_BF16) return ORC_ERR_DTYPE;
    if (ws < 1) return ORC_ERR_ARG;
    int nchunks = orc_ring_chunks(ws, schedule);
    int64_t ce = orc_ring_chunk_elems(n, ws, schedule);
    for (int c = 0; c < nchunks; c++) {
        int64_t start = (int64_t)c * ce;
        int64_t len = ce < n - start ? ce : n - start;
        if (len <= 0) continue;
        int s = orc_ring_first_rank(c, ws, schedule);
        for (int64_t i = start; i < start + len; i++) {
            if (dtype == ORC_F32) {
                float acc = ((const float*)in[s])[i];
                for (int j = 1; j < ws; j++) {
                    float local = ((const float*)in[(s + j) % ws])[i];
                    volatile float t = apply_op(local, acc, op);
                    acc = t;
                }
                if (apply_scale) acc = acc * scale;
                ((float*)out)[i] = acc;
            } else {
                float acc = widen(((const uint16_t*)in[s])[i], dtype);
                for (int j = 1; j < ws; j++) {
                    float local = widen(((const uint16_t*)in[(s + j) % ws])[i], dtype);
                    volatile float t = apply_op(local, acc, op);
                    acc = t;
                    if (stepwise) acc = widen(narrow(acc, dtype), dtype);
                }
                if (apply_scale) acc = acc * scale;
                ((uint16_t*)out)[i] = narrow(acc, dtype);
            }
        }
    }
    return ORC_OK;
}

int orc_ring_simulate_f32(float* out, const float* const* in, int ws, int64_t n,
                          int schedule, int op) {
    if (!op_ok(op)) return ORC_ERR_OP;
    if (ws < 1) return ORC_ERR_ARG;
    int nchunks = orc_ring_chunks(ws, schedule);
    int64_t ce = orc_ring_chunk_elems(n, ws, schedule);
    int nsteps = schedule == ORC_RING_CHUNKED ? 2 * (ws - 1) : ws - 1;
    float** local = (float**)malloc(sizeof(float*) * (size_t)ws);
    float** wire = (float**)malloc(sizeof(float*) * (size_t)ws);
    int* holder = (int*)malloc(sizeof(int) * (size_t)nchunks);
    for (int r = 0; r < ws; r++) {
        local[r] = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
        wire[r] = (float*)malloc(sizeof(float) * (size_t)(ce > 0 ? ce : 1));
        memcpy(local[r], in[r], sizeof(float) * (size_t)n);
    }
    for (int c = 0; c < nchunks; c++) holder[c] = orc_ring_first_rank(c, ws, schedule);
    for (int step = 0; step < nsteps; step++) {
        /* TX: every rank puts its send chunk on the wire to its right peer */
        for (int r = 0; r < ws; r++) {
            int send_idx = schedule == ORC_RING_CHUNKED
                               ? (2 * r - step + 2 * ws * 4) % (2 * ws)
                               : (r - step + ws * 4) % ws;
            int64_t start = (int64_t)send_idx * ce;
            int64_t len = ce < n - start ? ce : n - start;
            if (len > 0) memcpy(wire[r], local[r] + start, sizeof(float) * (size_t)len);
        }
        /* RX: rank r reduces what its left peer sent into its own chunk */
        for (int r = 0; r < ws; r++) {
            int left = (r - 1 + ws) % ws;
            int recv_idx = schedule == ORC_RING_CHUNKED
                               ? (2 * r - step - 2 + 2 * ws * 4) % (2 * ws)
                               : (r - step - 1 + ws * 4) % ws;
            int64_t start = (int64_t)recv_idx * ce;
            int64_t len = ce < n - start ? ce : n - start;
            for (int64_t i = 0; i < len; i++) {
                volatile float t = apply_op(local[r][start + i], wire[left][i], op);
                local[r][start + i] = t;
            }
            holder[recv_idx] = r;
        }
    }
    for (int c = 0; c < nchunks; c++) {
        int64_t start = (int64_t)c * ce;
        int64_t len = ce < n - start ? ce : n - start;
        if (len > 0) memcpy(out + start, local[holder[c]] + start, sizeof(float) * (size_t)len);
    }
    for (int r = 0; r < ws; r++) { free(local[r]); free(wire[r]); }
    free(local); free(wire); free(holder);
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* Top-k with error feedback (csrc/compression/TopKCompression.cpp:38-120).
 *   k = max(1, uint32(count * ratio)) with the product in double (:45-47)
 *   adjusted = grad + residual, one fp32 add (:73-75)
 *   pick the k largest |adjusted| (:80-87); ties at the threshold go to the
 *   lower index (the reference leaves the choice to std::nth_element)
 *   picks sorted by index (:90); wire = [u32 k][k x {u32 index, f32 value}]
 *   (:93-113); residual = adjusted, then 0.0f at every pick (:103,:112).   */

uint32_t orc_topk_k(uint64_t count, double ratio) {
    uint32_t k = (uint32_t)((double)count * ratio);
    return k < 1u ? 1u : k;
}

/* csrc/compression/TopKCompression.cpp:154-158 */
uint64_t orc_topk_max_compressed_size(uint64_t nbytes, double ratio) {
    uint64_t count = nbytes / 4;
    uint32_t k = (uint32_t)((double)count * ratio) + 1u;
    return 4u + (uint64_t)k * 8u;
}

int64_t orc_topk_compress(const float* grad, float* residual, uint64_t count,
                          double ratio, void* dst, uint64_t dst_capacity) {
    if (count == 0 || !(ratio > 0.0 && ratio <= 1.0)) return ORC_ERR_ARG;
    uint32_t k = orc_topk_k(count, ratio);
    if ((uint64_t)k > count) return ORC_ERR_ARG;
    uint64_t out_size = 4u + (uint64_t)k * 8u;
    if (dst_capacity < out_size) return ORC_ERR_CAPACITY;

    /* residual <- adjusted */
    for (uint64_t i = 0; i < count; i++) residual[i] = grad[i] + residual[i];

    /* k-th largest magnitude by 3-round radix select on |x| bit patterns
     * (for non-NaN floats fabs order == unsigned order of bits & 0x7FFFFFFF) */
    uint32_t prefix = 0, prefix_mask = 0;
    uint64_t remaining = k; /* how many still to take among the current prefix */
    static const int shifts[3] = {20, 10, 0};
    static const uint32_t widths[3] = {11, 10, 10};
    uint64_t* hist = (uint64_t*)malloc(sizeof(uint64_t) * 2048);
    for (int round = 0; round < 3; round++) {
        uint32_t bins = 1u << widths[round];
        memset(hist, 0, sizeof(uint64_t) * bins);
        for (uint64_t i = 0; i < count; i++) {
            uint32_t key = f2u(residual[i]) & 0x7FFFFFFFu;
            if ((key & prefix_mask) == prefix) hist[(key >> shifts[round]) & (bins - 1u)]++;
        }
        uint32_t b = bins;
        while (b-- > 0) {
            if (hist[b] >= remaining) break;
            remaining -= hist[b];
        }
        prefix |= b << shifts[round];
        prefix_mask |= (bins - 1u) << shifts[round];
    }
    free(hist);
    uint32_t T = prefix;        /* exact key of the k-th largest */
    uint64_t need = remaining;  /* how many elements with key == T are taken */

    uint8_t* out = (uint8_t*)dst;
    memcpy(out, &k, 4);
    out += 4;
    for (uint64_t i = 0; i < count; i++) {
        uint32_t key = f2u(residual[i]) & 0x7FFFFFFFu;
        int take = 0;
        if (key > T) take = 1;
        else if (key == T && need > 0) { take = 1; need--; }
        if (take) {
            uint32_t idx = (uint32_t)i;
            float v = residual[i];
            memcpy(out, &idx, 4);
            memcpy(out + 4, &v, 4);
            out += 8;
            residual[i] = 0.0f;
        }
    }
    return (int64_t)out_size;
}

/* csrc/compression/TopKCompression.cpp:122-152.  On an error the reference
 * throws after having zeroed dst and written the pairs before the bad one;
 * this restatement does the same and returns the code.                     */
int orc_topk_decompress(const void* src, uint64_t compressed_size, float* dst,
                        uint64_t count) {
    memset(dst, 0, count * 4);
    if (compressed_size < 4) return ORC_ERR_SIZE;
    const uint8_t* in = (const uint8_t*)src;
    uint32_t k;
    memcpy(&k, in, 4);
    in += 4;
    if (compressed_size != 4u + (uint64_t)k * 8u) return ORC_ERR_SIZE;
    for (uint32_t i = 0; i < k; i++) {
        uint32_t idx;
        float v;
        memcpy(&idx, in, 4);
        memcpy(&v, in + 4, 4);
        in += 8;
        if ((uint64_t)idx >= count) return ORC_ERR_INDEX;
        dst[idx] = v;
    }
    return ORC_OK;
}

/* Hub accumulate of compressed contributions: every peer's payload is
 * decompressed into a dense buffer and folded with a dense add in ascending
 * rank order, then one AVG multiply
 * (csrc/backend/ProcessGroupMCCL.cpp:1692-1709, :2272-2296).  Here the
 * accumulator starts at +0.0 and all ws payloads are folded into it.        */
int orc_sparse_accumulate(float* acc, uint64_t count, const void* const* wires,
                          const uint64_t* wire_bytes, int ws, int apply_scale,
                          float scale) {
    float* tmp = (float*)malloc(sizeof(float) * (size_t)(count ? count : 1));
    for (uint64_t i = 0; i < count; i++) acc[i] = 0.0f;
    int rc = ORC_OK;
    for (int r = 0; r < ws && rc == ORC_OK; r++) {
        rc = orc_topk_decompress(wires[r], wire_bytes[r], tmp, count);
        if (rc != ORC_OK) break;
        for (uint64_t i = 0; i < count; i++) acc[i] = acc[i] + tmp[i];
    }
    if (rc == ORC_OK && apply_scale)
        for (uint64_t i = 0; i < count; i++) acc[i] = acc[i] * scale;
    free(tmp);
    return rc;
}
