/*
 * mccl_hip.h -- C ABI of the MI355X (gfx950) implementation of MCCL's per-rank
 * data-parallel compute path: chunk fold, AVG scale, ring-order W-way fold,
 * top-k compression with error feedback, decompress and rank-ordered sparse
 * accumulate.
 *
 * Conventions
 *   - Every pointer is DEVICE memory unless its name starts with `host_`.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *     Calls only enqueue work; completion is observed through the stream, a
 *     fence ticket (below) or mccl_hip_sync().
 *   - Return value: MCCL_HIP_OK or a negative MCCL_HIP_ERR_* code.  Nothing
 *     throws, nothing takes ownership of caller memory.
 *   - `dtype` uses the numeric values of at::ScalarType, `op` those of
 *     c10d::ReduceOp::RedOpType, so a torch binding can pass them through.
 *
 * Each entry point names the reference interface it replaces (paths are
 * relative to the reference checkout).
 */
#ifndef MCCL_HIP_H
#define MCCL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MCCL_HIP_ABI_VERSION 1

/* ---- status codes ------------------------------------------------------ */
#define MCCL_HIP_OK 0
#define MCCL_HIP_ERR_OP (-1)        /* "Unsupported ReduceOp" (csrc/metal/MetalKernels.mm:798-800) */
#define MCCL_HIP_ERR_DTYPE (-2)     /* no kernel for this element type (MetalKernels.mm:542-544)   */
#define MCCL_HIP_ERR_CAPACITY (-3)  /* "TopK compress: buffer too small" (TopKCompression.cpp:94)  */
#define MCCL_HIP_ERR_SIZE (-4)      /* "TopK decompress: size mismatch" (TopKCompression.cpp:138)  */
#define MCCL_HIP_ERR_INDEX (-5)     /* "TopK decompress: index out of bounds" (:148)               */
#define MCCL_HIP_ERR_ARG (-6)       /* null pointer, zero/oversized count, bad ratio, bad world size */
#define MCCL_HIP_ERR_RUNTIME (-7)   /* a HIP runtime call failed; see mccl_hip_last_hip_error()     */
#define MCCL_HIP_ERR_WORKSPACE (-8) /* workspace smaller than mccl_hip_topk_workspace_bytes()       */
#define MCCL_HIP_ERR_TIMEOUT (-9)   /* fence wait exceeded its limit (csrc/metal/EventSync.mm:37-71) */
#define MCCL_HIP_ERR_POINTER (-10)  /* the bytes are not memory a kernel on the current GPU can reach */

/* ---- element types (at::ScalarType values) ------------------------------ */
#define MCCL_HIP_U8 0
#define MCCL_HIP_I32 3
#define MCCL_HIP_I64 4
#define MCCL_HIP_F16 5
#define MCCL_HIP_F32 6
#define MCCL_HIP_BOOL 11
#define MCCL_HIP_BF16 15

/* ---- reduce ops (c10d::ReduceOp::RedOpType values) ---------------------- */
#define MCCL_HIP_SUM 0
#define MCCL_HIP_AVG 1 /* folds like SUM; the caller scales afterwards */
#define MCCL_HIP_PRODUCT 2
#define MCCL_HIP_MIN 3
#define MCCL_HIP_MAX 4

/* ---- ring schedules ----------------------------------------------------- */
#define MCCL_HIP_RING_BASIC 0   /* ws chunks of ceil(n/ws)       (ProcessGroupMCCL.cpp:1989-2034) */
#define MCCL_HIP_RING_CHUNKED 1 /* 2*ws chunks of ceil(n/(2*ws)) (ProcessGroupMCCL.cpp:1725-1772) */

#define MCCL_HIP_MAX_WORLD 64

/* Largest element count a single call accepts (the reference caps kernels at
 * UINT32_MAX elements, csrc/metal/MetalKernels.mm:292-299; this library takes
 * 64-bit counts up to 2^40). */
#define MCCL_HIP_MAX_ELEMS (1ull << 40)

/* ---- library state ------------------------------------------------------ */

/* Replaces metal_kernels_init() (csrc/metal/MetalKernels.mm:360-366) and
 * event_sync_init() (csrc/metal/EventSync.mm:76-100).  Idempotent and
 * thread-safe.  Fails with MCCL_HIP_ERR_RUNTIME when no gfx950 device is
 * current. */
int mccl_hip_init(void);
int mccl_hip_abi_version(void);
const char* mccl_hip_strerror(int code);
/* hipError_t value of the most recent failing runtime call on this thread. */
int mccl_hip_last_hip_error(void);

/* The reference's raw-pointer folds (csrc/metal/AccelerateOps.hpp:18-59) run
 * on CPU-visible memory that the GPU shares.  Their counterparts here launch
 * kernels, so a caller holding a raw pointer first asks whether a kernel on the
 * current device can reach [ptr, ptr + nbytes): device memory of the current
 * GPU (the range must lie inside one allocation), managed memory, or pinned
 * host memory.  On success *device_ptr receives the address to hand to the
 * kernels (for pinned host memory its device-side alias).  Pageable host memory
 * and foreign pointers give MCCL_HIP_ERR_POINTER; nothing is launched. */
int mccl_hip_pointer_check(const void* ptr, uint64_t nbytes, void** device_ptr);

/* ---- binary folds: one ring step ---------------------------------------- */

/* dst[i] = dst[i] (op) src[i], in place on dst, dst = local chunk, src =
 * incoming chunk.  Replaces metal_reduce_op / metal_accumulate_chunk /
 * metal_elementwise_{min,max,product} (csrc/metal/MetalKernels.hpp:17-31,
 * MetalKernels.mm:521-565,:712-802) and cpu_reduce_op[_half|_bf16|_integral]
 * (csrc/metal/AccelerateOps.hpp:21-59).  F16/BF16: widen, one fp32 operation,
 * one round-to-nearest-even narrow.  MIN/MAX are compare-selects
 * `(src < dst) ? src : dst`.  dst and src need only element alignment. */
int mccl_hip_fold2(void* dst, const void* src, uint64_t n, int dtype, int op, void* stream);

/* host_dsts[i] = host_dsts[i] (op) host_srcs[i] over host_counts[i] elements, for
 * i < nfolds: the binary fold above on a list of chunk views, one launch per 128
 * folds, every fold's result bit-identical to mccl_hip_fold2 on the same pair.
 * For a caller that holds several folds which do not depend on one another -
 * the folds of one ring step over all gradient buckets, which the reference
 * issues one by one (csrc/backend/ProcessGroupMCCL.cpp:492-512, reduce_op ->
 * metal_accumulate_chunk / cpu_reduce_op per chunk).  The three arrays are host
 * arrays of device pointers and lengths, read before the call returns.  The
 * folds run in no particular order: a destination that overlaps any other
 * fold's destination or source gives MCCL_HIP_ERR_ARG and nothing is launched;
 * folds of length 0 are skipped. */
int mccl_hip_fold2_batch(void* const* host_dsts, const void* const* host_srcs,
                         const uint64_t* host_counts, uint32_t nfolds, int dtype, int op,
                         void* stream);

/* buf[i] = buf[i] * scale (one fp32 multiply; F16/BF16 multiply in fp32 and
 * round once).  Integral types: T(float(x) * scale), truncating for
 * I64/U8/BOOL and rounding half away from zero for I32.  Replaces
 * metal_scale_inplace (MetalKernels.mm:568-613, csrc/metal/shaders.metal:
 * 233-332,:622-665) and cpu_scale_inplace* (AccelerateOps.mm:103-120). */
int mccl_hip_scale(void* buf, uint64_t n, int dtype, float scale, void* stream);

/* dst[i] = (dst[i] + src[i]) * scale with the sum rounded to fp32 before the
 * multiply.  Integral types run the add and then the scale rule above.
 * Replaces metal_accumulate_and_scale (MetalKernels.mm:616-675) and
 * cpu_accumulate_and_scale* (AccelerateOps.mm:122-142). */
int mccl_hip_fold2_scale(void* dst, const void* src, uint64_t n, int dtype, float scale,
                         void* stream);

/* ---- W-way fold in ring-step order -------------------------------------- */

/* The reduce half of a ring allreduce over `ws` simulated ranks whose buffers
 * all live in this GPU's memory.  host_in[r] is rank r's buffer of n_total
 * elements; out receives the reduced result (out may alias one host_in[r]).
 * The n_total elements are cut into buckets of bucket_elems (the last one may
 * be shorter; bucket_elems >= n_total means one bucket), every bucket into the
 * schedule's chunks, and chunk c is folded left to right starting at the rank
 * that owns it in the reference's step plan
 * (send_idx/recv_idx, ProcessGroupMCCL.cpp:1754-1762,:2016-2024; receive side
 * reduces local (op)= incoming, :492-512):
 *     acc = x[s]; for j = 1..ws-1: acc = x[(s+j) % ws] (op) acc
 * then, if apply_scale, one multiply by `scale` (the AVG tail,
 * ProcessGroupMCCL.cpp:1954-1956,:2177-2179).
 * F16/BF16: stepwise != 0 rounds the partial to the element type after every
 * step (what the reference sends between ranks); stepwise == 0 keeps the
 * partial in fp32 and rounds once at the end. */
int mccl_hip_ring_fold(void* out, const void* const* host_in, int ws, uint64_t n_total,
                       uint64_t bucket_elems, int schedule, int dtype, int op, int apply_scale,
                       float scale, int stepwise, void* stream);

/* ---- top-k compression with error feedback ------------------------------ */

/* k = max(1, uint32(count * ratio)), product in double
 * (csrc/compression/TopKCompression.cpp:45-47). */
uint32_t mccl_hip_topk_k(uint64_t count, double ratio);
/* TopKCompressor::max_compressed_size (TopKCompression.cpp:154-158). */
uint64_t mccl_hip_topk_max_compressed_size(uint64_t nbytes, double ratio);
/* Bytes of scratch mccl_hip_topk_compress needs for this shape. */
uint64_t mccl_hip_topk_workspace_bytes(uint64_t n_total, uint64_t bucket_elems, double ratio);

/* TopKCompressor::compress (TopKCompression.cpp:38-120) for every bucket of a
 * gradient in one call.  grad and residual hold n_total fp32 elements, cut
 * into buckets of bucket_elems (last may be shorter; bucket_elems >= n_total
 * means one bucket = one reference compress() call).  Per bucket b of count
 * n_b: residual += grad; the k_b = mccl_hip_topk_k(n_b, ratio) elements of
 * largest magnitude are written in ascending index order (indices relative to
 * the bucket) as [u32 k_b][k_b x {u32 index, f32 value}] at
 * wire + b * wire_stride, and residual is zeroed at those elements.  Ties at
 * the threshold magnitude go to the lower index.  wire_stride must be a
 * multiple of 4 and at least 4 + 8 * k_b for the largest bucket
 * (else MCCL_HIP_ERR_CAPACITY).
 * Magnitudes are ordered by the bit pattern `bits & 0x7FFFFFFF`: infinities
 * above every finite value, NaN patterns above infinity (by payload), ties to
 * the lower index; a NaN gradient is therefore picked, sent and cleared from the
 * residual like any other large value (the reference's comparator is undefined
 * on NaN, TopKCompression.cpp:80-87).
 * `status` (device int, may be null; the caller zeroes it) receives
 * MCCL_HIP_ERR_TIMEOUT if a block of the single-pass path gave up waiting for
 * another block of its launch (see "topk_barrier_ms"); the payload header of
 * the bucket concerned is then 0xFFFFFFFF, which mccl_hip_topk_decompress and
 * mccl_hip_sparse_accumulate reject with MCCL_HIP_ERR_SIZE. */
int mccl_hip_topk_compress(const float* grad, float* residual, uint64_t n_total,
                           uint64_t bucket_elems, double ratio, void* wire,
                           uint64_t wire_stride, void* workspace, uint64_t workspace_bytes,
                           int* status, void* stream);

/* TopKCompressor::compress for a LIST of buckets that are separate buffers of
 * their own lengths (the tensor list of a coalesced allreduce,
 * csrc/backend/ProcessGroupMCCL.cpp:2257-2313, compresses bucket by bucket), in
 * the same two launches as mccl_hip_topk_compress: per-bucket calls are bound
 * by launch latency, a list is not.  host_grads[b] / host_residuals[b] hold
 * host_counts[b] fp32 elements; bucket b's payload [u32 k_b][k_b x {u32 index,
 * f32 value}] goes to host_wires[b], which holds host_wire_capacities[b] bytes
 * (at least 4 + 8 * k_b, else MCCL_HIP_ERR_CAPACITY; 4-byte aligned).  At most
 * MCCL_HIP_TOPK_LIST_MAX buckets per call.  The host arrays are read before the
 * call returns.  Results are identical to one mccl_hip_topk_compress call per
 * bucket. */
#define MCCL_HIP_TOPK_LIST_MAX 64
uint64_t mccl_hip_topk_list_workspace_bytes(const uint64_t* host_counts, uint32_t nbuckets, double ratio);
int mccl_hip_topk_compress_list(const float* const* host_grads, float* const* host_residuals,
                                const uint64_t* host_counts, void* const* host_wires,
                                const uint64_t* host_wire_capacities, uint32_t nbuckets, double ratio,
                                void* workspace, uint64_t workspace_bytes, int* status, void* stream);

/* Diagnostics, no counterpart in the reference: after a compress call on
 * `stream` has been enqueued with this workspace and shape, waits for the
 * stream and reports how many buckets were finished by the single-pass path
 * (the others went through the exact fallback; results are identical). */
int mccl_hip_topk_path_report(const void* workspace, uint64_t n_total, uint64_t bucket_elems, double ratio,
                              uint32_t* host_single_pass_buckets, uint32_t* host_buckets, void* stream);

/* TopKCompressor::decompress (TopKCompression.cpp:122-152): dense[0..count) is
 * zeroed, then dense[index] = value for every pair.  wire_bytes is the size
 * that arrived with the payload; it must equal 4 + 8 * k for the k stored in
 * the payload.  Violations are reported through *status (a device int the
 * caller zeroes beforehand and reads after the stream has drained): it
 * receives MCCL_HIP_ERR_SIZE or MCCL_HIP_ERR_INDEX; offending pairs are
 * skipped.  status may be NULL. */
int mccl_hip_topk_decompress(const void* wire, uint64_t wire_bytes, float* dense, uint64_t count,
                             int* status, void* stream);

/* Decompress + accumulate of `ws` ranks' payloads into one dense buffer, the
 * sparse equivalent of decompressing every peer's payload and folding the
 * dense buffers in ascending rank order, then the AVG multiply
 * (ProcessGroupMCCL.cpp:1692-1709,:2272-2296):
 *     acc = +0.0; for r = 0..ws-1: acc[idx] += val for r's pairs; acc *= scale
 * host_wires[r] is rank r's payload buffer laid out like the output of
 * mccl_hip_topk_compress (bucket b at + b * wire_stride, indices relative to
 * the bucket).  Every element of acc is written exactly once.  Each payload's
 * k is read on the device; 4 + 8k > wire_stride sets *status to
 * MCCL_HIP_ERR_SIZE (the payload counts as empty), an index outside its bucket
 * sets MCCL_HIP_ERR_INDEX (the pair is skipped).  Pairs within one payload
 * must have strictly ascending indices (what compress emits): a payload that
 * does not sets MCCL_HIP_ERR_INDEX and leaves unspecified values in its
 * bucket of acc; nothing outside acc is ever written. */
int mccl_hip_sparse_accumulate(float* acc, uint64_t n_total, uint64_t bucket_elems,
                               const void* const* host_wires, int ws, uint64_t wire_stride,
                               int apply_scale, float scale, int* status, void* workspace,
                               uint64_t workspace_bytes, void* stream);
/* Scratch for mccl_hip_sparse_accumulate: per rank and bucket, a table of
 * positions in the payload (where the pairs of each run of output tiles
 * begin; one entry per 2048 output elements at most).  Passing
 * workspace = NULL is allowed: the ranges are then found by binary search in
 * every block, which costs about 3x the time on MI355X. */
uint64_t mccl_hip_sparse_accumulate_workspace_bytes(uint64_t n_total, uint64_t bucket_elems, int ws);

/* mccl_hip_sparse_accumulate for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments, meaning and
 * results as mccl_hip_sparse_accumulate with a workspace, but the position
 * table lives in a MCCL_HIP_SPARSE_STATIC_BYTES array inside the library's
 * device image (one copy per GPU, held until the process ends), and the call
 * itself allocates nothing.  Shapes whose table
 * (mccl_hip_sparse_accumulate_workspace_bytes) exceeds that size are refused
 * with MCCL_HIP_ERR_WORKSPACE.  All calls on one GPU share the array: calls
 * that may overlap on one GPU (different streams without ordering) race. */
#define MCCL_HIP_SPARSE_STATIC_BYTES (2u << 20)
int mccl_hip_sparse_accumulate_static(float* acc, uint64_t n_total, uint64_t bucket_elems,
                                      const void* const* host_wires, int ws, uint64_t wire_stride,
                                      int apply_scale, float scale, int* status, void* stream);

/* ---- fp16 transport casts ------------------------------------------------ */

/* FP16Compressor's casts (csrc/compression/FP16Compression.cpp:16-112):
 * fp32 -> fp16 round-to-nearest-even with gradual underflow and overflow to
 * infinity; NaN stays NaN (sign | 0x7C00 | mant >> 13 | 0x200); fp16 -> fp32
 * exact.  dst holds n 16-bit / 32-bit elements. */
int mccl_hip_cast_f32_to_f16(const float* src, void* dst, uint64_t n, void* stream);
int mccl_hip_cast_f16_to_f32(const void* src, float* dst, uint64_t n, void* stream);

/* ---- ordering ----------------------------------------------------------- */

/* Replaces next_fence_event_value() + signal_mccl_fence_gpu()
 * (csrc/metal/EventSync.mm:189-200): records an event on `stream` and returns
 * its ticket (monotonic, never 0) in *ticket.  A ticket covers the work
 * enqueued on ITS stream before the signal.  (The reference's shared-event
 * values are signalled from one queue, so there "value v reached" implies every
 * smaller value; here that holds per stream: wait on the last ticket of every
 * stream whose work matters.)  The library keeps the newest 1024 tickets'
 * events; a signal that pushes an older ticket out first waits, on the host,
 * until that ticket's work has completed, so a ticket that is no longer held is
 * always complete. */
int mccl_hip_fence_signal(void* stream, uint64_t* ticket);
/* Replaces wait_for_mccl_fence() (EventSync.mm:202-206): blocks the host until
 * everything enqueued on the ticket's stream before the signal has completed.
 * timeout_ms <= 0 uses the reference's 30 s limit. */
int mccl_hip_fence_wait(uint64_t ticket, int timeout_ms);
/* Non-blocking: 1 complete, 0 pending, negative on error. */
int mccl_hip_fence_query(uint64_t ticket);
/* Makes `stream` wait (on the device) for the ticket; the analogue of
 * block_mps_on_mccl() (EventSync.mm:173-187). */
int mccl_hip_fence_block_stream(uint64_t ticket, void* stream);
/* Replaces metal_sync() / metal_sync_queue_only() (MetalKernels.mm:816-824). */
int mccl_hip_sync(void* stream);

/* ---- tuning knobs (benchmarks and tests; defaults need no call) ---------- */
/* keys: "fold_blocks_per_cu", "nontemporal", "topk_path", "topk_barrier_ms", "topk_stall_test" (tests: 1 makes every wait
 * of the single-pass top-k path run into its limit, so that the give-up path can be exercised
 * without a stuck kernel),
 * "sparse_path" (0 auto, 1 tile kernels only), "sparse_run_steps" (0 auto),
 * "fp16_portable" (1: the casts follow the reference's portable branch, FP16Compression.cpp:38-73,:96-111) */
int mccl_hip_set_tuning(const char* key, int value);
int mccl_hip_get_tuning(const char* key);

#ifdef __cplusplus
}
#endif
#endif /* MCCL_HIP_H */
