// The reference's local-kernel API (csrc/metal/MetalKernels.hpp:10-48) with
// the same names, argument meaning and error behaviour, implemented as launches
// of the gfx950 kernels behind the C ABI (include/mccl_hip.h) on torch's
// current HIP stream.  Tensors are borrowed and mutated in place; calls only
// enqueue work.
#pragma once

#include <torch/torch.h>
#include <torch/csrc/distributed/c10d/Types.hpp>

#include <cstdint>

namespace mccl {

void metal_kernels_init();

void metal_accumulate_chunk(const at::Tensor& dst, const at::Tensor& src);
void metal_elementwise_min(const at::Tensor& dst, const at::Tensor& src);
void metal_elementwise_max(const at::Tensor& dst, const at::Tensor& src);
void metal_elementwise_product(const at::Tensor& dst, const at::Tensor& src);

void metal_reduce_op(const at::Tensor& dst, const at::Tensor& src, c10d::ReduceOp::RedOpType op);
/// Reduce, then record a fence on the stream; returns its ticket.
uint64_t metal_reduce_op_fenced(const at::Tensor& dst, const at::Tensor& src,
                                c10d::ReduceOp::RedOpType op);

/// metal_reduce_op on a list of (dst, src) pairs that do not depend on one another, in one
/// launch per 128 pairs; every pair's result is bit-identical to metal_reduce_op on it.  No
/// counterpart in the reference's header: its ring loop issues the folds of one ring step
/// one by one (csrc/backend/ProcessGroupMCCL.cpp:492-512).  All tensors share dtype and device;
/// a destination that overlaps another pair's destination or source throws.
void hip_reduce_op_batch(const std::vector<at::Tensor>& dsts, const std::vector<at::Tensor>& srcs,
                         c10d::ReduceOp::RedOpType op);

void metal_scale_inplace(const at::Tensor& buf, double scale);
void metal_accumulate_and_scale(const at::Tensor& dst, const at::Tensor& src, double scale);

/// Block until everything enqueued on the current stream has completed.
void metal_sync();
void metal_sync_queue_only();

/// W-way fold of `ins` (one tensor per simulated rank) in ring-step order into
/// `out`; AVG multiplies by 1/ins.size() at the end.  No counterpart in the
/// reference's header: there the same arithmetic is spread over ws-1 calls of
/// metal_reduce_op_fenced per chunk plus metal_scale_inplace
/// (csrc/backend/ProcessGroupMCCL.cpp:492-512,:1954-1956).
void hip_ring_fold(const at::Tensor& out, const std::vector<at::Tensor>& ins,
                   c10d::ReduceOp::RedOpType op, bool chunked_ring, int64_t bucket_elems,
                   bool stepwise_rounding);

// ---- fences (csrc/metal/EventSync.hpp) --------------------------------------
void event_sync_init();
bool event_sync_available();
uint64_t next_fence_event_value();
void signal_mccl_fence_gpu(uint64_t value);
void wait_for_mccl_fence(uint64_t value);

// ---- raw-pointer folds (csrc/metal/AccelerateOps.hpp:18-59) -----------------
// Same names and argument order.  The reference hands these memory that CPU and
// GPU share; here the pointers must be memory a kernel on the current device can
// reach (device, managed or pinned host memory): each call checks that first and
// throws TensorError otherwise, before anything is launched.  The calls return
// after the work has completed, like the reference's host folds.
void cpu_accumulate(float* dst, const float* src, int64_t count);
void cpu_scale_inplace(float* buf, int64_t count, float scale);
void cpu_accumulate_and_scale(float* dst, const float* src, int64_t count, float scale);
void cpu_elementwise_min(float* dst, const float* src, int64_t count);
void cpu_elementwise_max(float* dst, const float* src, int64_t count);
void cpu_elementwise_product(float* dst, const float* src, int64_t count);
void cpu_reduce_op(float* dst, const float* src, int64_t count, c10d::ReduceOp::RedOpType op);
void cpu_reduce_op_half(c10::Half* dst, const c10::Half* src, int64_t count, c10d::ReduceOp::RedOpType op);
void cpu_scale_inplace_half(c10::Half* buf, int64_t count, float scale);
void cpu_accumulate_and_scale_half(c10::Half* dst, const c10::Half* src, int64_t count, float scale);
void cpu_reduce_op_bf16(c10::BFloat16* dst, const c10::BFloat16* src, int64_t count,
                        c10d::ReduceOp::RedOpType op);
void cpu_scale_inplace_bf16(c10::BFloat16* buf, int64_t count, float scale);
void cpu_accumulate_and_scale_bf16(c10::BFloat16* dst, const c10::BFloat16* src, int64_t count,
                                   float scale);
void cpu_reduce_op_integral(void* dst, const void* src, int64_t count, at::ScalarType dtype,
                            c10d::ReduceOp::RedOpType op);
void cpu_scale_inplace_integral(void* buf, int64_t count, at::ScalarType dtype, float scale);

/// Throws the MCCLError matching a negative C-ABI status.
void throw_on_status(int rc, const char* where);

}  // namespace mccl
