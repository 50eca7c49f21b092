// Host dispatch of the local kernels: checks, buffer extraction, one C-ABI
// call on torch's current HIP stream.  Mirrors the control flow of
// csrc/metal/MetalKernels.mm:521-824 (op switch, dtype -> kernel selection,
// error text) without its command-buffer and CPU-fallback branches: on this
// hardware every size runs on the GPU.
#include "HipKernels.hpp"

#include <c10/hip/HIPStream.h>

#include <atomic>
#include <mutex>
#include <string>

#include "../../../include/mccl_hip.h"
#include "Errors.hpp"
#include "Logging.hpp"
#include "TensorChecks.hpp"

namespace mccl {

namespace {

// Serialises launches like the reference's process-wide recursive kernel mutex
// (csrc/metal/MetalKernels.mm:74); the C ABI itself is re-entrant.
std::recursive_mutex g_kernel_mutex;
std::atomic<bool> g_initialized{false};

void* current_stream(int device) { return c10::hip::getCurrentHIPStream(device).stream(); }

bool op_is_unsupported(c10d::ReduceOp::RedOpType op) {
    return !(op == c10d::ReduceOp::SUM || op == c10d::ReduceOp::AVG || op == c10d::ReduceOp::MIN ||
             op == c10d::ReduceOp::MAX || op == c10d::ReduceOp::PRODUCT);
}

int64_t safe_numel(const at::Tensor& t) {
    const int64_t n = t.numel();
    MCCL_CHECK(n >= 0 && static_cast<uint64_t>(n) <= MCCL_HIP_MAX_ELEMS,
               "Tensor too large for the HIP kernels (" + std::to_string(n) + " elements)");
    return n;
}

int dtype_code(const at::Tensor& t, const char* what) {
    switch (t.scalar_type()) {
        case at::kFloat: return MCCL_HIP_F32;
        case at::kHalf: return MCCL_HIP_F16;
        case at::kBFloat16: return MCCL_HIP_BF16;
        case at::kInt: return MCCL_HIP_I32;
        case at::kLong: return MCCL_HIP_I64;
        case at::kBool: return MCCL_HIP_BOOL;
        case at::kByte: return MCCL_HIP_U8;
        default:
            throw MCCLError(std::string("No HIP ") + what + " kernel for dtype " +
                            std::string(at::toString(t.scalar_type())));
    }
}

void binary(const at::Tensor& dst, const at::Tensor& src, int op, const char* what) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    MCCL_CHECK(g_initialized.load(), "metal_kernels_init() not called");
    check_same_shape_dtype(dst, src);
    HipBufferView d = extract_hip_buffer(dst);
    HipBufferView s = extract_hip_buffer(src);
    MCCL_CHECK_TENSOR(d.device == s.device, "dst and src live on different devices");
    const int64_t n = safe_numel(dst);
    const int rc = mccl_hip_fold2(d.ptr, s.ptr, static_cast<uint64_t>(n), dtype_code(dst, what), op,
                                  current_stream(d.device));
    throw_on_status(rc, what);
}

}  // namespace

void throw_on_status(int rc, const char* where) {
    if (rc == MCCL_HIP_OK) return;
    std::string msg = std::string(where) + ": " + mccl_hip_strerror(rc);
    if (rc == MCCL_HIP_ERR_RUNTIME) {
        msg += " (hipError_t " + std::to_string(mccl_hip_last_hip_error()) + ")";
        throw MetalError(msg);
    }
    if (rc == MCCL_HIP_ERR_TIMEOUT) throw TimeoutError(msg);
    throw MCCLError(msg);
}

void metal_kernels_init() {
    if (g_initialized.load(std::memory_order_acquire)) return;
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    if (g_initialized.load(std::memory_order_acquire)) return;
    throw_on_status(mccl_hip_init(), "metal_kernels_init");
    g_initialized.store(true, std::memory_order_release);
    MCCL_INFO("HIP kernel library initialised (ABI %d)", mccl_hip_abi_version());
}

void metal_accumulate_chunk(const at::Tensor& dst, const at::Tensor& src) {
    binary(dst, src, MCCL_HIP_SUM, "accumulate");
}
void metal_elementwise_min(const at::Tensor& dst, const at::Tensor& src) {
    binary(dst, src, MCCL_HIP_MIN, "min");
}
void metal_elementwise_max(const at::Tensor& dst, const at::Tensor& src) {
    binary(dst, src, MCCL_HIP_MAX, "max");
}
void metal_elementwise_product(const at::Tensor& dst, const at::Tensor& src) {
    binary(dst, src, MCCL_HIP_PRODUCT, "product");
}

void metal_reduce_op(const at::Tensor& dst, const at::Tensor& src, c10d::ReduceOp::RedOpType op) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    switch (op) {
        case c10d::ReduceOp::SUM:
        case c10d::ReduceOp::AVG: metal_accumulate_chunk(dst, src); break;
        case c10d::ReduceOp::MIN: metal_elementwise_min(dst, src); break;
        case c10d::ReduceOp::MAX: metal_elementwise_max(dst, src); break;
        case c10d::ReduceOp::PRODUCT: metal_elementwise_product(dst, src); break;
        default: throw MCCLError("Unsupported ReduceOp: " + std::to_string(static_cast<int>(op)));
    }
}

void hip_reduce_op_batch(const std::vector<at::Tensor>& dsts, const std::vector<at::Tensor>& srcs,
                         c10d::ReduceOp::RedOpType op) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    MCCL_CHECK_TENSOR(dsts.size() == srcs.size(), "as many sources as destinations");
    if (dsts.empty()) return;
    int code;
    switch (op) {
        case c10d::ReduceOp::SUM:
        case c10d::ReduceOp::AVG: code = MCCL_HIP_SUM; break;
        case c10d::ReduceOp::MIN: code = MCCL_HIP_MIN; break;
        case c10d::ReduceOp::MAX: code = MCCL_HIP_MAX; break;
        case c10d::ReduceOp::PRODUCT: code = MCCL_HIP_PRODUCT; break;
        default: throw MCCLError("Unsupported ReduceOp: " + std::to_string(static_cast<int>(op)));
    }
    std::vector<void*> dp(dsts.size());
    std::vector<const void*> sp(dsts.size());
    std::vector<uint64_t> cnt(dsts.size());
    int device = -1;
    for (size_t i = 0; i < dsts.size(); i++) {
        check_same_shape_dtype(dsts[i], srcs[i]);
        MCCL_CHECK_TENSOR(dsts[i].scalar_type() == dsts[0].scalar_type(), "the pairs of one list share a dtype");
        HipBufferView d = extract_hip_buffer(dsts[i]);
        HipBufferView s = extract_hip_buffer(srcs[i]);
        if (device < 0) device = d.device;
        MCCL_CHECK_TENSOR(d.device == device && s.device == device, "the pairs of one list live on one device");
        dp[i] = d.ptr;
        sp[i] = s.ptr;
        cnt[i] = static_cast<uint64_t>(safe_numel(dsts[i]));
    }
    const int rc = mccl_hip_fold2_batch(dp.data(), sp.data(), cnt.data(), static_cast<uint32_t>(dsts.size()),
                                        dtype_code(dsts[0], "reduce_op_batch"), code, current_stream(device));
    throw_on_status(rc, "reduce_op_batch");
}

uint64_t metal_reduce_op_fenced(const at::Tensor& dst, const at::Tensor& src,
                                c10d::ReduceOp::RedOpType op) {
    metal_reduce_op(dst, src, op);
    if (event_sync_available()) {
        const uint64_t v = next_fence_event_value();
        signal_mccl_fence_gpu(v);
        return v;
    }
    metal_sync_queue_only();
    return 0;
}

void metal_scale_inplace(const at::Tensor& buf, double scale) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    MCCL_CHECK(g_initialized.load(), "metal_kernels_init() not called");
    HipBufferView v = extract_hip_buffer(buf);
    const int64_t n = safe_numel(buf);
    // The reference casts the scale to the element type for fp16/bf16
    // (csrc/metal/MetalKernels.mm:595-604); here it stays fp32 and the product
    // is rounded once, as on the reference's CPU path (AccelerateOps.mm:43-52).
    const int rc = mccl_hip_scale(v.ptr, static_cast<uint64_t>(n), dtype_code(buf, "scale"),
                                  static_cast<float>(scale), current_stream(v.device));
    throw_on_status(rc, "scale");
}

void metal_accumulate_and_scale(const at::Tensor& dst, const at::Tensor& src, double scale) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    MCCL_CHECK(g_initialized.load(), "metal_kernels_init() not called");
    check_same_shape_dtype(dst, src);
    HipBufferView d = extract_hip_buffer(dst);
    HipBufferView s = extract_hip_buffer(src);
    MCCL_CHECK_TENSOR(d.device == s.device, "dst and src live on different devices");
    const int64_t n = safe_numel(dst);
    const int rc = mccl_hip_fold2_scale(d.ptr, s.ptr, static_cast<uint64_t>(n), dtype_code(dst, "fused"),
                                        static_cast<float>(scale), current_stream(d.device));
    throw_on_status(rc, "accumulate_and_scale");
}

void metal_sync() {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    throw_on_status(mccl_hip_sync(c10::hip::getCurrentHIPStream().stream()), "metal_sync");
}

void metal_sync_queue_only() { metal_sync(); }

void hip_ring_fold(const at::Tensor& out, const std::vector<at::Tensor>& ins,
                   c10d::ReduceOp::RedOpType op, bool chunked_ring, int64_t bucket_elems,
                   bool stepwise_rounding) {
    std::lock_guard<std::recursive_mutex> lock(g_kernel_mutex);
    MCCL_CHECK(g_initialized.load(), "metal_kernels_init() not called");
    MCCL_CHECK(!ins.empty() && ins.size() <= MCCL_HIP_MAX_WORLD, "world size out of range");
    HipBufferView o = extract_hip_buffer(out);
    std::vector<const void*> ptrs;
    for (const auto& t : ins) {
        check_same_shape_dtype(out, t);
        HipBufferView v = extract_hip_buffer(t);
        MCCL_CHECK_TENSOR(v.device == o.device, "rank buffers live on different devices");
        ptrs.push_back(v.ptr);
    }
    const int64_t n = safe_numel(out);
    const bool avg = op == c10d::ReduceOp::AVG;
    const int ws = static_cast<int>(ins.size());
    const int rc = mccl_hip_ring_fold(o.ptr, ptrs.data(), ws, static_cast<uint64_t>(n),
                                      bucket_elems > 0 ? static_cast<uint64_t>(bucket_elems)
                                                       : static_cast<uint64_t>(n > 0 ? n : 1),
                                      chunked_ring ? MCCL_HIP_RING_CHUNKED : MCCL_HIP_RING_BASIC,
                                      dtype_code(out, "ring fold"), static_cast<int>(op), avg ? 1 : 0,
                                      static_cast<float>(1.0 / ws), stepwise_rounding ? 1 : 0,
                                      current_stream(o.device));
    throw_on_status(rc, "ring_fold");
}

// ---- fences -----------------------------------------------------------------
// A fence value IS the C ABI's ticket.  The reference hands out the value first
// and signals afterwards (EventSync.mm:189-200); here recording produces the
// ticket, so next_fence_event_value() records and signal_mccl_fence_gpu() has
// nothing left to do for that value.
void event_sync_init() { metal_kernels_init(); }

bool event_sync_available() {
    static const bool enabled = [] {
        const char* v = std::getenv("MCCL_EVENT_SYNC");
        if (!v) return true;
        const std::string s(v);
        return !(s == "0" || s == "false" || s == "FALSE" || s == "no" || s == "NO");
    }();
    return enabled && g_initialized.load();
}

uint64_t next_fence_event_value() {
    uint64_t ticket = 0;
    throw_on_status(mccl_hip_fence_signal(c10::hip::getCurrentHIPStream().stream(), &ticket),
                    "next_fence_event_value");
    return ticket;
}

void signal_mccl_fence_gpu(uint64_t) {}

void wait_for_mccl_fence(uint64_t value) {
    const int rc = mccl_hip_fence_wait(value, 0);
    if (rc == MCCL_HIP_ERR_TIMEOUT)
        throw TimeoutError("wait_for_mccl_fence timed out after 30s waiting for event value " +
                           std::to_string(value));
    throw_on_status(rc, "wait_for_mccl_fence");
}

// ---- raw-pointer folds --------------------------------------------------------
// The reference calls this family with view.cpu_ptr, memory the CPU and the GPU
// share (csrc/backend/ProcessGroupMCCL.cpp:494-498).  Here the arithmetic runs in
// a kernel, so every pointer is first resolved to an address a kernel can use:
// device memory of the current GPU, managed memory, or pinned host memory (its
// device-side alias).  Anything else, pageable host memory above all, throws
// before a kernel is launched; there is no host fallback.
namespace {
size_t elem_bytes(int dtype) {
    switch (dtype) {
        case MCCL_HIP_F32: case MCCL_HIP_I32: return 4;
        case MCCL_HIP_F16: case MCCL_HIP_BF16: return 2;
        case MCCL_HIP_I64: return 8;
        default: return 1;
    }
}
void* kernel_pointer(const void* p, int64_t n, int dtype, const char* what) {
    MCCL_CHECK(n >= 0 && static_cast<uint64_t>(n) <= MCCL_HIP_MAX_ELEMS,
               std::string(what) + ": element count out of range");
    if (n == 0) return const_cast<void*>(p);
    void* dp = nullptr;
    const int rc = mccl_hip_pointer_check(p, static_cast<uint64_t>(n) * elem_bytes(dtype), &dp);
    if (rc == MCCL_HIP_ERR_POINTER || rc == MCCL_HIP_ERR_ARG)
        throw TensorError(std::string(what) + ": the buffer is not memory a GPU kernel can reach (device, managed "
                          "or pinned host memory of the current device is required; pageable host memory is "
                          "not accepted and there is no host fallback)");
    throw_on_status(rc, what);
    return dp;
}
void raw_fold(void* dst, const void* src, int64_t n, int dtype, c10d::ReduceOp::RedOpType op,
              const char* what) {
    metal_kernels_init();
    if (op_is_unsupported(op))
        throw MCCLError(std::string("Unsupported ReduceOp for ") + what + ": " +
                        std::to_string(static_cast<int>(op)));
    void* d = kernel_pointer(dst, n, dtype, what);
    const void* s = kernel_pointer(src, n, dtype, what);
    void* st = c10::hip::getCurrentHIPStream().stream();
    throw_on_status(mccl_hip_fold2(d, s, static_cast<uint64_t>(n), dtype, static_cast<int>(op), st), what);
    throw_on_status(mccl_hip_sync(st), what);
}
void raw_scale(void* buf, int64_t n, int dtype, float scale) {
    metal_kernels_init();
    void* b = kernel_pointer(buf, n, dtype, "scale");
    void* st = c10::hip::getCurrentHIPStream().stream();
    throw_on_status(mccl_hip_scale(b, static_cast<uint64_t>(n), dtype, scale, st), "scale");
    throw_on_status(mccl_hip_sync(st), "scale");
}
void raw_fused(void* dst, const void* src, int64_t n, int dtype, float scale) {
    metal_kernels_init();
    void* d = kernel_pointer(dst, n, dtype, "fused");
    const void* s = kernel_pointer(src, n, dtype, "fused");
    void* st = c10::hip::getCurrentHIPStream().stream();
    throw_on_status(mccl_hip_fold2_scale(d, s, static_cast<uint64_t>(n), dtype, scale, st), "fused");
    throw_on_status(mccl_hip_sync(st), "fused");
}
int integral_code(at::ScalarType t, const char* fn) {
    switch (t) {
        case at::kBool: return MCCL_HIP_BOOL;
        case at::kInt: return MCCL_HIP_I32;
        case at::kLong: return MCCL_HIP_I64;
        default: throw MCCLError(std::string(fn) + ": unsupported dtype " + std::string(at::toString(t)));
    }
}
}  // namespace

void cpu_accumulate(float* d, const float* s, int64_t n) { raw_fold(d, s, n, MCCL_HIP_F32, c10d::ReduceOp::SUM, "CPU path"); }
void cpu_scale_inplace(float* b, int64_t n, float sc) { raw_scale(b, n, MCCL_HIP_F32, sc); }
void cpu_accumulate_and_scale(float* d, const float* s, int64_t n, float sc) { raw_fused(d, s, n, MCCL_HIP_F32, sc); }
void cpu_elementwise_min(float* d, const float* s, int64_t n) { raw_fold(d, s, n, MCCL_HIP_F32, c10d::ReduceOp::MIN, "CPU path"); }
void cpu_elementwise_max(float* d, const float* s, int64_t n) { raw_fold(d, s, n, MCCL_HIP_F32, c10d::ReduceOp::MAX, "CPU path"); }
void cpu_elementwise_product(float* d, const float* s, int64_t n) { raw_fold(d, s, n, MCCL_HIP_F32, c10d::ReduceOp::PRODUCT, "CPU path"); }
void cpu_reduce_op(float* d, const float* s, int64_t n, c10d::ReduceOp::RedOpType op) { raw_fold(d, s, n, MCCL_HIP_F32, op, "CPU path"); }
void cpu_reduce_op_half(c10::Half* d, const c10::Half* s, int64_t n, c10d::ReduceOp::RedOpType op) { raw_fold(d, s, n, MCCL_HIP_F16, op, "CPU path"); }
void cpu_scale_inplace_half(c10::Half* b, int64_t n, float sc) { raw_scale(b, n, MCCL_HIP_F16, sc); }
void cpu_accumulate_and_scale_half(c10::Half* d, const c10::Half* s, int64_t n, float sc) { raw_fused(d, s, n, MCCL_HIP_F16, sc); }
void cpu_reduce_op_bf16(c10::BFloat16* d, const c10::BFloat16* s, int64_t n, c10d::ReduceOp::RedOpType op) { raw_fold(d, s, n, MCCL_HIP_BF16, op, "CPU path"); }
void cpu_scale_inplace_bf16(c10::BFloat16* b, int64_t n, float sc) { raw_scale(b, n, MCCL_HIP_BF16, sc); }
void cpu_accumulate_and_scale_bf16(c10::BFloat16* d, const c10::BFloat16* s, int64_t n, float sc) { raw_fused(d, s, n, MCCL_HIP_BF16, sc); }
void cpu_reduce_op_integral(void* d, const void* s, int64_t n, at::ScalarType t, c10d::ReduceOp::RedOpType op) {
    raw_fold(d, s, n, integral_code(t, "cpu_reduce_op_integral"), op, "integral CPU path");
}
void cpu_scale_inplace_integral(void* b, int64_t n, at::ScalarType t, float sc) {
    raw_scale(b, n, integral_code(t, "cpu_scale_inplace_integral"), sc);
}

}  // namespace mccl
