#include "Compression.hpp"

#include <c10/hip/HIPStream.h>

#include <algorithm>

#include "../../../include/mccl_hip.h"
#include <hip/hip_runtime_api.h>

#include "Errors.hpp"
#include "FP16Compression.hpp"
#include "HipKernels.hpp"
#include "Logging.hpp"
#include "TensorChecks.hpp"
#include "TopKCompression.hpp"

namespace mccl {

std::unique_ptr<Compressor> make_compressor(CompressionMode mode, double param) {
    switch (mode) {
        case CompressionMode::NONE: return nullptr;
        case CompressionMode::FP16: return std::make_unique<FP16Compressor>();
        case CompressionMode::TOPK: return std::make_unique<TopKCompressor>(param > 0 ? param : 0.01);
        default:
            throw MCCLError("Unknown compression mode: " + std::to_string(static_cast<int>(mode)));
    }
}

namespace {
void device_copy(void* dst, const void* src, size_t nbytes) {
    if (nbytes == 0) return;
    const hipError_t e = hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice,
                                        c10::hip::getCurrentHIPStream().stream());
    MCCL_CHECK(e == hipSuccess, std::string("FP16 passthrough copy failed: ") + hipGetErrorString(e));
}
}  // namespace

// csrc/compression/FP16Compression.cpp:117-143
size_t FP16Compressor::compress(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                                at::ScalarType dtype, uint64_t /*stable_id*/) {
    if (dtype == at::kHalf) {
        MCCL_CHECK(dst_capacity >= nbytes, "FP16 compress: buffer too small");
        device_copy(dst, src, nbytes);
        return nbytes;
    }
    MCCL_CHECK(dtype == at::kFloat, "FP16 compression only supports float32 input");
    const size_t count = nbytes / sizeof(float);
    const size_t compressed_bytes = count * sizeof(uint16_t);
    MCCL_CHECK(dst_capacity >= compressed_bytes, "FP16 compress: buffer too small");
    throw_on_status(mccl_hip_cast_f32_to_f16(static_cast<const float*>(src), dst, count,
                                             c10::hip::getCurrentHIPStream().stream()),
                    "FP16 compress");
    MCCL_TRACE("FP16 compress: %zu -> %zu bytes", nbytes, compressed_bytes);
    return compressed_bytes;
}

// csrc/compression/FP16Compression.cpp:145-163
void FP16Compressor::decompress(const void* src, size_t compressed_size, void* dst, size_t nbytes,
                                at::ScalarType dtype) {
    if (dtype == at::kHalf) {
        MCCL_CHECK(compressed_size == nbytes, "FP16 decompress: size mismatch");
        device_copy(dst, src, nbytes);
        return;
    }
    MCCL_CHECK(dtype == at::kFloat, "FP16 decompression only supports float32 output");
    const size_t count = nbytes / sizeof(float);
    MCCL_CHECK(compressed_size == count * sizeof(uint16_t), "FP16 decompress: compressed size mismatch");
    throw_on_status(mccl_hip_cast_f16_to_f32(src, static_cast<float*>(dst), count,
                                             c10::hip::getCurrentHIPStream().stream()),
                    "FP16 decompress");
}

TopKCompressor::TopKCompressor(double k_ratio) : k_ratio_(k_ratio) {
    MCCL_CHECK(k_ratio > 0 && k_ratio <= 1.0, "k_ratio must be in (0, 1], got " + std::to_string(k_ratio));
}

TopKCompressor::~TopKCompressor() = default;

// The residual map keeps the reference's rules (csrc/compression/TopKCompression.cpp:57-67):
// a new id while 1024 ids are live clears the map; an id whose element count changed starts
// again from zeros.  Caller holds mu_.
at::Tensor& TopKCompressor::residual_for(uint64_t stable_id, size_t count) {
    const auto opts_f = at::TensorOptions().dtype(at::kFloat).device(at::kCUDA);
    if (error_buffers_.size() >= kMaxErrorBuffers && error_buffers_.find(stable_id) == error_buffers_.end()) {
        MCCL_WARN("TopK: evicting all %zu error feedback buffers (unstable tensor identities?)",
                  error_buffers_.size());
        error_buffers_.clear();
    }
    auto it = error_buffers_.find(stable_id);
    if (it == error_buffers_.end() || static_cast<size_t>(it->second.numel()) != count) {
        error_buffers_[stable_id] = at::zeros({static_cast<int64_t>(count)}, opts_f);
    }
    return error_buffers_[stable_id];
}

// The device word the compress launches report a give-up through (a block of the single-pass
// path that waited too long for another block of its launch).  The launches are asynchronous,
// so the word is looked at by the calls that wait for the stream anyway: decompress() and
// check_compress_status().  Caller holds mu_.
int* TopKCompressor::compress_status() {
    if (!compress_status_.defined())
        compress_status_ = at::zeros({1}, at::TensorOptions().dtype(at::kInt).device(at::kCUDA));
    return compress_status_.data_ptr<int>();
}

void TopKCompressor::throw_if_compress_failed() {
    if (!compress_status_.defined()) return;
    const int st = compress_status_.item<int>();
    if (st == 0) return;
    compress_status_.zero_();
    if (st == MCCL_HIP_ERR_TIMEOUT)
        throw TimeoutError("TopK compress: a block gave up waiting for another block of its launch; "
                           "the payloads of that call are invalid");
    throw_on_status(st, "TopK compress");
}

void TopKCompressor::check_compress_status() {
    std::lock_guard<std::mutex> lock(mu_);
    throw_if_compress_failed();
}

// One bucket on `stream`: csrc/compression/TopKCompression.cpp:38-120.  Caller holds mu_.
size_t TopKCompressor::compress_on(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                                   at::Tensor& residual, at::Tensor& workspace, void* stream) {
    const size_t count = nbytes / sizeof(float);
    const uint32_t k = mccl_hip_topk_k(count, k_ratio_);
    const size_t output_size = sizeof(uint32_t) + static_cast<size_t>(k) * 8;
    const uint64_t ws_bytes = mccl_hip_topk_workspace_bytes(count, count, k_ratio_);
    if (!workspace.defined() || static_cast<uint64_t>(workspace.numel()) < ws_bytes) {
        workspace = at::empty({static_cast<int64_t>(ws_bytes)},
                              at::TensorOptions().dtype(at::kByte).device(at::kCUDA));
    }
    // The payload's pairs start 4 bytes in; the stride only has to be a multiple of 4.
    const uint64_t stride = static_cast<uint64_t>(dst_capacity) & ~uint64_t(3);
    const int rc = mccl_hip_topk_compress(static_cast<const float*>(src), residual.data_ptr<float>(), count,
                                          count, k_ratio_, dst, stride, workspace.data_ptr(),
                                          static_cast<uint64_t>(workspace.numel()), compress_status(), stream);
    if (rc == MCCL_HIP_ERR_CAPACITY) throw MCCLError("TopK compress: buffer too small");
    throw_on_status(rc, "TopK compress");
    MCCL_TRACE("TopK compress: %zu elements -> %u values, output %zu bytes", count, k, output_size);
    return output_size;
}

size_t TopKCompressor::compress(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                                at::ScalarType dtype, uint64_t stable_id) {
    MCCL_CHECK(dtype == at::kFloat, "TopK compression currently supports float32 only");
    const size_t count = nbytes / sizeof(float);
    MCCL_CHECK(count > 0, "TopK compress: empty input");
    const uint32_t k = mccl_hip_topk_k(count, k_ratio_);
    MCCL_CHECK(dst_capacity >= sizeof(uint32_t) + static_cast<size_t>(k) * 8, "TopK compress: buffer too small");
    std::lock_guard<std::mutex> lock(mu_);
    metal_kernels_init();
    at::Tensor& residual = residual_for(stable_id, count);
    return compress_on(src, nbytes, dst, dst_capacity, residual, workspace_,
                       c10::hip::getCurrentHIPStream().stream());
}

std::vector<at::Tensor> TopKCompressor::compress_many(const std::vector<at::Tensor>& buckets,
                                                      const std::vector<uint64_t>& stable_ids) {
    MCCL_CHECK(buckets.size() == stable_ids.size(), "compress_many: one stable id per bucket");
    std::vector<at::Tensor> payloads;
    if (buckets.empty()) return payloads;
    std::lock_guard<std::mutex> lock(mu_);
    metal_kernels_init();
    std::vector<at::Tensor*> residuals;
    for (size_t i = 0; i < buckets.size(); i++) {
        const at::Tensor& t = buckets[i];
        check_single_tensor(t);
        MCCL_CHECK(t.scalar_type() == at::kFloat, "TopK compression currently supports float32 only");
        MCCL_CHECK(t.numel() > 0, "TopK compress: empty input");
        for (size_t j = 0; j < i; j++)
            MCCL_CHECK(stable_ids[j] != stable_ids[i], "compress_many: the same stable id twice in one call");
        payloads.push_back(at::empty({static_cast<int64_t>(max_compressed_size(tensor_nbytes(t)))},
                                     at::TensorOptions().dtype(at::kByte).device(t.device())));
    }
    // (a second loop: residual_for may clear the map when the 1025th id arrives, and the
    // references it returned before that would dangle)
    for (size_t i = 0; i < buckets.size(); i++) residual_for(stable_ids[i], static_cast<size_t>(buckets[i].numel()));
    for (size_t i = 0; i < buckets.size(); i++) {
        auto it = error_buffers_.find(stable_ids[i]);
        MCCL_CHECK(it != error_buffers_.end() && it->second.numel() == buckets[i].numel(),
                   "compress_many: more distinct stable ids than the compressor holds residuals for");
        residuals.push_back(&it->second);
    }
    // the list goes to the library in chunks of MCCL_HIP_TOPK_LIST_MAX buckets: two launches per chunk
    const int device = buckets[0].get_device();
    void* stream = c10::hip::getCurrentHIPStream(device).stream();
    std::vector<size_t> used(buckets.size());
    for (size_t first = 0; first < buckets.size(); first += MCCL_HIP_TOPK_LIST_MAX) {
        const size_t n = std::min<size_t>(MCCL_HIP_TOPK_LIST_MAX, buckets.size() - first);
        std::vector<const float*> grads(n);
        std::vector<float*> res(n);
        std::vector<uint64_t> counts(n), caps(n);
        std::vector<void*> wires(n);
        for (size_t i = 0; i < n; i++) {
            grads[i] = buckets[first + i].data_ptr<float>();
            res[i] = residuals[first + i]->data_ptr<float>();
            counts[i] = static_cast<uint64_t>(buckets[first + i].numel());
            wires[i] = payloads[first + i].data_ptr();
            caps[i] = static_cast<uint64_t>(payloads[first + i].numel());
            used[first + i] = sizeof(uint32_t) + static_cast<size_t>(mccl_hip_topk_k(counts[i], k_ratio_)) * 8;
        }
        const uint64_t need = mccl_hip_topk_list_workspace_bytes(counts.data(), static_cast<uint32_t>(n), k_ratio_);
        if (!list_workspace_.defined() || static_cast<uint64_t>(list_workspace_.numel()) < need)
            list_workspace_ = at::empty({static_cast<int64_t>(need)},
                                        at::TensorOptions().dtype(at::kByte).device(at::kCUDA));
        const int rc = mccl_hip_topk_compress_list(grads.data(), res.data(), counts.data(), wires.data(), caps.data(),
                                                   static_cast<uint32_t>(n), k_ratio_, list_workspace_.data_ptr(),
                                                   static_cast<uint64_t>(list_workspace_.numel()), compress_status(),
                                                   stream);
        if (rc == MCCL_HIP_ERR_CAPACITY) throw MCCLError("TopK compress: buffer too small");
        throw_on_status(rc, "TopK compress");
    }
    for (size_t i = 0; i < buckets.size(); i++) payloads[i] = payloads[i].narrow(0, 0, static_cast<int64_t>(used[i]));
    return payloads;
}

// csrc/compression/TopKCompression.cpp:122-152.  The reference validates while
// it scatters and throws; here the kernel reports through a device flag that
// is read back once the stream has drained (the call is synchronous, as the
// reference's is).
void TopKCompressor::decompress(const void* src, size_t compressed_size, void* dst, size_t nbytes,
                                at::ScalarType dtype) {
    MCCL_CHECK(dtype == at::kFloat, "TopK decompression currently supports float32 only");
    const size_t count = nbytes / sizeof(float);
    std::lock_guard<std::mutex> lock(mu_);
    metal_kernels_init();
    if (!status_.defined()) status_ = at::zeros({1}, at::TensorOptions().dtype(at::kInt).device(at::kCUDA));
    status_.zero_();
    const int rc = mccl_hip_topk_decompress(src, compressed_size, static_cast<float*>(dst), count,
                                            status_.data_ptr<int>(), c10::hip::getCurrentHIPStream().stream());
    if (rc == MCCL_HIP_ERR_SIZE) throw MCCLError("TopK decompress: size mismatch");
    throw_on_status(rc, "TopK decompress");
    const int st = status_.item<int>();
    throw_if_compress_failed();
    if (st == MCCL_HIP_ERR_SIZE) throw MCCLError("TopK decompress: size mismatch");
    if (st == MCCL_HIP_ERR_INDEX) throw MCCLError("TopK decompress: index out of bounds");
}

size_t TopKCompressor::max_compressed_size(size_t nbytes) const {
    return static_cast<size_t>(mccl_hip_topk_max_compressed_size(nbytes, k_ratio_));
}

void TopKCompressor::reset_error_feedback() {
    std::lock_guard<std::mutex> lock(mu_);
    error_buffers_.clear();
    MCCL_DEBUG("TopK: all error feedback buffers reset");
}

void TopKCompressor::reset_error_feedback_for_tensor(uint64_t stable_id) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = error_buffers_.find(stable_id);
    if (it != error_buffers_.end()) it->second.zero_();
}

size_t TopKCompressor::error_feedback_buffer_count() const {
    std::lock_guard<std::mutex> lock(mu_);
    return error_buffers_.size();
}

at::Tensor TopKCompressor::error_feedback_buffer(uint64_t stable_id) const {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = error_buffers_.find(stable_id);
    return it == error_buffers_.end() ? at::Tensor() : it->second;
}

}  // namespace mccl
