// Top-k sparsification with error feedback
// (csrc/compression/TopKCompression.hpp:21-60), device resident.
// Wire format: [uint32 count][count x (uint32 index, float value)].
#pragma once

#include <mutex>
#include <unordered_map>

#include "Compression.hpp"

namespace mccl {

class TopKCompressor : public Compressor {
public:
    explicit TopKCompressor(double k_ratio);

    size_t compress(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                    at::ScalarType dtype, uint64_t stable_id = 0) override;
    void decompress(const void* src, size_t compressed_size, void* dst, size_t nbytes,
                    at::ScalarType dtype) override;
    size_t max_compressed_size(size_t nbytes) const override;
    std::string name() const override { return "topk"; }

    void reset_error_feedback();
    void reset_error_feedback_for_tensor(uint64_t stable_id);
    size_t error_feedback_buffer_count() const;

    /// The residual kept for stable_id (undefined tensor if none); for
    /// checkpointing and tests.
    at::Tensor error_feedback_buffer(uint64_t stable_id) const;

    double k_ratio() const { return k_ratio_; }

private:
    double k_ratio_;
    mutable std::mutex mu_;
    // stable id -> fp32 residual in HBM, one element per gradient element
    std::unordered_map<uint64_t, at::Tensor> error_buffers_;
    at::Tensor workspace_;
    at::Tensor status_;  // device int32[1], written by decompress
    static constexpr size_t kMaxErrorBuffers = 1024;
};

}  // namespace mccl
