// Top-k sparsification with error feedback
// (csrc/compression/TopKCompression.hpp:21-60), device resident.
// Wire format: [uint32 count][count x (uint32 index, float value)].
#pragma once

#include <mutex>
#include <unordered_map>
#include <vector>

#include "Compression.hpp"

namespace mccl {

class TopKCompressor : public Compressor {
public:
    explicit TopKCompressor(double k_ratio);
    ~TopKCompressor() override;

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

    /// compress() for a list of buckets (float32 device tensors, one stable id each), the shape
    /// of a coalesced allreduce (csrc/backend/ProcessGroupMCCL.cpp:2257-2313 walks its tensor
    /// list bucket by bucket).  Returns one payload tensor per bucket, identical to what the
    /// per-bucket calls give.  A bucket's launches are latency-bound (and fifteen calls are
    /// bound by the host's launch rate), so the whole list goes through the same two launches
    /// (mccl_hip_topk_compress_list).
    std::vector<at::Tensor> compress_many(const std::vector<at::Tensor>& buckets,
                                          const std::vector<uint64_t>& stable_ids);

    /// Waits for the stream and throws TimeoutError if a compress launch since the last check
    /// gave up (its payload headers then hold 0xFFFFFFFF and decompress rejects them).  No
    /// counterpart in the reference, whose compress is synchronous host code.
    void check_compress_status();

    double k_ratio() const { return k_ratio_; }

private:
    double k_ratio_;
    mutable std::mutex mu_;
    // stable id -> fp32 residual in HBM, one element per gradient element
    std::unordered_map<uint64_t, at::Tensor> error_buffers_;
    at::Tensor workspace_;       // scratch of a one-bucket call
    at::Tensor list_workspace_;  // scratch of a list call
    at::Tensor status_;  // device int32[1], written by decompress
    at::Tensor compress_status_;  // device int32[1], written by a compress launch that gives up
    int* compress_status();
    void throw_if_compress_failed();
    at::Tensor& residual_for(uint64_t stable_id, size_t count);
    size_t compress_on(const void* src, size_t nbytes, void* dst, size_t dst_capacity, at::Tensor& residual,
                       at::Tensor& workspace, void* stream);
    static constexpr size_t kMaxErrorBuffers = 1024;
};

}  // namespace mccl
