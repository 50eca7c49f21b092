// fp16 transport compression (csrc/compression/FP16Compression.hpp:15-32),
// device resident: a float32 bucket is narrowed to half precision for the wire
// and widened again by the receiver; a float16 bucket passes through as a copy.
#pragma once

#include "Compression.hpp"

namespace mccl {

class FP16Compressor : public Compressor {
public:
    size_t compress(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                    at::ScalarType dtype, uint64_t stable_id = 0) override;
    void decompress(const void* src, size_t compressed_size, void* dst, size_t nbytes,
                    at::ScalarType dtype) override;
    size_t max_compressed_size(size_t nbytes) const override { return nbytes; }
    std::string name() const override { return "fp16"; }
};

}  // namespace mccl
