// Compressor interface of the reference (csrc/compression/Compression.hpp:12-52)
// with the same virtual signatures.  `src` / `dst` are DEVICE pointers here:
// the gradient bucket, the compressed payload and the error-feedback residual
// all stay in HBM.
#pragma once

#include <torch/torch.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>

namespace mccl {

enum class CompressionMode : int {
    NONE = 0,
    FP16 = 1,
    TOPK = 2,
};

class Compressor {
public:
    virtual ~Compressor() = default;

    /// Compresses nbytes at src into dst (capacity dst_capacity); returns the
    /// payload size.  stable_id names the logical tensor across steps; stateful
    /// compressors key their residual on it.
    virtual size_t compress(const void* src, size_t nbytes, void* dst, size_t dst_capacity,
                            at::ScalarType dtype, uint64_t stable_id = 0) = 0;

    /// Expands compressed_size bytes at src into nbytes at dst.
    virtual void decompress(const void* src, size_t compressed_size, void* dst, size_t nbytes,
                            at::ScalarType dtype) = 0;

    virtual size_t max_compressed_size(size_t nbytes) const = 0;
    virtual std::string name() const = 0;
};

/// NONE -> nullptr, FP16 -> FP16Compressor, TOPK -> TopKCompressor(param > 0 ?
/// param : 0.01); anything else throws (csrc/compression/Compression.cpp:8-20).
std::unique_ptr<Compressor> make_compressor(CompressionMode mode, double param = 0.0);

}  // namespace mccl
