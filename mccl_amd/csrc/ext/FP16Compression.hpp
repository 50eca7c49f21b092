// fp16 transport compression (csrc/compression/FP16Compression.hpp:15-32),
// device resident: a float32 bucket is narrowed to half precision for the wire
// and widened again by the receiver; a float16 bucket passes through as a copy.
// Stateless; name() is "fp16" and the payload is never larger than the input.
#pragma once

#include "Compression.hpp"

namespace mccl {

class FP16Compressor : public Compressor {
public:
    MCCL_COMPRESSOR_MEMBERS(, override)
};

}  // namespace mccl
