// ref_shim.cpp -- TEST INFRASTRUCTURE ONLY.
//
// C binding over the reference's own compression classes, compiled together
// with the reference sources where they lie (see oracle/Makefile, target
// `ref`).  Nothing here restates an algorithm: every call goes straight into
// mccl::TopKCompressor / mccl::make_compressor from
// csrc/compression/{Compression,TopKCompression,FP16Compression}.cpp.
#include "compression/Compression.hpp"
#include "compression/TopKCompression.hpp"

#include <cstdint>
#include <cstdio>
#include <exception>

extern "C" {

void* ref_make_compressor(int mode, double param) {
    try {
        return mccl::make_compressor(static_cast<mccl::CompressionMode>(mode), param).release();
    } catch (const std::exception& e) {
        std::fprintf(stderr, "ref_make_compressor: %s\n", e.what());
        return nullptr;
    }
}

void ref_free_compressor(void* c) { delete static_cast<mccl::Compressor*>(c); }

// Returns compressed bytes, or -1 when the reference throws.
long long ref_compress(void* c, const void* src, unsigned long long nbytes, void* dst,
                       unsigned long long cap, int dtype, unsigned long long stable_id) {
    try {
        return static_cast<long long>(static_cast<mccl::Compressor*>(c)->compress(
            src, nbytes, dst, cap, static_cast<at::ScalarType>(dtype), stable_id));
    } catch (const std::exception&) {
        return -1;
    }
}

int ref_decompress(void* c, const void* src, unsigned long long csize, void* dst,
                   unsigned long long nbytes, int dtype) {
    try {
        static_cast<mccl::Compressor*>(c)->decompress(src, csize, dst, nbytes,
                                                      static_cast<at::ScalarType>(dtype));
        return 0;
    } catch (const std::exception&) {
        return -1;
    }
}

unsigned long long ref_max_compressed_size(void* c, unsigned long long nbytes) {
    return static_cast<mccl::Compressor*>(c)->max_compressed_size(nbytes);
}

unsigned long long ref_error_feedback_buffer_count(void* c) {
    auto* t = dynamic_cast<mccl::TopKCompressor*>(static_cast<mccl::Compressor*>(c));
    return t ? t->error_feedback_buffer_count() : 0;
}

void ref_reset_error_feedback(void* c) {
    auto* t = dynamic_cast<mccl::TopKCompressor*>(static_cast<mccl::Compressor*>(c));
    if (t) t->reset_error_feedback();
}

void ref_reset_error_feedback_for_tensor(void* c, unsigned long long id) {
    auto* t = dynamic_cast<mccl::TopKCompressor*>(static_cast<mccl::Compressor*>(c));
    if (t) t->reset_error_feedback_for_tensor(id);
}

}  // extern "C"
