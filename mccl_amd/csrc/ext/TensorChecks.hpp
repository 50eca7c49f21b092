// Tensor pre-checks and buffer extraction for the kernel entry points.
//
// check_single_tensor / check_same_shape_dtype / tensor_nbytes keep the
// conditions of csrc/common/TensorChecks.hpp:10-56 with the device rule changed
// from "MPS or CPU" to "a ROCm device tensor".  extract_hip_buffer plays the
// part of extract_mps_buffer (csrc/metal/MPSInterop.mm:414-442): a contiguous
// tensor becomes base pointer + byte offset + size; on this hardware that is
// just data_ptr().
#pragma once

#include <torch/torch.h>

#include <cstddef>
#include <string>

#include "Errors.hpp"

namespace mccl {

namespace detail {
// Element types a collective accepts: the training types, the metadata types and float64.
inline bool accepted_dtype(at::ScalarType dt) {
    constexpr at::ScalarType kAccepted[] = {at::kFloat, at::kHalf, at::kBFloat16, at::kLong,
                                            at::kInt,   at::kBool, at::kByte,     at::kDouble};
    for (at::ScalarType a : kAccepted)
        if (a == dt) return true;
    return false;
}
}  // namespace detail

// Empty tensors pass: collectives treat them as no-ops.
inline void check_single_tensor(const at::Tensor& t) {
    if (!t.is_cuda())
        detail::fail<TensorError>("Tensor check failed: ", "t.is_cuda()", nullptr, 0,
                                  "MCCL requires tensors on a ROCm GPU device, got device: " + t.device().str());
    if (!t.is_contiguous())
        detail::fail<TensorError>("Tensor check failed: ", "t.is_contiguous()", nullptr, 0,
                                  "MCCL v1 requires contiguous tensors. Call .contiguous() before passing to "
                                  "collective.");
    if (!detail::accepted_dtype(t.scalar_type()))
        detail::fail<TensorError>("Tensor check failed: ", "accepted_dtype(t.scalar_type())", nullptr, 0,
                                  std::string("MCCL supports float32/float16/bfloat16 (training), "
                                              "int64/int32/bool/uint8 (metadata), and float64, got: ") +
                                      at::toString(t.scalar_type()));
}

inline void check_same_shape_dtype(const at::Tensor& a, const at::Tensor& b) {
    const bool same_shape = a.sizes() == b.sizes();
    const bool same_dtype = a.scalar_type() == b.scalar_type();
    if (!same_shape || !same_dtype)
        detail::fail<TensorError>("Tensor check failed: ", same_shape ? "same dtype" : "same shape", nullptr, 0,
                                  same_shape ? "Dtype mismatch in collective" : "Shape mismatch in collective");
}

inline size_t tensor_nbytes(const at::Tensor& t) { return t.element_size() * static_cast<size_t>(t.numel()); }

struct HipBufferView {
    void* base;          // start of the storage
    size_t byte_offset;  // offset of the tensor's first element inside it
    size_t nbytes;
    void* ptr;           // base + byte_offset: what the kernels receive
    int device;
};

inline HipBufferView extract_hip_buffer(const at::Tensor& t) {
    check_single_tensor(t);
    HipBufferView v;
    v.byte_offset = static_cast<size_t>(t.storage_offset()) * t.element_size();
    v.nbytes = tensor_nbytes(t);
    v.ptr = t.data_ptr();
    v.base = static_cast<char*>(v.ptr) - v.byte_offset;
    v.device = t.get_device();
    return v;
}

}  // namespace mccl
