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

inline void check_single_tensor(const at::Tensor& t) {
    MCCL_CHECK_TENSOR(t.is_cuda(),
                      "MCCL requires tensors on a ROCm GPU device, got device: " + t.device().str());
    MCCL_CHECK_TENSOR(t.is_contiguous(),
                      "MCCL v1 requires contiguous tensors. Call .contiguous() before passing to collective.");
    const auto dt = t.scalar_type();
    MCCL_CHECK_TENSOR(dt == at::kFloat || dt == at::kHalf || dt == at::kBFloat16 || dt == at::kLong ||
                          dt == at::kInt || dt == at::kBool || dt == at::kByte || dt == at::kDouble,
                      "MCCL supports float32/float16/bfloat16 (training), int64/int32/bool/uint8 "
                      "(metadata), and float64, got: " + std::string(at::toString(dt)));
}

inline void check_same_shape_dtype(const at::Tensor& a, const at::Tensor& b) {
    MCCL_CHECK_TENSOR(a.sizes() == b.sizes(), "Shape mismatch in collective");
    MCCL_CHECK_TENSOR(a.scalar_type() == b.scalar_type(), "Dtype mismatch in collective");
}

inline size_t tensor_nbytes(const at::Tensor& t) {
    return static_cast<size_t>(t.numel()) * t.element_size();
}

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
