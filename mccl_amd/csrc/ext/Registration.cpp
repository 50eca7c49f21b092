// pybind module `mccl_amd._C`: the part of the reference's `mccl._C`
// (csrc/backend/Registration.cpp:220-312) that belongs to the per-rank compute
// path -- version attributes, CompressionMode, MCCLOptions and the six
// `_metal_*` kernel helpers with their "init, sync producer, kernel, sync"
// shape and "returns the same tensor" contract -- plus tensor-level access to
// the compressor and the ring fold.
#include <torch/extension.h>
#include <torch/csrc/utils/pybind.h>

#include <c10/hip/HIPStream.h>

#include "../../../include/mccl_hip.h"
#include "Compression.hpp"
#include "Errors.hpp"
#include "HipKernels.hpp"
#include "Options.hpp"
#include "RingDriver.hpp"
#include "TensorChecks.hpp"
#include "FP16Compression.hpp"
#include "TopKCompression.hpp"

namespace py = pybind11;

namespace {

// Producer-side sync of the helpers: the reference drains torch's MPS stream
// before touching the buffers (mps_stream_sync).  The kernels here run on
// torch's current stream, so ordering is already given; the sync is kept so the
// helpers stay blocking calls.
void producer_sync() { mccl::metal_sync(); }

// Argument checks of the raw-pointer test bindings: the tensors only lend their
// data pointers, so they may be GPU tensors or (pinned) host tensors.
void raw_check(const at::Tensor& dst, const at::Tensor* src, c10::optional<at::ScalarType> only = c10::nullopt) {
    MCCL_CHECK_TENSOR(dst.is_contiguous(), "MCCL v1 requires contiguous tensors. Call .contiguous() before passing "
                                           "to collective.");
    if (src) {
        mccl::check_same_shape_dtype(dst, *src);
        MCCL_CHECK_TENSOR(src->is_contiguous(), "MCCL v1 requires contiguous tensors. Call .contiguous() before "
                                                "passing to collective.");
    }
    if (only) MCCL_CHECK(dst.scalar_type() == *only, "float32 only");
}

// A compressed payload handed to decompress: uint8, contiguous, on the GPU, and
// at least as long as the size the caller says arrived.
void check_payload(const at::Tensor& wire, const py::object& size, int64_t numel) {
    mccl::check_single_tensor(wire);
    MCCL_CHECK_TENSOR(wire.scalar_type() == at::kByte, "compressed payload must be a uint8 tensor");
    MCCL_CHECK(numel >= 0, "decompress: negative element count");
    if (!size.is_none())
        MCCL_CHECK(size.cast<size_t>() <= static_cast<size_t>(wire.numel()),
                   "decompress: compressed_size exceeds the payload tensor");
}

uint64_t stable_id_of(const at::Tensor& t) {
    // storage address + offset, stable across steps for DDP buckets
    // (csrc/backend/ProcessGroupMCCL.cpp:1080-1083)
    return reinterpret_cast<uint64_t>(t.storage().data()) +
           static_cast<uint64_t>(t.storage_offset()) * t.element_size();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.attr("__version__") = "0.5.0";
    m.attr("__protocol_version__") = 5;
    m.attr("__hip_abi_version__") = mccl_hip_abi_version();

    py::enum_<mccl::CompressionMode>(m, "CompressionMode")
        .value("NONE", mccl::CompressionMode::NONE)
        .value("FP16", mccl::CompressionMode::FP16)
        .value("TOPK", mccl::CompressionMode::TOPK);

    py::class_<mccl::MCCLOptions, c10d::Backend::Options, c10::intrusive_ptr<mccl::MCCLOptions>>(m, "MCCLOptions")
        .def(py::init<>())
        .def(py::init<std::chrono::milliseconds>(), py::arg("timeout"))
        .def_readwrite("transport", &mccl::MCCLOptions::transport)
        .def_readwrite("listen_addr", &mccl::MCCLOptions::listen_addr)
        .def_readwrite("port_base", &mccl::MCCLOptions::port_base)
        .def_readwrite("ifname", &mccl::MCCLOptions::ifname)
        .def_readwrite("chunk_bytes", &mccl::MCCLOptions::chunk_bytes)
        .def_readwrite("small_msg_threshold", &mccl::MCCLOptions::small_msg_threshold)
        .def_readwrite("transport_crc", &mccl::MCCLOptions::transport_crc)
        .def_readwrite("fast_math", &mccl::MCCLOptions::fast_math)
        .def_readwrite("gpu_threshold", &mccl::MCCLOptions::gpu_threshold)
        .def_readwrite("overlap_comm", &mccl::MCCLOptions::overlap_comm)
        .def_readwrite("max_queue_depth", &mccl::MCCLOptions::max_queue_depth)
        .def_readwrite("compression", &mccl::MCCLOptions::compression)
        .def_readwrite("topk_ratio", &mccl::MCCLOptions::topk_ratio)
        .def_readwrite("watchdog_timeout", &mccl::MCCLOptions::watchdog_timeout)
        .def_readwrite("heartbeat_interval", &mccl::MCCLOptions::heartbeat_interval);

    // ---- kernel helpers: same names as the reference's test bindings ----------
    m.def("_metal_accumulate_chunk", [](at::Tensor dst, const at::Tensor& src) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_accumulate_chunk(dst, src);
        mccl::metal_sync();
        return dst;
    }, "dst += src via the HIP kernel; returns dst");
    m.def("_metal_elementwise_min", [](at::Tensor dst, const at::Tensor& src) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_elementwise_min(dst, src);
        mccl::metal_sync();
        return dst;
    }, "dst = min(dst, src); returns dst");
    m.def("_metal_elementwise_max", [](at::Tensor dst, const at::Tensor& src) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_elementwise_max(dst, src);
        mccl::metal_sync();
        return dst;
    }, "dst = max(dst, src); returns dst");
    m.def("_metal_elementwise_product", [](at::Tensor dst, const at::Tensor& src) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_elementwise_product(dst, src);
        mccl::metal_sync();
        return dst;
    }, "dst *= src; returns dst");
    m.def("_metal_scale_inplace", [](at::Tensor buf, double scale) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_scale_inplace(buf, scale);
        mccl::metal_sync();
        return buf;
    }, "buf *= scale; returns buf");
    m.def("_metal_accumulate_and_scale", [](at::Tensor dst, const at::Tensor& src, double scale) {
        mccl::metal_kernels_init(); producer_sync();
        mccl::metal_accumulate_and_scale(dst, src, scale);
        mccl::metal_sync();
        return dst;
    }, "dst = (dst + src) * scale; returns dst");

    // ---- the C++ entry points the process group calls, asynchronous ---------
    m.def("_metal_reduce_op", [](at::Tensor dst, const at::Tensor& src, int op) {
        mccl::metal_kernels_init();
        mccl::metal_reduce_op(dst, src, static_cast<c10d::ReduceOp::RedOpType>(op));
        return dst;
    });
    m.def("_hip_reduce_op_batch", [](const std::vector<at::Tensor>& dsts, const std::vector<at::Tensor>& srcs, int op) {
        mccl::metal_kernels_init();
        mccl::hip_reduce_op_batch(dsts, srcs, static_cast<c10d::ReduceOp::RedOpType>(op));
    }, "dsts[i] (op)= srcs[i] for independent pairs, one launch per 128 pairs");
    m.def("_metal_reduce_op_fenced", [](at::Tensor dst, const at::Tensor& src, int op) {
        mccl::metal_kernels_init();
        return mccl::metal_reduce_op_fenced(dst, src, static_cast<c10d::ReduceOp::RedOpType>(op));
    });
    m.def("_wait_for_mccl_fence", &mccl::wait_for_mccl_fence);
    m.def("_event_sync_available", [] { mccl::event_sync_init(); return mccl::event_sync_available(); });
    m.def("_metal_sync", &mccl::metal_sync);
    m.def("_hip_ring_fold", [](at::Tensor out, const std::vector<at::Tensor>& ins, int op, bool chunked,
                               int64_t bucket_elems, bool stepwise) {
        mccl::metal_kernels_init();
        mccl::hip_ring_fold(out, ins, static_cast<c10d::ReduceOp::RedOpType>(op), chunked, bucket_elems, stepwise);
        return out;
    }, py::arg("out"), py::arg("ins"), py::arg("op"), py::arg("chunked") = false,
       py::arg("bucket_elems") = 0, py::arg("stepwise") = false);
    // ---- raw-pointer family (csrc/metal/AccelerateOps.hpp:18-59) on tensors' data pointers.
    // Tensors may live on the GPU or in pinned host memory; the functions themselves
    // refuse memory a kernel cannot reach.  The *_ptr forms take plain addresses.
    m.def("_cpu_reduce_op", [](at::Tensor dst, const at::Tensor& src, int op) {
        raw_check(dst, &src);
        const auto rop = static_cast<c10d::ReduceOp::RedOpType>(op);
        const int64_t n = dst.numel();
        switch (dst.scalar_type()) {
            case at::kFloat: mccl::cpu_reduce_op(dst.data_ptr<float>(), src.data_ptr<float>(), n, rop); break;
            case at::kHalf: mccl::cpu_reduce_op_half(dst.data_ptr<c10::Half>(), src.data_ptr<c10::Half>(), n, rop); break;
            case at::kBFloat16:
                mccl::cpu_reduce_op_bf16(dst.data_ptr<c10::BFloat16>(), src.data_ptr<c10::BFloat16>(), n, rop);
                break;
            default: mccl::cpu_reduce_op_integral(dst.data_ptr(), src.data_ptr(), n, dst.scalar_type(), rop);
        }
        return dst;
    });
    m.def("_cpu_scale_inplace", [](at::Tensor buf, double scale) {
        raw_check(buf, nullptr);
        const int64_t n = buf.numel();
        const float s = static_cast<float>(scale);
        switch (buf.scalar_type()) {
            case at::kFloat: mccl::cpu_scale_inplace(buf.data_ptr<float>(), n, s); break;
            case at::kHalf: mccl::cpu_scale_inplace_half(buf.data_ptr<c10::Half>(), n, s); break;
            case at::kBFloat16: mccl::cpu_scale_inplace_bf16(buf.data_ptr<c10::BFloat16>(), n, s); break;
            default: mccl::cpu_scale_inplace_integral(buf.data_ptr(), n, buf.scalar_type(), s);
        }
        return buf;
    });
    m.def("_cpu_accumulate_and_scale", [](at::Tensor dst, const at::Tensor& src, double scale) {
        raw_check(dst, &src);
        const int64_t n = dst.numel();
        const float s = static_cast<float>(scale);
        switch (dst.scalar_type()) {
            case at::kFloat: mccl::cpu_accumulate_and_scale(dst.data_ptr<float>(), src.data_ptr<float>(), n, s); break;
            case at::kHalf:
                mccl::cpu_accumulate_and_scale_half(dst.data_ptr<c10::Half>(), src.data_ptr<c10::Half>(), n, s);
                break;
            case at::kBFloat16:
                mccl::cpu_accumulate_and_scale_bf16(dst.data_ptr<c10::BFloat16>(), src.data_ptr<c10::BFloat16>(), n, s);
                break;
            default: throw mccl::MCCLError("cpu_accumulate_and_scale: float32/float16/bfloat16 only");
        }
        return dst;
    });
    m.def("_cpu_accumulate", [](at::Tensor dst, const at::Tensor& src) {
        raw_check(dst, &src, at::kFloat);
        mccl::cpu_accumulate(dst.data_ptr<float>(), src.data_ptr<float>(), dst.numel());
        return dst;
    });
    m.def("_cpu_elementwise_min", [](at::Tensor dst, const at::Tensor& src) {
        raw_check(dst, &src, at::kFloat);
        mccl::cpu_elementwise_min(dst.data_ptr<float>(), src.data_ptr<float>(), dst.numel());
        return dst;
    });
    m.def("_cpu_elementwise_max", [](at::Tensor dst, const at::Tensor& src) {
        raw_check(dst, &src, at::kFloat);
        mccl::cpu_elementwise_max(dst.data_ptr<float>(), src.data_ptr<float>(), dst.numel());
        return dst;
    });
    m.def("_cpu_elementwise_product", [](at::Tensor dst, const at::Tensor& src) {
        raw_check(dst, &src, at::kFloat);
        mccl::cpu_elementwise_product(dst.data_ptr<float>(), src.data_ptr<float>(), dst.numel());
        return dst;
    });
    m.def("_cpu_reduce_op_ptr", [](uint64_t dst, uint64_t src, int64_t count, int op) {
        mccl::cpu_reduce_op(reinterpret_cast<float*>(dst), reinterpret_cast<const float*>(src), count,
                            static_cast<c10d::ReduceOp::RedOpType>(op));
    }, "cpu_reduce_op on two raw addresses of `count` floats");

    // ---- compressor -------------------------------------------------------------
    py::class_<mccl::Compressor>(m, "Compressor");
    py::class_<mccl::TopKCompressor, mccl::Compressor>(m, "TopKCompressor")
        .def(py::init<double>(), py::arg("k_ratio"))
        .def("name", &mccl::TopKCompressor::name)
        .def("max_compressed_size", &mccl::TopKCompressor::max_compressed_size)
        .def("compress", [](mccl::TopKCompressor& c, const at::Tensor& t, py::object stable_id, py::object capacity) {
            mccl::check_single_tensor(t);
            const size_t nbytes = mccl::tensor_nbytes(t);
            const size_t cap = capacity.is_none() ? c.max_compressed_size(nbytes) : capacity.cast<size_t>();
            at::Tensor out = at::empty({static_cast<int64_t>(cap)},
                                       at::TensorOptions().dtype(at::kByte).device(t.device()));
            const uint64_t id = stable_id.is_none() ? stable_id_of(t) : stable_id.cast<uint64_t>();
            const size_t used = c.compress(t.data_ptr(), nbytes, out.data_ptr(), cap, t.scalar_type(), id);
            return out.narrow(0, 0, static_cast<int64_t>(used));
        }, py::arg("tensor"), py::arg("stable_id") = py::none(), py::arg("capacity") = py::none(),
           "Top-k payload of a gradient bucket as a uint8 device tensor; error feedback is kept per stable_id")
        .def("decompress", [](mccl::TopKCompressor& c, const at::Tensor& wire, int64_t numel, py::object size) {
            check_payload(wire, size, numel);
            at::Tensor out = at::empty({numel}, at::TensorOptions().dtype(at::kFloat).device(wire.device()));
            const size_t sz = size.is_none() ? static_cast<size_t>(wire.numel()) : size.cast<size_t>();
            c.decompress(wire.data_ptr(), sz, out.data_ptr(), static_cast<size_t>(numel) * 4, at::kFloat);
            return out;
        }, py::arg("wire"), py::arg("numel"), py::arg("compressed_size") = py::none())
        .def("compress_many", [](mccl::TopKCompressor& c, const std::vector<at::Tensor>& buckets, py::object stable_ids) {
            std::vector<uint64_t> ids;
            if (stable_ids.is_none()) for (const auto& t : buckets) ids.push_back(stable_id_of(t));
            else ids = stable_ids.cast<std::vector<uint64_t>>();
            return c.compress_many(buckets, ids);
        }, py::arg("buckets"), py::arg("stable_ids") = py::none(),
           "Top-k payloads of a list of gradient buckets, one uint8 device tensor each")
        .def("reset_error_feedback", &mccl::TopKCompressor::reset_error_feedback)
        .def("reset_error_feedback_for_tensor", &mccl::TopKCompressor::reset_error_feedback_for_tensor)
        .def("check_compress_status", &mccl::TopKCompressor::check_compress_status)
        .def("error_feedback_buffer_count", &mccl::TopKCompressor::error_feedback_buffer_count)
        .def("error_feedback_buffer", [](mccl::TopKCompressor& c, uint64_t id) -> py::object {
            at::Tensor t = c.error_feedback_buffer(id);
            if (!t.defined()) return py::none();
            return py::cast(t);
        });
    py::class_<mccl::FP16Compressor, mccl::Compressor>(m, "FP16Compressor")
        .def(py::init<>())
        .def("name", &mccl::FP16Compressor::name)
        .def("max_compressed_size", &mccl::FP16Compressor::max_compressed_size)
        .def("compress", [](mccl::FP16Compressor& c, const at::Tensor& t, py::object capacity) {
            mccl::check_single_tensor(t);
            const size_t nbytes = mccl::tensor_nbytes(t);
            const size_t cap = capacity.is_none() ? c.max_compressed_size(nbytes) : capacity.cast<size_t>();
            at::Tensor out = at::empty({static_cast<int64_t>(cap)},
                                       at::TensorOptions().dtype(at::kByte).device(t.device()));
            const size_t used = c.compress(t.data_ptr(), nbytes, out.data_ptr(), cap, t.scalar_type());
            return out.narrow(0, 0, static_cast<int64_t>(used));
        }, py::arg("tensor"), py::arg("capacity") = py::none(),
           "Half-precision payload of a float32 bucket (a float16 bucket is copied) as a uint8 device tensor")
        .def("decompress", [](mccl::FP16Compressor& c, const at::Tensor& wire, int64_t numel, py::object size,
                              at::ScalarType dtype) {
            check_payload(wire, size, numel);
            at::Tensor out = at::empty({numel}, at::TensorOptions().dtype(dtype).device(wire.device()));
            const size_t sz = size.is_none() ? static_cast<size_t>(wire.numel()) : size.cast<size_t>();
            c.decompress(wire.data_ptr(), sz, out.data_ptr(), static_cast<size_t>(numel) * out.element_size(), dtype);
            return out;
        }, py::arg("wire"), py::arg("numel"), py::arg("compressed_size") = py::none(),
           py::arg("dtype") = at::kFloat);
    m.def("make_compressor", [](mccl::CompressionMode mode, double param) -> py::object {
        auto c = mccl::make_compressor(mode, param);
        if (!c) return py::none();
        if (auto* half = dynamic_cast<mccl::FP16Compressor*>(c.get())) {
            c.release();
            return py::cast(half, py::return_value_policy::take_ownership);
        }
        auto* topk = dynamic_cast<mccl::TopKCompressor*>(c.get());
        MCCL_CHECK(topk != nullptr, "unexpected compressor type");
        c.release();
        return py::cast(topk, py::return_value_policy::take_ownership);
    }, py::arg("mode"), py::arg("param") = 0.0);
    m.def("_compression_stable_id", &stable_id_of);

    // ---- ring plan, payload framing, W ranks on one GPU ------------------------
    m.def("_ring_plan", [](int rank, int ws, bool chunked) {
        py::list out;
        for (const auto& st : mccl::ring_plan(rank, ws, chunked ? mccl::RingAlgo::CHUNKED : mccl::RingAlgo::BASIC))
            out.append(py::make_tuple(st.send_idx, st.recv_idx, st.send_tid, st.recv_tid,
                                      st.kind == mccl::RingRecvKind::REDUCE ? "reduce" : "copy"));
        return out;
    }, py::arg("rank"), py::arg("world_size"), py::arg("chunked") = true,
       "(send_idx, recv_idx, send_tid, recv_tid, kind) per step: reduce-scatter, then all-gather");
    m.def("_ring_chunk_views", [](const at::Tensor& t, int ws, bool chunked) {
        return mccl::ring_chunk_views(t, ws, chunked ? mccl::RingAlgo::CHUNKED : mccl::RingAlgo::BASIC);
    }, py::arg("tensor"), py::arg("world_size"), py::arg("chunked") = true);
    m.def("_ring_algo_from_env", [] { return mccl::ring_algo_from_env() == mccl::RingAlgo::CHUNKED ? "chunked" : "basic"; });
    m.def("_compressed_pack", [](mccl::Compressor& c, const at::Tensor& t) {
        mccl::CompressedFrame f = mccl::compressed_pack(&c, t);
        return py::make_tuple(f.wire_size, f.payload);
    }, py::arg("compressor"), py::arg("tensor"), "(size header, payload of exactly that many bytes)");
    m.def("_compressed_unpack", [](mccl::Compressor& c, uint32_t wire_size, const at::Tensor& payload, at::Tensor out) {
        mccl::CompressedFrame f;
        f.wire_size = wire_size;
        f.payload = payload;
        mccl::compressed_unpack(&c, f, out);
        return out;
    }, py::arg("compressor"), py::arg("wire_size"), py::arg("payload"), py::arg("out"));

    py::class_<mccl::LoopbackGroup>(m, "LoopbackGroup")
        .def(py::init([](int ws, py::object opts, bool rank_streams) {
            if (opts.is_none()) return std::make_unique<mccl::LoopbackGroup>(ws, mccl::MCCLOptions(), rank_streams);
            return std::make_unique<mccl::LoopbackGroup>(ws, *opts.cast<c10::intrusive_ptr<mccl::MCCLOptions>>(),
                                                         rank_streams);
        }), py::arg("world_size"), py::arg("options") = py::none(), py::arg("rank_streams") = true)
        .def("size", &mccl::LoopbackGroup::size)
        .def("compressor", [](mccl::LoopbackGroup& g, int rank) -> mccl::Compressor* {
            MCCL_CHECK(rank >= 0 && rank < g.size(), "rank out of range");
            return g.compressor(rank);
        }, py::return_value_policy::reference_internal)
        .def("allreduce", [](mccl::LoopbackGroup& g, std::vector<at::Tensor> t, int op) {
            g.allreduce(t, static_cast<c10d::ReduceOp::RedOpType>(op));
        }, py::arg("rank_tensors"), py::arg("op") = 0)
        .def("allreduce_coalesced", [](mccl::LoopbackGroup& g, std::vector<std::vector<at::Tensor>> lists, int op) {
            g.allreduce_coalesced(lists, static_cast<c10d::ReduceOp::RedOpType>(op));
        }, py::arg("rank_lists"), py::arg("op") = 0)
        .def("reduce_scatter", [](mccl::LoopbackGroup& g, std::vector<at::Tensor> outputs,
                                  std::vector<std::vector<at::Tensor>> inputs, int op) {
            g.reduce_scatter(outputs, inputs, static_cast<c10d::ReduceOp::RedOpType>(op));
        }, py::arg("outputs"), py::arg("inputs"), py::arg("op") = 0)
        .def("allreduce_ring", [](mccl::LoopbackGroup& g, std::vector<at::Tensor> t, int op, bool chunked) {
            g.allreduce_ring(t, static_cast<c10d::ReduceOp::RedOpType>(op),
                             chunked ? mccl::RingAlgo::CHUNKED : mccl::RingAlgo::BASIC);
        }, py::arg("rank_tensors"), py::arg("op") = 0, py::arg("chunked") = true)
        .def("allreduce_two_rank", [](mccl::LoopbackGroup& g, std::vector<at::Tensor> t, int op) {
            g.allreduce_two_rank(t, static_cast<c10d::ReduceOp::RedOpType>(op));
        }, py::arg("rank_tensors"), py::arg("op") = 0)
        .def("allreduce_small", [](mccl::LoopbackGroup& g, std::vector<at::Tensor> t, int op) {
            g.allreduce_small(t, static_cast<c10d::ReduceOp::RedOpType>(op));
        }, py::arg("rank_tensors"), py::arg("op") = 0)
        .def("stats", [](const mccl::LoopbackGroup& g) {
            const auto& s = g.stats();
            py::dict d;
            d["collectives"] = s.collectives;
            d["reduce_launches"] = s.reduce_launches;
            d["copy_launches"] = s.copy_launches;
            d["fences_signalled"] = s.fences_signalled;
            d["stream_waits"] = s.stream_waits;
            d["wire_bytes"] = s.wire_bytes;
            d["last_algo"] = s.last_algo;
            return d;
        });
}
