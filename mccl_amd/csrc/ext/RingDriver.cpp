#include "RingDriver.hpp"

#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstdlib>

#include "../../../include/mccl_hip.h"
#include "Errors.hpp"
#include "HipKernels.hpp"
#include "Logging.hpp"
#include "TensorChecks.hpp"

namespace mccl {

// ---- plan --------------------------------------------------------------------

RingAlgo ring_algo_from_env() {
    const char* v = std::getenv("MCCL_RING_ALGO");
    if (!v) return RingAlgo::CHUNKED;
    const std::string s(v);
    return (s == "basic" || s == "ring" || s == "plain") ? RingAlgo::BASIC : RingAlgo::CHUNKED;
}

int ring_chunk_count(int ws, RingAlgo algo) { return algo == RingAlgo::CHUNKED ? 2 * ws : ws; }

// Both schedules are one formula in the number of chunks a rank owns, c (1 or
// 2), over m = c * ws chunk slots.  Reduce-scatter step s sends slot c*rank - s
// and folds into slot c*rank - s - c; all-gather step s sends c*rank + c - s and
// overwrites c*rank - s (all mod m).  With c = 2 these are the reference's
// (2r - step) / (2r - step - 2) and (2r + 2 - step) / (2r - step); with c = 1
// its (r - step) / (r - step - 1) and (r - step + 1) / (r - step).  A tag is the
// global step in the high half and the chunk slot in the low half.
std::vector<RingStep> ring_plan(int rank, int ws, RingAlgo algo) {
    MCCL_CHECK(ws >= 1 && rank >= 0 && rank < ws, "ring_plan: rank out of range");
    const int c = algo == RingAlgo::CHUNKED ? 2 : 1;
    const int m = c * ws;
    const int phase_steps = c * (ws - 1);
    auto slot = [m](int v) { return ((v % m) + m) % m; };
    std::vector<RingStep> plan;
    plan.reserve(2 * static_cast<size_t>(phase_steps));
    for (int g = 0; g < 2 * phase_steps; g++) {
        const bool gather = g >= phase_steps;
        const int s = gather ? g - phase_steps : g;
        RingStep st;
        st.send_idx = slot(c * rank - s + (gather ? c : 0));
        st.recv_idx = slot(c * rank - s - (gather ? 0 : c));
        st.send_tid = (static_cast<uint32_t>(g) << 16) | static_cast<uint32_t>(st.send_idx);
        st.recv_tid = (static_cast<uint32_t>(g) << 16) | static_cast<uint32_t>(st.recv_idx);
        st.kind = gather ? RingRecvKind::COPY : RingRecvKind::REDUCE;
        plan.push_back(st);
    }
    return plan;
}

std::vector<at::Tensor> ring_chunk_views(const at::Tensor& tensor, int ws, RingAlgo algo) {
    MCCL_CHECK_TENSOR(tensor.is_contiguous(),
                      "MCCL v1 requires contiguous tensors. Call .contiguous() before passing to collective.");
    const int m = ring_chunk_count(ws, algo);
    const int64_t total = tensor.numel();
    const int64_t per = (total + m - 1) / m;
    at::Tensor flat = tensor.view({total});
    std::vector<at::Tensor> out;
    out.reserve(m);
    for (int i = 0; i < m; i++) {
        const int64_t start = std::min<int64_t>(static_cast<int64_t>(i) * per, total);
        out.push_back(flat.narrow(0, start, std::min(per, total - start)));
    }
    return out;
}

// ---- framing -------------------------------------------------------------------

namespace {
const char* kNoBf16 =
    "BFloat16 tensors are not supported with compression enabled. "
    "Disable compression (MCCL_COMPRESSION=none) or use float32/float16.";
}

uint64_t compression_stable_id(const at::Tensor& tensor) {
    return reinterpret_cast<uint64_t>(tensor.storage().data()) +
           static_cast<uint64_t>(tensor.storage_offset()) * tensor.element_size();
}

CompressedFrame compressed_pack(Compressor* compressor, const at::Tensor& tensor) {
    MCCL_CHECK(compressor != nullptr, "compressed_pack needs a compressor");
    MCCL_CHECK(tensor.scalar_type() != at::kBFloat16, kNoBf16);
    check_single_tensor(tensor);
    const size_t nbytes = tensor_nbytes(tensor);
    const size_t max_comp = compressor->max_compressed_size(nbytes);
    at::Tensor buf = at::empty({static_cast<int64_t>(max_comp)},
                               at::TensorOptions().dtype(at::kByte).device(tensor.device()));
    const size_t used = compressor->compress(tensor.data_ptr(), nbytes, buf.data_ptr(), max_comp,
                                             tensor.scalar_type(), compression_stable_id(tensor));
    CompressedFrame f;
    f.wire_size = static_cast<uint32_t>(used);
    f.payload = buf.narrow(0, 0, static_cast<int64_t>(used));
    return f;
}

void compressed_unpack(Compressor* compressor, const CompressedFrame& frame, const at::Tensor& out) {
    MCCL_CHECK(compressor != nullptr, "compressed_unpack needs a compressor");
    MCCL_CHECK(out.scalar_type() != at::kBFloat16, kNoBf16);
    check_single_tensor(out);
    const size_t nbytes = tensor_nbytes(out);
    const size_t max_comp = compressor->max_compressed_size(nbytes);
    MCCL_CHECK(frame.wire_size > 0 && frame.wire_size <= max_comp,
               "Compressed payload size " + std::to_string(frame.wire_size) + " out of range (max " +
                   std::to_string(max_comp) + ")");
    MCCL_CHECK_TENSOR(frame.payload.defined() && frame.payload.is_cuda() &&
                          frame.payload.get_device() == out.get_device(),
                      "compressed payload must live on the output tensor's GPU");
    MCCL_CHECK(frame.payload.defined() && frame.payload.scalar_type() == at::kByte && frame.payload.is_contiguous() &&
                   static_cast<uint64_t>(frame.payload.numel()) == frame.wire_size,
               "compressed_recv recv_chunks failed");
    compressor->decompress(frame.payload.data_ptr(), frame.wire_size, out.data_ptr(), nbytes, out.scalar_type());
}

// ---- the group -----------------------------------------------------------------

namespace {

struct StreamScope {
    c10::hip::HIPStream prev;
    explicit StreamScope(c10::hip::HIPStream s) : prev(c10::hip::getCurrentHIPStream(s.device_index())) {
        c10::hip::setCurrentHIPStream(s);
    }
    ~StreamScope() { c10::hip::setCurrentHIPStream(prev); }
    StreamScope(const StreamScope&) = delete;
    StreamScope& operator=(const StreamScope&) = delete;
};

// The fence ring of the kernel library holds 1024 events; a collective that
// would have more than this many tickets alive runs on one stream instead.
constexpr size_t kMaxTickets = 512;

}  // namespace

LoopbackGroup::LoopbackGroup(int world_size, const MCCLOptions& opts, bool rank_streams)
    : ws_(world_size), rank_streams_(rank_streams), small_msg_threshold_(opts.small_msg_threshold) {
    MCCL_CHECK(world_size >= 1 && world_size <= 1024, "world size must be in [1, 1024]");
    compressors_.reserve(world_size);
    for (int r = 0; r < world_size; r++) compressors_.push_back(make_compressor(opts.compression, opts.topk_ratio));
    if (compressors_[0]) MCCL_INFO("Compression enabled: %s", compressors_[0]->name().c_str());
}

void LoopbackGroup::check_ranks(const std::vector<at::Tensor>& t) const {
    MCCL_CHECK_TENSOR(static_cast<int>(t.size()) == ws_, "one tensor per rank expected, got " +
                                                             std::to_string(t.size()) + " for world size " +
                                                             std::to_string(ws_));
    for (const auto& x : t) {
        check_single_tensor(x);
        check_same_shape_dtype(t[0], x);
        MCCL_CHECK_TENSOR(x.get_device() == t[0].get_device(), "all ranks of a loopback group share one device");
    }
    MCCL_CHECK_TENSOR(t[0].get_device() == c10::hip::current_device(), "tensors must be on the current device");
    for (size_t a = 0; a < t.size(); a++)
        for (size_t b = a + 1; b < t.size(); b++)
            MCCL_CHECK_TENSOR(t[a].numel() == 0 || t[a].data_ptr() != t[b].data_ptr(),
                              "each rank needs a buffer of its own");
}

void LoopbackGroup::allreduce(std::vector<at::Tensor>& t, c10d::ReduceOp::RedOpType op) {
    check_ranks(t);
    if (t[0].numel() == 0 || ws_ == 1) return;
    if (ws_ == 2) return allreduce_two_rank(t, op);
    if (tensor_nbytes(t[0]) <= small_msg_threshold_) return allreduce_small(t, op);
    allreduce_ring(t, op, ring_algo_from_env());
}

void LoopbackGroup::allreduce_coalesced(std::vector<std::vector<at::Tensor>>& lists, c10d::ReduceOp::RedOpType op) {
    MCCL_CHECK_TENSOR(static_cast<int>(lists.size()) == ws_, "one tensor list per rank expected");
    std::vector<at::Tensor> flats;
    flats.reserve(ws_);
    for (auto& list : lists) {
        MCCL_CHECK_TENSOR(!list.empty(), "allreduce_coalesced: empty tensor list");
        MCCL_CHECK_TENSOR(list.size() == lists[0].size(), "allreduce_coalesced: ranks disagree on the tensor count");
        std::vector<at::Tensor> parts;
        for (auto& x : list) {
            check_single_tensor(x);
            if (x.numel() != 0) parts.push_back(x.flatten());
        }
        if (parts.empty()) return;
        flats.push_back(at::cat(parts, 0));
    }
    if (ws_ == 1) return;
    allreduce(flats, op);
    for (int r = 0; r < ws_; r++) {
        int64_t offset = 0;
        for (auto& x : lists[r]) {
            at::Tensor piece = flats[r].narrow(0, offset, x.numel());
            x.view_as(piece).copy_(piece);
            offset += x.numel();
        }
    }
}

void LoopbackGroup::reduce_scatter(std::vector<at::Tensor>& outputs, std::vector<std::vector<at::Tensor>>& inputs,
                                   c10d::ReduceOp::RedOpType op) {
    MCCL_CHECK_TENSOR(static_cast<int>(outputs.size()) == ws_ && static_cast<int>(inputs.size()) == ws_,
                      "one output and one input list per rank expected");
    for (int r = 0; r < ws_; r++) {
        MCCL_CHECK_TENSOR(static_cast<int>(inputs[r].size()) == ws_, "Input tensor list size must equal world_size");
        check_single_tensor(outputs[r]);
        for (auto& x : inputs[r]) {
            MCCL_CHECK_TENSOR(x.is_contiguous(), "MCCL v1 requires contiguous tensors. Call .contiguous() before passing to collective.");
            check_single_tensor(x);
            check_same_shape_dtype(outputs[r], x);
        }
        check_same_shape_dtype(outputs[0], outputs[r]);
    }
    if (outputs[0].numel() == 0) return;
    metal_kernels_init();
    if (ws_ == 1) {
        outputs[0].copy_(inputs[0][0]);
    } else if (ws_ == 2) {
        // step 0 of the ring: rank r sends chunk (r + 1) % 2 and folds the incoming
        // partial into its own chunk r; both folds read the peer's untouched chunk
        for (int r = 0; r < 2; r++) {
            metal_reduce_op_fenced(inputs[r][r], inputs[1 - r][r], op);
            stats_.reduce_launches++;
            stats_.fences_signalled++;
            stats_.wire_bytes += tensor_nbytes(outputs[r]);
        }
        for (int r = 0; r < 2; r++) outputs[r].copy_(inputs[r][r]);
        stats_.copy_launches += 2;
    } else {
        for (int d = 0; d < ws_; d++) {
            outputs[d].copy_(inputs[d][d]);
            stats_.copy_launches++;
            for (int src = 0; src < ws_; src++) {
                if (src == d) continue;
                metal_reduce_op(outputs[d], inputs[src][d], op);
                stats_.reduce_launches++;
                stats_.wire_bytes += tensor_nbytes(outputs[d]);
            }
        }
    }
    stats_.collectives++;
    stats_.last_algo = ws_ >= 3 ? "reduce_scatter_star" : "reduce_scatter_ring";
}

// What `from_rank`'s tensor looks like on the far side of the link: compressed
// with the sender's state and expanded again, or the bytes themselves.
at::Tensor LoopbackGroup::through_wire(int from_rank, const at::Tensor& tensor) {
    Compressor* c = compressors_[from_rank].get();
    if (!c) {
        stats_.wire_bytes += tensor_nbytes(tensor);
        stats_.copy_launches++;
        return tensor.clone();
    }
    CompressedFrame f = compressed_pack(c, tensor);
    at::Tensor out = at::empty_like(tensor);
    compressed_unpack(c, f, out);
    stats_.wire_bytes += sizeof(uint32_t) + f.wire_size;
    return out;
}

// csrc/backend/ProcessGroupMCCL.cpp:1632-1709: both ranks fold the other's
// tensor into their own; AVG is the fused (local + incoming) * 0.5.
void LoopbackGroup::allreduce_two_rank(std::vector<at::Tensor>& t, c10d::ReduceOp::RedOpType op) {
    check_ranks(t);
    MCCL_CHECK(ws_ == 2, "allreduce_two_rank needs a world size of 2");
    if (t[0].numel() == 0) return;
    metal_kernels_init();
    at::Tensor at0 = through_wire(1, t[1]);
    at::Tensor at1 = through_wire(0, t[0]);
    const at::Tensor* incoming[2] = {&at0, &at1};
    for (int r = 0; r < 2; r++) {
        if (op == c10d::ReduceOp::AVG) {
            metal_accumulate_and_scale(t[r], *incoming[r], 0.5);
        } else {
            metal_reduce_op_fenced(t[r], *incoming[r], op);
            stats_.fences_signalled++;
        }
        stats_.reduce_launches++;
    }
    stats_.collectives++;
    stats_.last_algo = "two_rank";
}

// csrc/backend/ProcessGroupMCCL.cpp:2257-2313: rank 0 folds the peers' tensors
// into its own in rank order, scales for AVG, and sends the result to every
// peer -- through the compressor again when one is set, once per peer.
void LoopbackGroup::allreduce_small(std::vector<at::Tensor>& t, c10d::ReduceOp::RedOpType op) {
    check_ranks(t);
    if (t[0].numel() == 0 || ws_ == 1) return;
    metal_kernels_init();
    for (int peer = 1; peer < ws_; peer++) {
        at::Tensor incoming = through_wire(peer, t[peer]);
        metal_reduce_op_fenced(t[0], incoming, op);
        stats_.reduce_launches++;
        stats_.fences_signalled++;
    }
    if (op == c10d::ReduceOp::AVG) metal_scale_inplace(t[0], 1.0 / ws_);
    for (int peer = 1; peer < ws_; peer++) {
        at::Tensor result = through_wire(0, t[0]);
        t[peer].copy_(result);
        stats_.copy_launches++;
    }
    stats_.collectives++;
    stats_.last_algo = "small";
}

// The ring proper.  At step s rank q folds (or copies) its left neighbour's
// chunk plan[left][s].send_idx into its own chunk of the same slot.  Rank q's
// work is enqueued on stream q; before each operation that stream is made to
// wait for the last write of the chunk it reads and for the last read of the
// chunk it overwrites, and afterwards one fence covers both new facts.
void LoopbackGroup::allreduce_ring(std::vector<at::Tensor>& t, c10d::ReduceOp::RedOpType op, RingAlgo algo) {
    check_ranks(t);
    const int ws = ws_;
    if (t[0].numel() == 0 || ws == 1) return;
    metal_kernels_init();
    const int m = ring_chunk_count(ws, algo);
    std::vector<std::vector<RingStep>> plan(ws);
    std::vector<std::vector<at::Tensor>> chunk(ws);
    for (int r = 0; r < ws; r++) {
        plan[r] = ring_plan(r, ws, algo);
        chunk[r] = ring_chunk_views(t[r], ws, algo);
    }
    const size_t nsteps = plan[0].size();
    const auto dev = static_cast<c10::DeviceIndex>(t[0].get_device());
    const c10::hip::HIPStream caller = c10::hip::getCurrentHIPStream(dev);
    const bool fan_out = rank_streams_ && static_cast<size_t>(ws) * (nsteps + 3) <= kMaxTickets;
    std::vector<c10::hip::HIPStream> stream(ws, caller);
    if (fan_out)
        for (int r = 0; r < ws; r++) stream[r] = c10::hip::getStreamFromPool(false, dev);

    auto signal = [&](const c10::hip::HIPStream& s) {
        uint64_t ticket = 0;
        throw_on_status(mccl_hip_fence_signal(s.stream(), &ticket), "ring fence signal");
        stats_.fences_signalled++;
        return ticket;
    };
    auto wait = [&](const c10::hip::HIPStream& s, uint64_t ticket) {
        if (!ticket) return;
        throw_on_status(mccl_hip_fence_block_stream(ticket, s.stream()), "ring fence wait");
        stats_.stream_waits++;
    };

    if (fan_out) {
        const uint64_t start = signal(caller);
        for (int r = 0; r < ws; r++) wait(stream[r], start);
    }
    std::vector<std::vector<uint64_t>> wrote(ws, std::vector<uint64_t>(m, 0));
    std::vector<std::vector<uint64_t>> read(ws, std::vector<uint64_t>(m, 0));

    for (size_t s = 0; s < nsteps; s++) {
        for (int q = 0; q < ws; q++) {
            const int p = (q + ws - 1) % ws;
            const RingStep& st = plan[q][s];
            MCCL_CHECK(plan[p][s].send_idx == st.recv_idx && plan[p][s].send_tid == st.recv_tid,
                       "ring plan mismatch between neighbours at step " + std::to_string(s));
            const at::Tensor& dst = chunk[q][st.recv_idx];
            const at::Tensor& src = chunk[p][st.recv_idx];
            if (dst.numel() == 0) continue;
            if (fan_out) {
                wait(stream[q], wrote[p][st.recv_idx]);
                wait(stream[q], read[q][st.recv_idx]);
            }
            {
                StreamScope scope(stream[q]);
                if (st.kind == RingRecvKind::REDUCE) {
                    metal_reduce_op(dst, src, op);
                    stats_.reduce_launches++;
                } else {
                    const hipError_t e = hipMemcpyAsync(dst.data_ptr(), src.data_ptr(), tensor_nbytes(dst),
                                                        hipMemcpyDeviceToDevice, stream[q].stream());
                    MCCL_CHECK(e == hipSuccess, std::string("ring all-gather copy failed: ") + hipGetErrorString(e));
                    stats_.copy_launches++;
                }
            }
            stats_.wire_bytes += tensor_nbytes(dst);
            if (fan_out) {
                const uint64_t ticket = signal(stream[q]);
                wrote[q][st.recv_idx] = ticket;
                read[p][st.recv_idx] = ticket;
            }
        }
    }

    // AVG tail: the whole tensor is scaled in place (csrc/backend/ProcessGroupMCCL.cpp:1954-1956),
    // which must not start before the right neighbour has read its last chunk.
    std::vector<uint64_t> gathered(ws, 0), done(ws, 0);
    if (fan_out)
        for (int r = 0; r < ws; r++) done[r] = gathered[r] = signal(stream[r]);
    if (op == c10d::ReduceOp::AVG) {
        for (int r = 0; r < ws; r++) {
            if (fan_out) wait(stream[r], gathered[(r + 1) % ws]);
            StreamScope scope(stream[r]);
            metal_scale_inplace(t[r], 1.0 / ws);
            if (fan_out) done[r] = signal(stream[r]);
        }
    }
    if (fan_out)
        for (int r = 0; r < ws; r++) wait(caller, done[r]);
    stats_.collectives++;
    stats_.last_algo = algo == RingAlgo::CHUNKED ? "ring_chunked" : "ring";
}

}  // namespace mccl
