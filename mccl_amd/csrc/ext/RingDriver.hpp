// Host side of the ring collectives for ranks that live on one GPU.
//
// The reference runs one process per machine and moves chunks over TCP/RDMA
// between ring steps (csrc/backend/ProcessGroupMCCL.cpp:1711-2179).  Here the
// ranks are W tensors in one GPU's HBM: a "send" is the right neighbour reading
// the sender's chunk, so what is left of the collective is its compute half --
// the step plan, the per-chunk folds and copies in the reference's order, and
// the ordering between them.  Each rank's work is enqueued on a HIP stream of
// its own; a fold waits (on the device, never on the host) only for the fences
// of the chunks it touches, which is the role of the reference's per-chunk
// kernel fences (:1752-1772,:2014-2034).
#pragma once

#include <torch/torch.h>
#include <torch/csrc/distributed/c10d/Types.hpp>

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "Compression.hpp"
#include "Options.hpp"

namespace mccl {

enum class RingRecvKind : uint8_t {
    REDUCE,  // fold the incoming chunk into the local one (reduce-scatter phase)
    COPY,    // the incoming chunk replaces the local one (all-gather phase)
};

// One step of one rank's schedule (csrc/backend/ProcessGroupMCCL.cpp:170-181).
struct RingStep {
    int send_idx;
    int recv_idx;
    uint32_t send_tid;
    uint32_t recv_tid;
    RingRecvKind kind;
};

enum class RingAlgo : int {
    BASIC = 0,    // ws chunks, 2(ws-1) steps
    CHUNKED = 1,  // 2ws chunks, 4(ws-1) steps
};

/// MCCL_RING_ALGO=basic|ring|plain selects the basic ring; anything else, or
/// nothing, the chunked one (csrc/backend/ProcessGroupMCCL.cpp:42-53).  Read on
/// every call.
RingAlgo ring_algo_from_env();

int ring_chunk_count(int ws, RingAlgo algo);

/// Reduce-scatter steps followed by all-gather steps of `rank`
/// (csrc/backend/ProcessGroupMCCL.cpp:1764-1785 chunked, :2016-2035 basic).
std::vector<RingStep> ring_plan(int rank, int ws, RingAlgo algo);

/// ceil(numel / chunks)-element views of a flat tensor; trailing views may be
/// empty (csrc/backend/ProcessGroupMCCL.cpp:1725-1738,:1995-2006).
std::vector<at::Tensor> ring_chunk_views(const at::Tensor& tensor, int ws, RingAlgo algo);

// ---- compressed payload framing (csrc/backend/ProcessGroupMCCL.cpp:1087-1160)
// A message is a 4-byte size followed by exactly that many payload bytes.
struct CompressedFrame {
    uint32_t wire_size = 0;
    at::Tensor payload;  // uint8, wire_size elements, on the tensor's device
};

uint64_t compression_stable_id(const at::Tensor& tensor);
CompressedFrame compressed_pack(Compressor* compressor, const at::Tensor& tensor);
void compressed_unpack(Compressor* compressor, const CompressedFrame& frame, const at::Tensor& out);

// ---- W ranks on one GPU ------------------------------------------------------
class LoopbackGroup {
public:
    struct Stats {
        uint64_t collectives = 0;
        uint64_t reduce_launches = 0;
        uint64_t copy_launches = 0;
        uint64_t fences_signalled = 0;
        uint64_t stream_waits = 0;
        uint64_t wire_bytes = 0;  // size headers + payload bytes, or raw chunk bytes
        std::string last_algo;
    };

    /// One compressor per rank (each rank of the reference owns its own
    /// residual state), made from opts.compression / opts.topk_ratio.
    LoopbackGroup(int world_size, const MCCLOptions& opts, bool rank_streams = true);

    int size() const { return ws_; }
    Compressor* compressor(int rank) const { return compressors_[rank].get(); }
    const Stats& stats() const { return stats_; }

    /// In place on every rank's tensor; dispatch as in
    /// csrc/backend/ProcessGroupMCCL.cpp:1339-1352: two ranks exchange whole
    /// tensors, three or more use the hub below small_msg_threshold bytes and
    /// the ring above.  Returns once the work is enqueued on the current stream.
    void allreduce(std::vector<at::Tensor>& rank_tensors, c10d::ReduceOp::RedOpType op);

    /// Flatten, one allreduce, scatter back (csrc/backend/ProcessGroupMCCL.cpp:1381-1468).
    void allreduce_coalesced(std::vector<std::vector<at::Tensor>>& rank_lists, c10d::ReduceOp::RedOpType op);

    /// outputs[d] = fold over ranks of inputs[rank][d]
    /// (csrc/backend/ProcessGroupMCCL.cpp:3133-3313): with three or more ranks the
    /// star form, rank d's own contribution first and the others in ascending
    /// rank order (:2764-2815); with two ranks one ring step that folds into the
    /// input chunk in place (:3257-3301).  AVG adds and does not scale: the
    /// reference's reduce_scatter never multiplies by 1/ws.
    void reduce_scatter(std::vector<at::Tensor>& outputs, std::vector<std::vector<at::Tensor>>& inputs,
                        c10d::ReduceOp::RedOpType op);

    void allreduce_ring(std::vector<at::Tensor>& rank_tensors, c10d::ReduceOp::RedOpType op, RingAlgo algo);
    void allreduce_two_rank(std::vector<at::Tensor>& rank_tensors, c10d::ReduceOp::RedOpType op);
    void allreduce_small(std::vector<at::Tensor>& rank_tensors, c10d::ReduceOp::RedOpType op);

private:
    void check_ranks(const std::vector<at::Tensor>& rank_tensors) const;
    at::Tensor through_wire(int from_rank, const at::Tensor& tensor);

    int ws_;
    bool rank_streams_;
    size_t small_msg_threshold_;
    std::vector<std::unique_ptr<Compressor>> compressors_;
    Stats stats_;
};

}  // namespace mccl
