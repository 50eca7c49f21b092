// Backend options exposed to Python; field names and defaults follow
// csrc/backend/Options.hpp:12-45.  Only compression and topk_ratio change what this
// build does (no transport, no engine); fast_math and gpu_threshold are accepted and
// ignored: there is one arithmetic (IEEE, no contraction) and no host fold to fall back to.
#pragma once

#include <torch/csrc/distributed/c10d/Backend.hpp>

#include <chrono>
#include <string>

#include "Compression.hpp"

namespace mccl {

struct MCCLOptions : public c10d::Backend::Options {
    MCCLOptions() : c10d::Backend::Options("mccl", std::chrono::milliseconds(30000)) {}
    explicit MCCLOptions(std::chrono::milliseconds timeout) : c10d::Backend::Options("mccl", timeout) {}

    std::string transport = "auto";
    std::string listen_addr = "0.0.0.0";
    uint16_t port_base = 20100;
    std::string ifname;
    size_t chunk_bytes = 16 * 1024 * 1024;
    size_t small_msg_threshold = 262144;
    bool transport_crc = false;

    bool fast_math = true;
    uint32_t gpu_threshold = 4096;
    bool overlap_comm = true;

    size_t max_queue_depth = 1024;

    CompressionMode compression = CompressionMode::NONE;
    double topk_ratio = 0.01;

    std::chrono::milliseconds watchdog_timeout{300000};
    std::chrono::milliseconds heartbeat_interval{5000};
};

}  // namespace mccl
