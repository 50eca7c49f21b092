// Backend options exposed to Python.  The field list is one table: every row is
// an option of the reference's MCCLOptions with its type and default
// (csrc/backend/Options.hpp:19-44); the struct members and the Python
// properties are both generated from it.  Only compression, topk_ratio,
// small_msg_threshold, fast_math and gpu_threshold mean something to this build
// (no transport, no engine); the rest is kept so that option objects written for
// the reference load unchanged.
#pragma once

#include <torch/csrc/distributed/c10d/Backend.hpp>

#include <chrono>
#include <string>

#include "Compression.hpp"

// X(type, name, default)
#define MCCL_OPTION_TABLE(X)                                                              \
    X(std::string, transport, "auto")                                                     \
    X(std::string, listen_addr, "0.0.0.0")                                                \
    X(uint16_t, port_base, 20100)                                                         \
    X(std::string, ifname, "")                                                            \
    X(size_t, chunk_bytes, size_t(16) << 20)                                              \
    X(size_t, small_msg_threshold, size_t(256) << 10)                                     \
    X(bool, transport_crc, false)                                                         \
    X(bool, fast_math, true)                                                              \
    X(uint32_t, gpu_threshold, 4096u)                                                     \
    X(bool, overlap_comm, true)                                                           \
    X(size_t, max_queue_depth, 1024)                                                      \
    X(::mccl::CompressionMode, compression, ::mccl::CompressionMode::NONE)                \
    X(double, topk_ratio, 0.01)                                                           \
    X(std::chrono::milliseconds, watchdog_timeout, std::chrono::milliseconds(300000))     \
    X(std::chrono::milliseconds, heartbeat_interval, std::chrono::milliseconds(5000))

namespace mccl {

struct MCCLOptions : public c10d::Backend::Options {
    explicit MCCLOptions(std::chrono::milliseconds timeout = std::chrono::milliseconds(30000))
        : c10d::Backend::Options("mccl", timeout) {}

#define MCCL_OPTION_MEMBER(type, name, init) type name = init;
    MCCL_OPTION_TABLE(MCCL_OPTION_MEMBER)
#undef MCCL_OPTION_MEMBER
};

}  // namespace mccl
