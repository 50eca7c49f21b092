// Error types of the host layer.  Class names, the "[MCCL] " / "Tensor: "
// prefixes and the two check macros follow csrc/common/Errors.hpp:9-66 of the
// reference so that callers (and tests matching on message text) see the same
// exceptions; pybind turns them into RuntimeError.
#pragma once

#include <sstream>
#include <stdexcept>
#include <string>

namespace mccl {

struct MCCLError : std::runtime_error {
    explicit MCCLError(const std::string& what) : std::runtime_error("[MCCL] " + what) {}
};
struct TensorError : MCCLError {
    explicit TensorError(const std::string& what) : MCCLError("Tensor: " + what) {}
};
struct TimeoutError : MCCLError {
    explicit TimeoutError(const std::string& what) : MCCLError("Timeout: " + what) {}
};
// The reference's MetalError: a failure of the device kernel layer.
struct MetalError : MCCLError {
    explicit MetalError(const std::string& what) : MCCLError("Metal: " + what) {}
};

namespace detail {
template <class E>
[[noreturn]] inline void fail(const char* head, const char* cond, const char* file, int line,
                              const std::string& extra) {
    std::ostringstream os;
    os << head << cond;
    if (file) os << " at " << file << ":" << line;
    if (!extra.empty()) os << " — " << extra;
    throw E(os.str());
}
}  // namespace detail

}  // namespace mccl

#define MCCL_CHECK(cond, ...)                                                                       \
    do {                                                                                            \
        if (!(cond))                                                                                \
            ::mccl::detail::fail<::mccl::MCCLError>("Check failed: ", #cond, __FILE__, __LINE__,    \
                                                    std::string(__VA_ARGS__));                      \
    } while (false)

#define MCCL_CHECK_TENSOR(cond, ...)                                                                \
    do {                                                                                            \
        if (!(cond))                                                                                \
            ::mccl::detail::fail<::mccl::TensorError>("Tensor check failed: ", #cond, nullptr, 0,   \
                                                      std::string(__VA_ARGS__));                    \
    } while (false)
