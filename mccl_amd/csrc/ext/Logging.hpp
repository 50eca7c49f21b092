// stderr logger gated by MCCL_LOG_LEVEL (TRACE..OFF, default WARN), the same
// variable and level names the reference reads (csrc/common/Logging.hpp:22-34).
#pragma once

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace mccl {

enum class LogLevel : int { TRACE = 0, DEBUG = 1, INFO = 2, WARN = 3, ERROR = 4, FATAL = 5, OFF = 6 };

inline LogLevel parse_log_level(const char* s) {
    static const char* names[] = {"TRACE", "DEBUG", "INFO", "WARN", "ERROR", "FATAL", "OFF"};
    if (!s) return LogLevel::WARN;
    for (int i = 0; i < 7; i++) {
        if (!strcasecmp(s, names[i]) || (s[0] == '0' + i && s[1] == 0)) return static_cast<LogLevel>(i);
    }
    return LogLevel::WARN;
}

inline LogLevel& log_level() {
    static LogLevel lvl = parse_log_level(std::getenv("MCCL_LOG_LEVEL"));
    return lvl;
}

inline void refresh_log_level() { log_level() = parse_log_level(std::getenv("MCCL_LOG_LEVEL")); }

inline void log_line(LogLevel lvl, const char* tag, const char* fmt, ...) {
    if (lvl < log_level()) return;
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    std::fprintf(stderr, "[MCCL %s] %s\n", tag, buf);
}

}  // namespace mccl

#define MCCL_TRACE(...) ::mccl::log_line(::mccl::LogLevel::TRACE, "TRACE", __VA_ARGS__)
#define MCCL_DEBUG(...) ::mccl::log_line(::mccl::LogLevel::DEBUG, "DEBUG", __VA_ARGS__)
#define MCCL_INFO(...) ::mccl::log_line(::mccl::LogLevel::INFO, "INFO ", __VA_ARGS__)
#define MCCL_WARN(...) ::mccl::log_line(::mccl::LogLevel::WARN, "WARN ", __VA_ARGS__)
