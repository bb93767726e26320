// Logging.hpp -- stderr logger of the backend.
//
// Same knobs and line shape as the reference's csrc/common/Logging.hpp:22-78:
// DISTRO_LOG_LEVEL = TRACE|DEBUG|INFO|WARN|ERROR|FATAL|OFF (any case, or 0..6),
// default WARN, read once; a line reads
//   [MCCL <LEVEL> <epoch ms> <file>:<line>] message
#pragma once

#include <strings.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <mutex>

namespace mccl {
namespace log {

enum Level { kTrace = 0, kDebug, kInfo, kWarn, kError, kFatal, kOff };

inline const char* const* level_names() {
    static const char* const names[] = {"TRACE", "DEBUG", "INFO", "WARN", "ERROR", "FATAL", "OFF"};
    return names;
}

inline int parse_level(const char* text) {
    if (!text || !*text) return kWarn;
    for (int l = kTrace; l <= kOff; ++l)
        if (strcasecmp(text, level_names()[l]) == 0 || (text[0] == '0' + l && text[1] == '\0')) return l;
    return kWarn;
}

inline int& threshold() {
    static int level = parse_level(std::getenv("DISTRO_LOG_LEVEL"));
    return level;
}

inline bool enabled(int level) { return level >= threshold() && level < kOff; }

inline void emit(int level, const char* file, int line, const char* fmt, ...) {
    if (!enabled(level)) return;
    char msg[1024];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(msg, sizeof msg, fmt, ap);
    va_end(ap);
    const long long ms = std::chrono::duration_cast<std::chrono::milliseconds>(
                             std::chrono::system_clock::now().time_since_epoch()).count();
    static std::mutex mu;  // whole lines, also from the engine threads
    std::lock_guard<std::mutex> lk(mu);
    std::fprintf(stderr, "[MCCL %-5s %lld %s:%d] %s\n", level_names()[level], ms, file, line, msg);
    std::fflush(stderr);
}

}  // namespace log
}  // namespace mccl

#define MCCL_LOG_AT(level, ...) ::mccl::log::emit(::mccl::log::level, __FILE__, __LINE__, __VA_ARGS__)
#define MCCL_TRACE(...) MCCL_LOG_AT(kTrace, __VA_ARGS__)
#define MCCL_DEBUG(...) MCCL_LOG_AT(kDebug, __VA_ARGS__)
#define MCCL_INFO(...) MCCL_LOG_AT(kInfo, __VA_ARGS__)
#define MCCL_WARN(...) MCCL_LOG_AT(kWarn, __VA_ARGS__)
#define MCCL_ERROR(...) MCCL_LOG_AT(kError, __VA_ARGS__)
