// Errors.hpp -- exception types of the backend and the check macro.
//
// Observable contract of the reference's csrc/common/Errors.hpp:9-66: every
// error is a std::runtime_error whose text starts with "[MCCL] "; the kinds the
// path raises add "Tensor: " / "Timeout: " after it; a failed check reads
//   [MCCL] Check failed: <cond> at <file>:<line> — <extra>
// Errors raised inside libmcclx arrive as return codes and are re-thrown here
// with the library's own text (which already carries the prefix).
#pragma once

#include <stdexcept>
#include <string>

#include "mcclx.h"

namespace mccl {

class MCCLError : public std::runtime_error {
public:
    explicit MCCLError(const std::string& text) : std::runtime_error(with_prefix(text)) {}

private:
    static std::string with_prefix(const std::string& text) {
        static const char kPrefix[] = "[MCCL] ";
        return text.compare(0, sizeof kPrefix - 1, kPrefix) == 0 ? text : kPrefix + text;
    }
};

// An error of a named kind: "[MCCL] <Kind>: <text>".
struct TensorKind { static const char* name() { return "Tensor"; } };
struct TimeoutKind { static const char* name() { return "Timeout"; } };

template <class Kind>
class KindError : public MCCLError {
public:
    explicit KindError(const std::string& text) : MCCLError(std::string(Kind::name()) + ": " + text) {}
};
using TensorError = KindError<TensorKind>;
using TimeoutError = KindError<TimeoutKind>;

// A failure reported by libmcclx (its text is complete as it is).
class KernelError : public MCCLError {
public:
    using MCCLError::MCCLError;
};

// Turns a libmcclx return code back into an exception.
inline void check_rc(int rc) {
    if (rc != MCCLX_OK) throw KernelError(mcclx_last_error());
}

[[noreturn]] inline void check_failed(const char* condition, const char* file, int line, const std::string& extra) {
    std::string text = std::string("Check failed: ") + condition + " at " + file + ":" + std::to_string(line);
    if (!extra.empty()) text += " — " + extra;
    throw MCCLError(text);
}

}  // namespace mccl

// MCCL_CHECK(cond) or MCCL_CHECK(cond, "what went wrong")
#define MCCL_CHECK(cond, ...) \
    ((cond) ? (void)0 : ::mccl::check_failed(#cond, __FILE__, __LINE__, std::string(__VA_ARGS__)))
