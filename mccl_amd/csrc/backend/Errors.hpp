// Errors.hpp -- exception types of the backend and the check macro.
//
// Same observable contract as the reference's csrc/common/Errors.hpp:9-66:
// every error is a std::runtime_error whose message starts with "[MCCL] ";
// a failed check reads "[MCCL] Check failed: <cond> at <file>:<line> — <extra>".
// Errors raised inside libmcclx arrive as return codes and are re-thrown here
// with the library's own message (which already carries the prefix).
#pragma once

#include <sstream>
#include <stdexcept>
#include <string>

#include "mcclx.h"

namespace mccl {

class MCCLError : public std::runtime_error {
public:
    explicit MCCLError(const std::string& msg) : std::runtime_error(prefixed(msg)) {}

private:
    static std::string prefixed(const std::string& m) {
        return m.rfind("[MCCL] ", 0) == 0 ? m : "[MCCL] " + m;
    }
};

class TensorError : public MCCLError {
public:
    explicit TensorError(const std::string& msg) : MCCLError("Tensor: " + msg) {}
};

class TimeoutError : public MCCLError {
public:
    explicit TimeoutError(const std::string& msg) : MCCLError("Timeout: " + msg) {}
};

class KernelError : public MCCLError {
public:
    explicit KernelError(const std::string& msg) : MCCLError(msg) {}
};

// Turns a libmcclx return code back into an exception.
inline void check_rc(int rc) {
    if (rc != MCCLX_OK) throw KernelError(mcclx_last_error());
}

}  // namespace mccl

#define MCCL_CHECK(cond, ...)                                                        \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::ostringstream mccl_check_ss_;                                       \
            mccl_check_ss_ << "Check failed: " #cond " at " << __FILE__ << ":" << __LINE__; \
            const std::string mccl_check_extra_ = std::string(__VA_ARGS__);          \
            if (!mccl_check_extra_.empty()) mccl_check_ss_ << " — " << mccl_check_extra_; \
            throw ::mccl::MCCLError(mccl_check_ss_.str());                           \
        }                                                                            \
    } while (false)
