#include "backend/WorkMCCL.hpp"

#include <ATen/core/ivalue.h>

#include <cstdlib>

#include "backend/Errors.hpp"

namespace mccl {

WorkMCCL::WorkMCCL(c10d::OpType op, std::vector<at::Tensor> outputs, const char* title)
    : c10d::Work(/*rank=*/-1, op, title, outputs),
      outputs_(std::move(outputs)),
      // A Future that is told its value's devices records an event on each of them when it is
      // completed and makes every waiter's streams wait for those events (some 8 us of host
      // time per Work on this runtime).  Nothing here needs that: a Work settles only after
      // the host has seen the reduce queue finish the device work (a drain, or the launch's
      // completion ticket), so the result is visible to whatever any stream runs next.
      future_(c10::make_intrusive<c10::ivalue::Future>(c10::ListType::create(c10::TensorType::get()))) {}

WorkMCCL::~WorkMCCL() = default;

void WorkMCCL::settle(std::exception_ptr error) {
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (state_ != State::Pending) return;
        error_ = error;
        state_ = error ? State::Failed : State::Succeeded;
        done_.store(true, std::memory_order_release);
    }
    // outside the lock: the Future runs its callbacks inline
    if (error)
        future_->setError(error);
    else
        future_->markCompleted(c10::IValue(outputs_));
    settled_cv_.notify_all();
}

void WorkMCCL::finish() {
    std::exception_ptr failure;
    if (before_done_) {
        try {
            before_done_();
        } catch (...) {
            failure = std::current_exception();  // a failed drain fails the collective
        }
    }
    settle(failure);
}

void WorkMCCL::finishWithException(std::exception_ptr error) {
    settle(error ? error : std::make_exception_ptr(MCCLError("collective failed without an error object")));
}

namespace {
// How long wait() polls for a Work that is about to settle before it pays for a device-side
// wait instead (MCCL_WAIT_SPIN_US, default 30, 0 = not at all).  Putting torch's legacy stream
// behind an event costs the host 20-35 us on this runtime -- as long as the device work of a
// whole gradient bucket -- so a caller that waits for its buckets in the order it issued them
// is usually served sooner by the completer thread than by the event.  The poll is bounded by
// about what the event would cost, so the worst case is twice the better choice.
std::chrono::microseconds wait_spin() {
    static const long us = [] {
        const char* e = std::getenv("MCCL_WAIT_SPIN_US");
        if (!e || !*e) return 30L;
        const long v = std::strtol(e, nullptr, 10);
        return v < 0 ? 0L : v > 100000 ? 100000L : v;
    }();
    return std::chrono::microseconds(us);
}
}  // namespace

bool WorkMCCL::wait(std::chrono::milliseconds timeout) {
    if (on_wait_) {
        const auto settled_now = [this] {
            // settled already: the device work has been seen to end, nothing to order against
            std::lock_guard<std::mutex> lk(mu_);
            if (state_ == State::Failed) std::rethrow_exception(error_);
            return state_ == State::Succeeded;
        };
        if (settled_now()) return true;
        if (wait_spin().count() > 0) {
            const auto until = std::chrono::steady_clock::now() + wait_spin();
            while (std::chrono::steady_clock::now() < until) {
                if (done_.load(std::memory_order_acquire) && settled_now()) return true;
                __builtin_ia32_pause();
            }
        }
        on_wait_();  // stream-ordered: the caller's stream now waits for the result on the device
        std::unique_lock<std::mutex> lk(mu_);
        if (timeout != kNoTimeout) {
            // A caller that names a timeout asks for the reference's contract (host-blocking,
            // false when the time is up, WorkMCCL.cpp:51-55): wait until the Work has settled.
            const auto settled = [this] { return state_ != State::Pending; };
            if (!settled_cv_.wait_for(lk, timeout, settled)) return false;
        }
        if (state_ == State::Failed) std::rethrow_exception(error_);
        return true;
    }
    std::unique_lock<std::mutex> lk(mu_);
    const auto settled = [this] { return state_ != State::Pending; };
    if (timeout == kNoTimeout)
        settled_cv_.wait(lk, settled);
    else if (!settled_cv_.wait_for(lk, timeout, settled))
        return false;
    if (state_ == State::Failed) std::rethrow_exception(error_);
    return true;
}

bool WorkMCCL::isCompleted() {
    std::lock_guard<std::mutex> lk(mu_);
    return state_ != State::Pending;
}

bool WorkMCCL::isSuccess() const {
    std::lock_guard<std::mutex> lk(mu_);
    return state_ == State::Succeeded;
}

std::exception_ptr WorkMCCL::exception() const {
    std::lock_guard<std::mutex> lk(mu_);
    return error_;
}

std::vector<at::Tensor> WorkMCCL::result() { return outputs_; }

c10::intrusive_ptr<c10::ivalue::Future> WorkMCCL::getFuture() { return future_; }

}  // namespace mccl
