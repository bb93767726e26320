#include "backend/WorkMCCL.hpp"

#include <ATen/core/ivalue.h>

#include "backend/Errors.hpp"

namespace mccl {

namespace {

// The Future must know which devices its value lives on.
std::vector<c10::Device> devices_of(const std::vector<at::Tensor>& tensors) {
    std::vector<c10::Device> devices;
    for (const at::Tensor& t : tensors)
        if (t.defined() && t.device().has_index()) devices.push_back(t.device());
    return devices;
}

}  // namespace

WorkMCCL::WorkMCCL(c10d::OpType op, std::vector<at::Tensor> outputs, const char* title)
    : c10d::Work(/*rank=*/-1, op, title, outputs),
      outputs_(std::move(outputs)),
      future_(c10::make_intrusive<c10::ivalue::Future>(c10::ListType::create(c10::TensorType::get()),
                                                       devices_of(outputs_))) {}

WorkMCCL::~WorkMCCL() = default;

void WorkMCCL::settle(std::exception_ptr error) {
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (state_ != State::Pending) return;
        error_ = error;
        state_ = error ? State::Failed : State::Succeeded;
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

bool WorkMCCL::wait(std::chrono::milliseconds timeout) {
    if (on_wait_) {
        {
            // settled already: the device work has been seen to end, nothing to order against
            std::lock_guard<std::mutex> lk(mu_);
            if (state_ == State::Succeeded) return true;
            if (state_ == State::Failed) std::rethrow_exception(error_);
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
