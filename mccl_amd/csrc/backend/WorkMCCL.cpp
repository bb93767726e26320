#include "backend/WorkMCCL.hpp"

#include <ATen/core/ivalue.h>

namespace mccl {

WorkMCCL::WorkMCCL(c10d::OpType op, std::vector<at::Tensor> outputs, const char* title)
    : c10d::Work(/*rank=*/-1, op, title, outputs), outputs_(std::move(outputs)) {
    std::vector<c10::Device> devices;
    for (const auto& t : outputs_)
        if (t.defined() && t.device().has_index()) devices.push_back(t.device());
    future_ = c10::make_intrusive<c10::ivalue::Future>(c10::ListType::create(c10::TensorType::get()),
                                                       devices);
}

WorkMCCL::~WorkMCCL() = default;

bool WorkMCCL::isCompleted() { return done_.load(std::memory_order_acquire); }

bool WorkMCCL::isSuccess() const {
    std::lock_guard<std::mutex> lk(mu_);
    return done_.load(std::memory_order_acquire) && !error_;
}

std::exception_ptr WorkMCCL::exception() const {
    std::lock_guard<std::mutex> lk(mu_);
    return error_;
}

bool WorkMCCL::wait(std::chrono::milliseconds timeout) {
    std::unique_lock<std::mutex> lk(mu_);
    auto finished = [this] { return done_.load(std::memory_order_acquire); };
    if (timeout == kNoTimeout)
        done_cv_.wait(lk, finished);
    else if (!done_cv_.wait_for(lk, timeout, finished))
        return false;
    if (error_) std::rethrow_exception(error_);
    return true;
}

std::vector<at::Tensor> WorkMCCL::result() { return outputs_; }

c10::intrusive_ptr<c10::ivalue::Future> WorkMCCL::getFuture() { return future_; }

// First caller wins; later finish()/finishWithException() calls are no-ops.
bool WorkMCCL::complete(std::exception_ptr error) {
    std::lock_guard<std::mutex> lk(mu_);
    if (done_.load(std::memory_order_acquire)) return false;
    error_ = error;
    done_.store(true, std::memory_order_release);
    return true;
}

void WorkMCCL::finish() {
    if (sync_) {
        try {
            sync_();
        } catch (...) {
            finishWithException(std::current_exception());
            return;
        }
    }
    if (!complete(nullptr)) return;
    if (future_ && !future_->completed()) future_->markCompleted(c10::IValue(outputs_));
    done_cv_.notify_all();
}

void WorkMCCL::finishWithException(std::exception_ptr error) {
    if (!complete(error)) return;
    if (future_ && !future_->completed()) future_->setError(error);
    done_cv_.notify_all();
}

}  // namespace mccl
