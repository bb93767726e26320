// WorkMCCL.hpp -- completion object of one collective (c10d::Work).
//
// Observable contract of the reference's csrc/backend/WorkMCCL.{hpp,cpp}: the
// object exists from the moment the collective is issued; finish() first runs
// an optional callback (which drains the reduce queue) and then settles the
// Work and its Future with the output tensors; finishWithException() settles
// both with the error; wait() blocks until then, returns false when the
// timeout passes first and rethrows a stored error.
//
// One state variable under one mutex: Pending -> Succeeded | Failed, once.
#pragma once

#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>

#include <ATen/ATen.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <exception>
#include <functional>
#include <mutex>
#include <vector>

namespace mccl {

class WorkMCCL : public c10d::Work {
public:
    WorkMCCL(c10d::OpType op, std::vector<at::Tensor> outputs, const char* title = "mccl:work");
    ~WorkMCCL() override;

    // -- what the issuing side calls (the engine thread, or the caller's thread for allreduce)
    void setSyncCallback(std::function<void()> before_done) { before_done_ = std::move(before_done); }
    // Event-based completion: with a wait hook, wait() does not block the host until
    // the Work is settled.  It runs the hook -- which makes the caller's stream wait,
    // on the device, for the reduce queue -- and returns; the Work and its Future
    // settle later, when the device has finished.  A Work that has settled by the
    // time of the wait needs no hook (the device work is known to be over); one that
    // has failed rethrows from wait().  wait(timeout) with a timeout keeps the
    // reference's contract on top of that: it blocks the host until the Work has
    // settled and returns false when the time is up first.
    void setWaitHook(std::function<void()> on_wait) { on_wait_ = std::move(on_wait); }
    void finish();
    void finishWithException(std::exception_ptr error);

    // -- c10d::Work
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    bool isCompleted() override;
    bool isSuccess() const override;
    std::exception_ptr exception() const override;
    std::vector<at::Tensor> result() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

private:
    enum class State { Pending, Succeeded, Failed };

    // First call wins; later ones do nothing.
    void settle(std::exception_ptr error);

    std::vector<at::Tensor> outputs_;
    c10::intrusive_ptr<c10::ivalue::Future> future_;
    std::function<void()> before_done_;
    std::function<void()> on_wait_;

    mutable std::mutex mu_;
    std::condition_variable settled_cv_;
    State state_ = State::Pending;
    std::atomic<bool> done_{false};  // state_ != Pending, readable without the lock (polled by wait())
    std::exception_ptr error_;
};

}  // namespace mccl
