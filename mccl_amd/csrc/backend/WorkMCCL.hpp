// WorkMCCL.hpp -- completion object of one collective (c10d::Work).
//
// Contract of the reference's csrc/backend/WorkMCCL.{hpp,cpp}: created when the
// collective is issued; finish() runs an optional sync callback (which drains
// the reduce queue) and then completes the Work and its Future with the output
// tensors; finishWithException() completes both with the error; wait() blocks
// until then, returns false on timeout and rethrows the stored error.
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

    bool isCompleted() override;
    bool isSuccess() const override;
    std::exception_ptr exception() const override;
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    std::vector<at::Tensor> result() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

    void finish();
    void finishWithException(std::exception_ptr error);
    void setSyncCallback(std::function<void()> cb) { sync_ = std::move(cb); }

private:
    bool complete(std::exception_ptr error);

    mutable std::mutex mu_;
    std::condition_variable done_cv_;
    std::atomic<bool> done_{false};
    std::exception_ptr error_;
    std::vector<at::Tensor> outputs_;
    c10::intrusive_ptr<c10::ivalue::Future> future_;
    std::function<void()> sync_;
};

}  // namespace mccl
