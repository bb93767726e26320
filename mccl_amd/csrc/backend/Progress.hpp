// Progress.hpp -- one worker thread that runs submitted tasks strictly in
// submission order.  Each ProcessGroup owns one; every asynchronous collective
// becomes one task, so all ranks execute collectives in the same order.
//
// Behaviour matches the reference's csrc/backend/Progress.{hpp,cpp} as pinned by
// its tests/internal/test_progress.cpp: FIFO order, the destructor drains the
// queue, shutdown is idempotent, a throwing task does not stop the engine,
// submit never waits for a running task.
#pragma once

#include <condition_variable>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

namespace mccl {

class Progress {
public:
    using Task = std::function<void()>;

    Progress();
    ~Progress();
    Progress(const Progress&) = delete;
    Progress& operator=(const Progress&) = delete;

    // Enqueue; returns at once.  Tasks submitted after shutdown() are dropped.
    void submit(Task task);
    // Run everything already queued, then stop the worker.  Safe to call twice.
    void shutdown();
    // Tasks run so far (for tests and diagnostics).
    size_t completed() const;

private:
    void worker();

    mutable std::mutex mu_;
    std::condition_variable wake_;
    std::deque<Task> queue_;
    bool closing_ = false;
    size_t completed_ = 0;
    std::thread thread_;
};

}  // namespace mccl
