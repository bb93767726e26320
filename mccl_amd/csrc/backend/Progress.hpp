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

// A host with an interpreter lock (CPython's GIL) registers a pair of hooks.
// They bracket every place where a caller blocks until the worker thread has
// got somewhere, because a task may need that lock before it can end: when a
// task drops the last reference to a tensor that Python created, the tensor's
// destructor takes the GIL.  A caller that joined the worker while holding the
// GIL (a process group destroyed from Python does) would then wait for ever.
struct BlockingHooks {
    void* (*enter)() = nullptr;    // give the lock up if this thread holds it; returns a token
    void (*leave)(void*) = nullptr;  // take it back
};
void set_blocking_hooks(BlockingHooks hooks);

// RAII use of the hooks; a no-op when none are registered.
class BlockingRegion {
public:
    BlockingRegion();
    ~BlockingRegion();
    BlockingRegion(const BlockingRegion&) = delete;
    BlockingRegion& operator=(const BlockingRegion&) = delete;

private:
    void* token_ = nullptr;
    bool entered_ = false;
};

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
    // True when every task submitted so far has run to its end.
    bool idle() const;

private:
    void worker();

    mutable std::mutex mu_;
    std::condition_variable wake_;
    std::deque<Task> queue_;
    bool closing_ = false;
    size_t completed_ = 0;
    size_t submitted_ = 0;
    std::thread thread_;
};

}  // namespace mccl
