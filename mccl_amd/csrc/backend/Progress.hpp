// Progress.hpp -- one worker thread that runs submitted tasks strictly in
// submission order.  Each ProcessGroup owns one; every asynchronous collective
// becomes one task, so all ranks execute collectives in the same order.
//
// Behaviour matches the reference's csrc/backend/Progress.{hpp,cpp} as pinned by
// its tests/internal/test_progress.cpp: FIFO order, the destructor drains the
// queue, shutdown is idempotent, a throwing task does not stop the engine,
// submit never waits for a running task.
//
// One thing the reference leaves open is settled here: the engine may be shut
// down, or destroyed, from its own worker thread -- by a task (or a callback a
// task runs) that drops the last reference to whatever owns the engine.  A
// thread cannot join itself (std::thread::join throws, and a throw inside a
// destructor ends the process), so in that case shutdown() runs what is still
// queued right there, on the worker, and lets the thread go; the state the
// worker loop still needs afterwards is shared with it and outlives the engine,
// and the end of the process waits for every worker that is still running.
#pragma once

#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
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
    // Run everything already queued, then stop the worker.  Safe to call twice,
    // and from the worker thread itself (see above).
    void shutdown();
    // Tasks run so far (for tests and diagnostics).
    size_t completed() const;
    // True when every task submitted so far has run to its end.
    bool idle() const;
    // True on the engine's own worker thread.
    bool on_worker_thread() const;

private:
    // Everything the worker loop touches: shared with the thread, so that it stays
    // valid when the engine object is destroyed from inside one of its own tasks.
    struct State {
        std::mutex mu;
        std::condition_variable wake;
        std::deque<Task> queue;
        bool closing = false;
        size_t completed = 0;
        size_t submitted = 0;
    };
    static void worker(std::shared_ptr<State> st);
    // Takes the next task off the queue (the lock is held on entry and on return), runs it
    // and destroys it -- captures included -- with every exception contained.
    static void run_next(State& st, std::unique_lock<std::mutex>& lk);

    std::shared_ptr<State> st_;
    std::thread thread_;
};

}  // namespace mccl
