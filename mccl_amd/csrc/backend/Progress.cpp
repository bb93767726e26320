#include "backend/Progress.hpp"

#include <chrono>
#include <utility>

namespace mccl {

namespace {
BlockingHooks g_hooks;

// Every worker thread that is still running.  An engine shut down from inside one of its own
// tasks cannot join its thread and lets it go; such a thread -- typically the last holder of a
// process group, busy destroying it -- may still be unwinding when main() returns, and would
// then read the registries and allocators the process is tearing down.  The end of the process
// therefore waits here (this object is made with the first engine, so it goes before the
// statics that were there earlier) until every worker has left its loop.
struct Workers {
    std::mutex mu;
    int running = 0;
    void enter() {
        std::lock_guard<std::mutex> lk(mu);
        ++running;
    }
    void leave() {
        std::lock_guard<std::mutex> lk(mu);
        --running;
    }
    ~Workers() {
        BlockingRegion unlocked;  // a worker may need the caller's interpreter lock to finish its task
        for (int ms = 0; ms < 10000; ++ms) {  // polled: a worker that never ends must not keep the process
            {
                std::lock_guard<std::mutex> lk(mu);
                if (running == 0) return;
            }
            std::this_thread::sleep_for(std::chrono::milliseconds(1));
        }
    }
};
Workers& workers() {
    static Workers w;
    return w;
}
}  // namespace

void set_blocking_hooks(BlockingHooks hooks) { g_hooks = hooks; }

BlockingRegion::BlockingRegion() {
    if (g_hooks.enter && g_hooks.leave) {
        token_ = g_hooks.enter();
        entered_ = true;
    }
}

BlockingRegion::~BlockingRegion() {
    if (entered_) g_hooks.leave(token_);
}

Progress::Progress() : st_(std::make_shared<State>()) {
    workers().enter();  // counted before the thread exists: the count never reads zero while one is starting
    try {
        thread_ = std::thread(&Progress::worker, st_);
    } catch (...) {
        workers().leave();
        throw;
    }
}

Progress::~Progress() { shutdown(); }

void Progress::submit(Task task) {
    {
        std::lock_guard<std::mutex> lk(st_->mu);
        if (st_->closing) return;
        st_->queue.push_back(std::move(task));
        ++st_->submitted;
    }
    st_->wake.notify_one();
}

bool Progress::on_worker_thread() const { return std::this_thread::get_id() == thread_.get_id(); }

void Progress::shutdown() {
    if (!thread_.joinable()) return;  // shut down before (only the owner calls this: no race on thread_)
    if (on_worker_thread()) {
        // Called from inside one of this engine's own tasks.  What is queued behind that task
        // runs here and now, in order -- the caller is about to tear down what those tasks
        // use -- and the thread is let go instead of joined: the loop up the stack finds the
        // queue empty and closing, and ends on its own, on state it shares with this object.
        std::unique_lock<std::mutex> lk(st_->mu);
        st_->closing = true;
        while (!st_->queue.empty()) run_next(*st_, lk);
        lk.unlock();
        thread_.detach();
        return;
    }
    {
        std::lock_guard<std::mutex> lk(st_->mu);
        st_->closing = true;
    }
    st_->wake.notify_all();
    BlockingRegion unlocked;  // the last task may need the caller's interpreter lock to end
    thread_.join();
}

size_t Progress::completed() const {
    std::lock_guard<std::mutex> lk(st_->mu);
    return st_->completed;
}

bool Progress::idle() const {
    std::lock_guard<std::mutex> lk(st_->mu);
    return st_->completed == st_->submitted;
}

void Progress::run_next(State& st, std::unique_lock<std::mutex>& lk) {
    Task task = std::move(st.queue.front());
    st.queue.pop_front();
    lk.unlock();
    try {
        task();
    } catch (...) {
        // the task reports its own failure through its Work object
    }
    try {
        task = nullptr;  // its captures die here, outside the queue lock
    } catch (...) {
        // a capture's destructor threw: nothing to report it to, and the engine goes on
    }
    lk.lock();
    ++st.completed;
}

void Progress::worker(std::shared_ptr<State> st) {
    {
        std::unique_lock<std::mutex> lk(st->mu);
        for (;;) {
            st->wake.wait(lk, [&] { return st->closing || !st->queue.empty(); });
            if (st->queue.empty()) break;  // closing and drained
            run_next(*st, lk);
        }
    }
    st.reset();
    workers().leave();  // last: nothing of the process is touched after this
}

}  // namespace mccl
