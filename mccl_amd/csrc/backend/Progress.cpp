#include "backend/Progress.hpp"

#include <utility>

namespace mccl {

namespace {
BlockingHooks g_hooks;
}

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

Progress::Progress() { thread_ = std::thread([this] { worker(); }); }

Progress::~Progress() { shutdown(); }

void Progress::submit(Task task) {
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (closing_) return;
        queue_.push_back(std::move(task));
        ++submitted_;
    }
    wake_.notify_one();
}

void Progress::shutdown() {
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (closing_ && !thread_.joinable()) return;
        closing_ = true;
    }
    wake_.notify_all();
    if (thread_.joinable()) {
        BlockingRegion unlocked;  // the last task may need the caller's interpreter lock to end
        thread_.join();
    }
}

size_t Progress::completed() const {
    std::lock_guard<std::mutex> lk(mu_);
    return completed_;
}

bool Progress::idle() const {
    std::lock_guard<std::mutex> lk(mu_);
    return completed_ == submitted_;
}

void Progress::worker() {
    std::unique_lock<std::mutex> lk(mu_);
    for (;;) {
        wake_.wait(lk, [this] { return closing_ || !queue_.empty(); });
        if (queue_.empty()) return;  // closing and drained
        Task task = std::move(queue_.front());
        queue_.pop_front();
        lk.unlock();
        try {
            task();
        } catch (...) {
            // the task reports its own failure through its Work object
        }
        task = nullptr;  // its captures die here, outside the queue lock
        lk.lock();
        ++completed_;
    }
}

}  // namespace mccl
