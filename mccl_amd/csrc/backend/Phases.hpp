// Phases.hpp -- where the host's time goes in a collective: per-phase totals, off unless
// MCCL_PHASE_STATS=1 (then one clock read at each end of a phase; otherwise one branch).
// The reference traces the same path with MCCL_TRACE lines
// (csrc/backend/ProcessGroupMCCL.cpp:105-186); totals are what a tuning run wants.
#pragma once

#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdlib>

namespace mccl {
namespace phases {

enum Phase {
    kBuild = 0,      // argument checks, the rank's contribution, the engine flushed
    kMeet,           // a rank inside the meeting point (for the last arrival: minus what follows)
    kLeaderChecks,   // the last arrival: agreement checks, replay descriptors, workspace
    kStreamWait,     // reduce queue ordered behind the ranks' streams
    kLaunch,         // launches issued
    kDrain,          // host waits for the queue (synchronous completion)
    kSubmit,         // event-based: ticket recorded, completer task queued
    kWorkMake,       // Work and Future objects made / settled on the caller's side
    kWaitHook,       // event-based: Work::wait orders the caller's stream behind the queue
    kCompleterWait,  // completer thread blocked on a launch's ticket
    kSettle,         // completer thread settles Works and Futures
    kCount
};

inline const char* name(int p) {
    static const char* const n[kCount] = {"build", "meet", "leader_checks", "stream_wait", "launch", "drain",
                                          "submit", "work_make", "wait_hook", "completer_wait", "settle"};
    return n[p];
}

struct Totals {
    std::atomic<uint64_t> ns[kCount];
    std::atomic<uint64_t> calls[kCount];
};
inline Totals& totals() {
    static Totals t{};
    return t;
}
inline bool enabled() {
    static const bool on = [] {
        const char* e = std::getenv("MCCL_PHASE_STATS");
        return e && e[0] == '1';
    }();
    return on;
}
inline void reset() {
    for (int p = 0; p < kCount; ++p) {
        totals().ns[p] = 0;
        totals().calls[p] = 0;
    }
}

class Span {
public:
    explicit Span(Phase p) : p_(p), on_(enabled()) {
        if (on_) t0_ = std::chrono::steady_clock::now();
    }
    ~Span() { stop(); }
    void stop() {
        if (!on_) return;
        on_ = false;
        const auto dt = std::chrono::steady_clock::now() - t0_;
        totals().ns[p_] += static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(dt).count());
        ++totals().calls[p_];
    }
    Span(const Span&) = delete;
    Span& operator=(const Span&) = delete;

private:
    Phase p_;
    bool on_;
    std::chrono::steady_clock::time_point t0_;
};

// Time charged to `p` is taken off again here (a phase nested in another one).
inline void discount(Phase p, std::chrono::steady_clock::duration d) {
    if (!enabled()) return;
    totals().ns[p] -= static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(d).count());
}

}  // namespace phases
}  // namespace mccl
