#include "backend/LocalMesh.hpp"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <unistd.h>

#include "backend/Errors.hpp"

namespace mccl {

namespace {
std::mutex g_registry_mu;
std::map<std::string, std::weak_ptr<LocalMesh>> g_registry;
std::atomic<uint64_t> g_next_id{1};

int env_spin_us() {
    const char* e = std::getenv("MCCL_MEET_SPIN_US");
    if (!e || !*e) return 200;
    const long v = std::strtol(e, nullptr, 10);
    return v < 0 ? 0 : v > 100000 ? 100000 : static_cast<int>(v);
}
}  // namespace

LocalMesh::LocalMesh(int world)
    : world_(world), slots_(static_cast<size_t>(world)), spin_us_(env_spin_us()),
      boxes_(static_cast<size_t>(world) * static_cast<size_t>(world)),
      wires_(static_cast<size_t>(world) * static_cast<size_t>(world)) {
    MCCL_CHECK(world >= 1 && static_cast<uint64_t>(world) < kCountMask, "mesh: world size out of range");
}

std::string LocalMesh::fresh_key() {
    return "pid" + std::to_string(::getpid()) + "-mesh" + std::to_string(g_next_id.fetch_add(1));
}

std::shared_ptr<LocalMesh> LocalMesh::create(const std::string& key, int world) {
    auto mesh = std::make_shared<LocalMesh>(world);
    std::lock_guard<std::mutex> lk(g_registry_mu);
    g_registry[key] = mesh;
    return mesh;
}

std::shared_ptr<LocalMesh> LocalMesh::find(const std::string& key) {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    auto it = g_registry.find(key);
    return it == g_registry.end() ? nullptr : it->second.lock();
}

void LocalMesh::forget(const std::string& key) {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    auto it = g_registry.find(key);
    if (it != g_registry.end() && it->second.expired()) g_registry.erase(it);
}

// The meeting point takes no lock on its fast path: a rank puts its contribution into its own
// slot and counts itself in with one atomic add; whoever counts in last runs the leader and then
// moves the generation on, which is what the others poll.  (With a mutex around arrival and
// departure, three ranks that arrive within a microsecond of each other -- the usual case: they
// left the previous collective together -- queue up on it twice per collective, and where a
// contended mutex means a system call that cost up to 7 us per bucket.)  The mutex and the
// condition variable remain for ranks that have polled long enough and go to sleep.
//
// Generation and head count share one word (generation << 16 | arrived), so that a rank whose
// wait has timed out can take its arrival back only if the collective it arrived for is still
// the current one and has no leader yet: if the last rank has counted in meanwhile, the leader
// is working with this rank's buffers and the rank waits for it to finish instead of leaving.
//
// Why the slots need no lock: a rank writes its slot before it counts itself in (release), the
// leader reads the slots after it has counted in last (acquire); nobody can arrive for the next
// collective before the generation has moved on, which the leader does after its last read.
// The same holds for last_error_: written before the generation moves on, read after, and not
// written again until every rank has left this collective and arrived for the next.
void LocalMesh::rendezvous(int rank, Contribution c, std::chrono::milliseconds timeout,
                           const Leader& leader) {
    MCCL_CHECK(rank >= 0 && rank < world_, "rank outside the mesh");
    if (broken_.load(std::memory_order_acquire))
        throw MCCLError("mesh is broken by an earlier timeout; the group cannot continue");
    slots_[static_cast<size_t>(rank)] = std::move(c);
    const uint64_t before = state_.fetch_add(1, std::memory_order_acq_rel);
    const uint64_t my_generation = before >> kCountBits;
    if (static_cast<int>(before & kCountMask) + 1 == world_) {
        // Last arrival: every contribution is in.  Ranks must be inside the same collective.
        std::exception_ptr err;
        try {
            for (int r = 1; r < world_; ++r)
                MCCL_CHECK(slots_[static_cast<size_t>(r)].kind == slots_[0].kind,
                           "ranks issued different collectives (rank 0 kind " +
                               std::to_string(slots_[0].kind) + ", rank " + std::to_string(r) +
                               " kind " + std::to_string(slots_[static_cast<size_t>(r)].kind) + ")");
            for (int r = 0; r < world_; ++r)
                if (!slots_[static_cast<size_t>(r)].error.empty())
                    throw MCCLError(slots_[static_cast<size_t>(r)].error + " (raised on rank " +
                                    std::to_string(r) + ")");
            leader(slots_);
        } catch (...) {
            err = std::current_exception();
        }
        last_error_ = err;
        state_.store((my_generation + 1) << kCountBits, std::memory_order_release);
        { std::lock_guard<std::mutex> lk(mu_); }  // a waiter on its way to sleep has either seen the new generation or sleeps by now
        cv_.notify_all();
        if (err) std::rethrow_exception(err);
        return;
    }
    auto moved_on = [&] { return (state_.load(std::memory_order_acquire) >> kCountBits) != my_generation; };
    auto released = [&] { return moved_on() || broken_.load(std::memory_order_acquire); };
    bool out = false;
    if (spin_us_ > 0) {
        const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(spin_us_);
        for (;;) {
            for (int k = 0; k < 32 && !(out = released()); ++k) __builtin_ia32_pause();
            if (out || std::chrono::steady_clock::now() >= until) break;
        }
    }
    if (!out) {
        std::unique_lock<std::mutex> lk(mu_);
        if (timeout.count() <= 0) {
            cv_.wait(lk, released);
        } else if (!cv_.wait_for(lk, timeout, released)) {
            // Time is up.  Take the arrival back -- unless the last rank has counted in meanwhile.
            uint64_t cur = state_.load(std::memory_order_acquire);
            bool withdrew = false;
            while ((cur >> kCountBits) == my_generation && static_cast<int>(cur & kCountMask) < world_ && (cur & kCountMask) > 0)
                if (state_.compare_exchange_weak(cur, cur - 1, std::memory_order_acq_rel)) {
                    withdrew = true;
                    break;
                }
            if (withdrew) {
                broken_.store(true, std::memory_order_release);
                lk.unlock();
                cv_.notify_all();
                throw TimeoutError("rank " + std::to_string(rank) + ": peers did not reach the collective within " +
                                   std::to_string(timeout.count()) + " ms");
            }
            cv_.wait(lk, moved_on);  // a leader is at work on this collective: it ends when the leader does
        }
    }
    if (!moved_on() && broken_.load(std::memory_order_acquire))
        throw TimeoutError("rank " + std::to_string(rank) + ": a peer timed out in this collective");
    // generation advanced by exactly one: the error (if any) belongs to our collective
    if (last_error_) std::rethrow_exception(last_error_);
}

void LocalMesh::post(int src, int dst, Parcel p) {
    MCCL_CHECK(src >= 0 && src < world_ && dst >= 0 && dst < world_, "rank outside the mesh");
    {
        std::lock_guard<std::mutex> lk(box_mu_);
        boxes_[static_cast<size_t>(src) * static_cast<size_t>(world_) + static_cast<size_t>(dst)].push_back(std::move(p));
    }
    box_cv_.notify_all();
}

Parcel LocalMesh::take(int src, int dst, std::chrono::milliseconds timeout) {
    MCCL_CHECK(src >= 0 && src < world_ && dst >= 0 && dst < world_, "rank outside the mesh");
    auto& box = boxes_[static_cast<size_t>(src) * static_cast<size_t>(world_) + static_cast<size_t>(dst)];
    std::unique_lock<std::mutex> lk(box_mu_);
    auto ready = [&] { return !box.empty(); };
    if (timeout.count() <= 0) {
        box_cv_.wait(lk, ready);
    } else if (!box_cv_.wait_for(lk, timeout, ready)) {
        throw TimeoutError("rank " + std::to_string(dst) + ": nothing arrived from rank " + std::to_string(src) +
                           " within " + std::to_string(timeout.count()) + " ms");
    }
    Parcel p = std::move(box.front());
    box.pop_front();
    return p;
}

void LocalMesh::wire_send(int src, int dst, const void* buf, size_t len, std::shared_ptr<void> keep) {
    MCCL_CHECK(src >= 0 && src < world_ && dst >= 0 && dst < world_ && src != dst, "wire: bad peer");
    MCCL_CHECK(buf != nullptr || len == 0, "wire: send from a null buffer");
    WireMessage m;
    m.len = len;
    if (keep) {
        m.data = buf;
        m.keep = std::move(keep);
    } else {
        m.owned.assign(static_cast<const uint8_t*>(buf), static_cast<const uint8_t*>(buf) + len);
        m.data = m.owned.data();
    }
    {
        std::lock_guard<std::mutex> lk(wire_mu_);
        auto& q = wires_[static_cast<size_t>(src) * static_cast<size_t>(world_) + static_cast<size_t>(dst)];
        q.push_back(std::move(m));
        // `owned` may have moved: its bytes are where the vector's storage is now
        if (!q.back().keep) q.back().data = q.back().owned.data();
    }
    wire_cv_.notify_all();
}

void LocalMesh::wire_recv(int src, int dst, void* buf, size_t len, std::chrono::milliseconds timeout) {
    MCCL_CHECK(src >= 0 && src < world_ && dst >= 0 && dst < world_ && src != dst, "wire: bad peer");
    auto& q = wires_[static_cast<size_t>(src) * static_cast<size_t>(world_) + static_cast<size_t>(dst)];
    WireMessage m;
    {
        std::unique_lock<std::mutex> lk(wire_mu_);
        auto ready = [&] { return !q.empty(); };
        if (timeout.count() <= 0) {
            wire_cv_.wait(lk, ready);
        } else if (!wire_cv_.wait_for(lk, timeout, ready)) {
            throw TimeoutError("rank " + std::to_string(dst) + ": no bytes from rank " + std::to_string(src) +
                               " within " + std::to_string(timeout.count()) + " ms");
        }
        m = std::move(q.front());
        q.pop_front();
        if (!m.keep) m.data = m.owned.data();
    }
    MCCL_CHECK(m.len == len, "wire: rank " + std::to_string(dst) + " expects " + std::to_string(len) +
                                 " bytes from rank " + std::to_string(src) + ", which sent " + std::to_string(m.len));
    if (len) std::memcpy(buf, m.data, len);  // the wire's delivery into the receiver's buffer
}

}  // namespace mccl
