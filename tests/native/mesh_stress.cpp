// mesh_stress.cpp -- the host side of a process group's life under a sanitizer: groups of rank
// threads come and go, each rank with its FIFO engine; they meet in a LocalMesh on their own
// threads (the allreduce's path) and on their engine threads (every other collective's path),
// exchange a ring of messages over the byte transport, and tear everything down, the last
// rank to let go destroying the mesh.  WAIT_MS = 0 makes every wait untimed (a timed wait is
// pthread_cond_clockwait, which ThreadSanitizer builds of this toolchain do not model).
#include <atomic>
#include <cstdio>
#include <cstring>
#include <memory>
#include <thread>
#include <vector>
#include "backend/Errors.hpp"
#include "backend/LocalMesh.hpp"
#include "backend/Progress.hpp"
using namespace mccl;
#ifndef WAIT_MS
#define WAIT_MS 0
#endif
int main(int argc, char** argv) {
    const int groups = argc > 1 ? atoi(argv[1]) : 300;
    std::atomic<long> leaders{0};
    for (int g = 0; g < groups; ++g) {
        const int world = 2 + g % 3;
        const std::string key = LocalMesh::fresh_key();
        auto mesh = LocalMesh::create(key, world);
        std::vector<std::thread> ts;
        std::atomic<int> found{0};
        for (int r = 0; r < world; ++r)
            ts.emplace_back([&, r] {
                auto mine = LocalMesh::find(key);
                ++found;
                auto engine = std::make_unique<Progress>();
                LocalPeer peer(mine, r, std::chrono::milliseconds(WAIT_MS));
                for (int i = 0; i < 5; ++i) {
                    // a collective on the caller's thread
                    Contribution c; c.kind = i; c.numel = {uint64_t(r)};
                    mine->rendezvous(r, c, std::chrono::milliseconds(WAIT_MS), [&](const std::vector<Contribution>& all) {
                        for (int q = 0; q < world; ++q) if (all[q].numel[0] != uint64_t(q)) abort();
                        ++leaders;
                    });
                    // a collective on the engine thread
                    std::mutex mu; std::condition_variable cv; bool done = false;
                    engine->submit([&] {
                        Contribution d; d.kind = 100 + i; d.numel = {uint64_t(r)};
                        mine->rendezvous(r, d, std::chrono::milliseconds(WAIT_MS), [&](const std::vector<Contribution>&) { ++leaders; });
                        std::lock_guard<std::mutex> lk(mu); done = true; cv.notify_all();
                    });
                    { std::unique_lock<std::mutex> lk(mu); cv.wait(lk, [&] { return done; }); }
                    while (!engine->idle()) std::this_thread::yield();
                    // wire ring
                    uint8_t out[64], in[64]; memset(out, r + i, sizeof out);
                    peer.send((r + 1) % world, out, sizeof out);
                    peer.recv((r + world - 1) % world, in, sizeof in);
                    if (in[0] != uint8_t((r + world - 1) % world + i)) abort();
                }
                engine->shutdown();
                engine.reset();
                mine.reset();
                LocalMesh::forget(key);
            });
        while (found.load() < world) std::this_thread::yield();
        mesh.reset();   // the last rank to let go destroys the mesh, as in the process group
        for (auto& t : ts) t.join();
    }
    printf("ok: %d groups, %ld leader runs\n", groups, leaders.load());
    return 0;
}
