// pg_stress.cpp -- the ownership side of the c10d backend under a sanitizer, without a GPU: the real
// ProcessGroupMCCL, WorkMCCL, Progress, LocalMesh, HostWire and chunk scheduler, compiled with
// -DMCCL_NULL_DEVICE (backend/Device.hpp) over a host stand-in of the kernel layer
// (null_mcclx.cpp).  Groups of 2-4 rank threads come and go; every second group completes its
// allreduces event-based (completer thread, two queues, parked buckets).  What the test is after
// is who lets go of what, where:
//   * the registry of meshes and shared contexts while ranks join and leave at different times;
//   * Works and Futures settled on the engine and completer threads;
//   * the LAST reference to a process group dropped by a Future callback on the group's own
//     engine thread, and on the mesh's completer thread -- the group, its engine, the shared
//     context and the completer are then destroyed from inside one of their own tasks.
// Results of the fp32 sums are checked, so that a buffer freed or reused too early shows up as
// a wrong value as well as a sanitizer report.  WAIT_MS = 0 makes every wait untimed (a timed
// wait is pthread_cond_clockwait, which ThreadSanitizer builds of this toolchain do not model).
#include <torch/csrc/distributed/c10d/HashStore.hpp>

#include <ATen/ATen.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "backend/ProcessGroupMCCL.hpp"

#ifndef WAIT_MS
#define WAIT_MS 0
#endif

using namespace mccl;

namespace {
std::atomic<long> g_bad{0}, g_checked{0};

void expect(const at::Tensor& t, float want) {
    const float* p = t.data_ptr<float>();
    for (int64_t i = 0; i < t.numel(); ++i)
        if (p[i] != want) {
            ++g_bad;
            return;
        }
    ++g_checked;
}

void settled(const c10::intrusive_ptr<c10d::Work>& w) { w->getFuture()->wait(); }  // untimed, and the Work has settled after it
}  // namespace

int main(int argc, char** argv) {
    const int groups = argc > 1 ? atoi(argv[1]) : 60;
    for (int g = 0; g < groups; ++g) {
        const int world = 2 + g % 3;
        const bool async = (g & 1) != 0;
        if (async)
            setenv("MCCL_ALLREDUCE_ASYNC", "1", 1);
        else
            unsetenv("MCCL_ALLREDUCE_ASYNC");
        if (g % 4 == 3)
            setenv("MCCL_ASYNC_QUEUES", "1", 1);
        else
            unsetenv("MCCL_ASYNC_QUEUES");
        auto store = c10::make_intrusive<c10d::HashStore>();
        const float total = world * (world + 1) / 2.0f;
        std::vector<std::thread> ts;
        for (int r = 0; r < world; ++r)
            ts.emplace_back([&, r] {
                ProcessGroupMCCL::Options opts;
                opts.timeout = std::chrono::milliseconds(WAIT_MS);
                auto pg = c10::make_intrusive<ProcessGroupMCCL>(store, r, world, opts);
                c10d::AllreduceOptions sum;
                // a few buckets back to back (in the event-based mode they park and coalesce)
                std::vector<std::vector<at::Tensor>> buckets;
                std::vector<c10::intrusive_ptr<c10d::Work>> works;
                for (int b = 0; b < 5; ++b) {
                    buckets.push_back({at::full({1000 + 37 * b}, float(r + 1))});
                    works.push_back(pg->allreduce(buckets.back(), sum));
                }
                for (int b = 4; b >= 0; --b) {
                    works[size_t(b)]->wait();
                    settled(works[size_t(b)]);
                    expect(buckets[size_t(b)][0], total);
                }
                works.clear();
                // engine-thread collectives
                at::Tensor mine = at::full({33}, float(r)), all = at::empty({33 * world});
                auto wg = pg->_allgather_base(all, mine);
                auto wb = pg->barrier();
                wg->wait();
                wb->wait();
                for (int p = 0; p < world; ++p)
                    if (all.data_ptr<float>()[33 * p] != float(p)) ++g_bad;
                // the last reference to the group goes with a Future callback: on the completer
                // thread (event-based allreduce) or on the group's own engine thread (barrier)
                std::vector<at::Tensor> last = {at::full({257}, float(r + 1))};
                c10::intrusive_ptr<c10d::Work> w = (g % 3 == 0) ? pg->barrier() : pg->allreduce(last, sum);
                auto fut = w->getFuture();
                fut->addCallback([keep = pg](c10::ivalue::Future&) {});
                pg.reset();   // this thread lets go first
                w.reset();
                fut->wait();
                if (g % 3 != 0) expect(last[0], total);
                fut.reset();  // whoever held the callback last has destroyed the group by now, or does so here
            });
        for (auto& t : ts) t.join();
    }
    if (g_bad.load()) {
        printf("FAILED: %ld wrong results\n", g_bad.load());
        return 1;
    }
    printf("ok: %d groups, %ld results checked\n", groups, g_checked.load());
    return 0;
}
