#include "backend/ProcessGroupMCCL.hpp"

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <tuple>

#include "backend/Device.hpp"
#include "backend/Errors.hpp"
#include "backend/HostWire.hpp"
#include "backend/LocalMesh.hpp"
#include "backend/Logging.hpp"
#include "backend/Phases.hpp"
#include "backend/Progress.hpp"
#include "backend/WorkMCCL.hpp"

namespace mccl {

namespace {

enum Kind { K_ALLREDUCE = 1, K_BROADCAST, K_ALLGATHER_BASE, K_ALLGATHER, K_REDUCE_SCATTER_BASE,
            K_REDUCE_SCATTER, K_BARRIER, K_ALLTOALL_BASE, K_ALLTOALL };

c10::intrusive_ptr<c10d::Work> make_completed(c10d::OpType op, std::vector<at::Tensor> outputs,
                                              const char* title) {
    auto w = c10::make_intrusive<WorkMCCL>(op, std::move(outputs), title);
    w->finish();
    return w;
}

// check_mps_ (ProcessGroupMCCL.cpp:72-79) for ROCm tensors.
void check_gpu_(const at::Tensor& t, const char* op) {
    MCCL_CHECK(dev::on_device(t), std::string(op) + ": MCCL on MI355X is GPU-only; got " +
                                std::string(c10::DeviceTypeName(t.device().type())) + " tensor");
    MCCL_CHECK(t.is_contiguous(), std::string(op) + ": tensor must be contiguous");
}

// dtypes the reduce kernels cover (shaders.metal: f32 / f16 / bf16); -1 otherwise.
int reduce_dtype(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kFloat: return MCCLX_F32;
        case at::kHalf: return MCCLX_F16;
        case at::kBFloat16: return MCCLX_BF16;
        default: return -1;
    }
}

int need_reduce_dtype(const at::Tensor& t, const char* op) {
    int d = reduce_dtype(t);
    // select_op_pipeline returns nil -> "No Metal pipeline for dtype" (MetalKernels.mm:634-635)
    MCCL_CHECK(d >= 0, std::string(op) + ": No HIP kernel for dtype " + std::string(at::toString(t.scalar_type())));
    return d;
}

int reduce_op_code(const c10d::ReduceOp& op) {
    switch (static_cast<c10d::ReduceOp::RedOpType>(op)) {
        case c10d::ReduceOp::SUM: return MCCLX_SUM;
        case c10d::ReduceOp::AVG: return MCCLX_AVG;
        case c10d::ReduceOp::PRODUCT: return MCCLX_PRODUCT;
        case c10d::ReduceOp::MIN: return MCCLX_MIN;
        case c10d::ReduceOp::MAX: return MCCLX_MAX;
        default:
            // MetalKernels.mm:546-548
            throw MCCLError("Unsupported ReduceOp: " +
                            std::to_string(static_cast<int>(static_cast<c10d::ReduceOp::RedOpType>(op))));
    }
}

}  // namespace

namespace {
// torch's caching allocator hands out blocks whose earlier users may still be
// running on the stream the block belongs to (the allocating thread's current
// stream); the reduce queue is another stream, so it waits for that one before
// it touches a fresh block.
void order_after_allocator(mcclx_ctx* ctx, int device) {
    check_rc(mcclx_queue_wait_stream(ctx, dev::current_stream(device)));
}
}  // namespace

// One reduce queue and one grow-only scratch buffer per mesh (per group of
// ranks sharing the GPU).  The scratch replaces the reference's per-call
// at::empty recv buffers (ProcessGroupMCCL.cpp:152-162).
struct ProcessGroupMCCL::Shared : std::enable_shared_from_this<ProcessGroupMCCL::Shared> {
    mcclx_ctx* ctx = nullptr;
    at::Tensor scratch;
    int device = 0;

    // Recorded allreduces.  A DDP bucket is reduced again and again at the same
    // addresses; from its second occurrence on, the launches of one allreduce
    // (encode, fold, decode/copy legs) are recorded into a HIP graph and replayed
    // with one submission, which removes the host's launch gaps between them.
    // The key is everything the launches depend on; MCCL_GRAPH_CACHE=0 turns it off.
    struct GraphKey {
        int world, algo, op, dtype, wire, mode;
        uint64_t numel;
        void* workspace;
        std::vector<void*> tensors;
        bool operator<(const GraphKey& o) const {
            return std::tie(world, algo, op, dtype, wire, mode, numel, workspace, tensors) <
                   std::tie(o.world, o.algo, o.op, o.dtype, o.wire, o.mode, o.numel, o.workspace, o.tensors);
        }
    };
    struct GraphEntry {
        mcclx_graph* graph = nullptr;
        uint64_t seen = 0, last_use = 0;
        uint64_t launches = 0;  // kernel launches of its first, eager issue
    };
    // Replaying a recorded graph costs the host about 22 us whatever it holds, an eager
    // launch 3.5 us: only an allreduce of this many launches or more is recorded
    // (MCCL_GRAPH_MIN_LAUNCHES; a sum of up to eight ranks is one or two launches).
    uint64_t graph_min_launches = 6;
    static constexpr size_t kMaxGraphs = 256;
    std::map<GraphKey, GraphEntry> graphs;
    uint64_t use_clock = 0;
    uint64_t graph_hits = 0;
    bool graphs_enabled = true;

    // Event-based completion (MCCL_ALLREDUCE_ASYNC=1).  An allreduce of the group
    // becomes a Bucket.  Buckets go to two reduce queues in turn (two contexts, two
    // streams: `ctx` and `alt`), so that one bucket's ramp-up runs in the other's drain
    // and the gap between dependent launches is hidden (a 25 MiB allreduce: 46 -> 39 us
    // per bucket on the device).  Each queue holds up to two launches; what arrives for
    // a queue that is full is parked, and everything parked for it goes out together --
    // one launch per phase for all of it -- as soon as one of its launches has finished
    // (or a rank waits on one of the parked Works).  A worker thread waits for each
    // launch's completion ticket, issues what is parked and settles the ranks' Works.
    // MCCL_ASYNC_QUEUES=1 keeps everything on one queue.
    //
    // Order between the queues is kept where it matters: a launch whose buffers overlap
    // those of an unfinished launch (or of an earlier parked bucket) on the other queue
    // waits for it on the device; every other use of the main queue (the synchronous
    // allreduce, all other collectives) first issues what is parked and lets the main
    // queue wait for the second one, and the second queue's next launch waits for the
    // main queue in turn.
    struct Span {
        uintptr_t lo, hi;
    };
    struct Bucket {
        std::vector<mcclx_replay> reps;
        std::vector<std::vector<void*>> ptrs;  // reps[i].tensors points into ptrs[i]
        at::Tensor workspace;                  // wire copies / recv scratch of this call
        std::vector<c10::intrusive_ptr<WorkMCCL>> works;  // one per rank
        std::atomic<bool> launched{false};
        std::atomic<uint64_t> flight{0};       // id of the launch that carries it (ids grow with every launch of the mesh)
        int queue = 0;
        bool small = false;                    // below MCCL_COALESCE_BELOW: see submit_bucket
        uint64_t arrival = 0;
        std::vector<Span> spans;               // every byte range the launch reads or writes
    };
    struct Flight {
        uint64_t id;
        std::vector<Span> spans;
    };
    static constexpr size_t kPooledWorkspaces = 16;
    std::mutex amu;
    mcclx_ctx* alt = nullptr;                    // the second queue, made when first needed (under amu)
    int queues = 2;
    std::deque<std::shared_ptr<Bucket>> parked[2];
    std::deque<Flight> flights[2];               // launches not yet seen to finish (by the completer: it is
                                                 // blocked in a wait on the newest event, and a query from
                                                 // another thread would block with it)
    uint64_t arrivals = 0, next_flight = 1;
    uint64_t newest_flight[2] = {0, 0};          // the last launch enqueued on each queue
    bool main_touched = true;                    // the main queue got work the second queue has not waited for
    std::vector<at::Tensor> workspace_pool;      // workspaces of finished buckets, for reuse
    std::unique_ptr<Progress> completer;
    std::atomic<uint64_t> async_launches{0}, async_buckets{0};

    Shared() {
        const char* e = std::getenv("MCCL_GRAPH_CACHE");
        graphs_enabled = !(e && e[0] == '0');
        if (const char* m = std::getenv("MCCL_GRAPH_MIN_LAUNCHES")) graph_min_launches = std::strtoull(m, nullptr, 10);
        const char* q = std::getenv("MCCL_ASYNC_QUEUES");
        if (q && q[0] == '1') queues = 1;
        if (const char* c = std::getenv("MCCL_COALESCE_BELOW")) coalesce_below = std::strtoull(c, nullptr, 10);
    }
    ~Shared() {
        try {
            std::lock_guard<std::mutex> lk(amu);
            flush_locked(0);  // their completion tasks must be queued before the worker closes
            flush_locked(1);
        } catch (...) {
        }
        if (completer) completer->shutdown();  // settles what is still in flight
        workspace_pool.clear();
        drop_graphs();
        if (drain_word.host && ctx) {
            (void)mcclx_queue_drain(ctx);  // the last copy into the word has landed
            (void)mcclx_host_free(ctx, drain_word.host);
        }
        if (alt) mcclx_destroy(alt);
        if (ctx) mcclx_destroy(ctx);
    }

    static constexpr size_t kDepth = 2;  // launches in flight per queue: the next one is behind the one that runs

    // Small buckets.  A launch of a 1 MiB bucket keeps the device busy for under 3 us (15 % of
    // what the memory system can do: a launch's fixed cost dominates), four of them in one
    // launch for 4 us.  A bucket of fewer bytes than this (per rank; MCCL_COALESCE_BELOW,
    // default 8 MiB, 0 = off) therefore goes out at once only when its queue is empty; while
    // ANY launch of that queue is still in flight it is parked, and everything parked goes out
    // as one launch when that one has finished (or a rank waits for one of them) -- the window
    // in which buckets gather is the time the completer needs to see a launch end, some 20 us.
    // Small buckets all take the main queue: two queues would halve what gathers on either.
    uint64_t coalesce_below = 8ull << 20;

    // Which queue the next event-based allreduce goes to, and that queue.
    mcclx_ctx* pick_queue(int* q, bool small) {
        std::lock_guard<std::mutex> lk(amu);
        *q = (queues == 2 && !small) ? static_cast<int>(arrivals & 1) : 0;
        if (*q == 1 && !alt) check_rc(mcclx_init(device, &alt));
        return *q ? alt : ctx;
    }
    mcclx_ctx* queue(int q) const { return q ? alt : ctx; }
    uint64_t newest_on(int q) {
        std::lock_guard<std::mutex> lk(amu);
        return newest_flight[q];
    }

    // A workspace for one asynchronous call (several may be in flight, each keeps its
    // own until it has finished).  One that comes back from a finished bucket has no
    // user left on any queue and needs no ordering against the allocator.
    at::Tensor take_workspace(uint64_t nbytes, mcclx_ctx* on) {
        {
            std::lock_guard<std::mutex> lk(amu);
            size_t best = workspace_pool.size();
            for (size_t i = 0; i < workspace_pool.size(); ++i) {
                const auto n = static_cast<uint64_t>(workspace_pool[i].numel());
                if (n >= nbytes && n <= 2 * nbytes + (1u << 20) &&
                    (best == workspace_pool.size() || n < static_cast<uint64_t>(workspace_pool[best].numel())))
                    best = i;
            }
            if (best != workspace_pool.size()) {
                at::Tensor t = std::move(workspace_pool[best]);
                workspace_pool.erase(workspace_pool.begin() + static_cast<std::ptrdiff_t>(best));
                return t;
            }
        }
        at::Tensor t = dev::empty_bytes(static_cast<int64_t>(nbytes), device);
        order_after_allocator(on, device);
        return t;
    }

    static bool overlap(const std::vector<Span>& a, const std::vector<Span>& b) {
        for (const Span& x : a)
            for (const Span& y : b)
                if (x.lo < y.hi && y.lo < x.hi) return true;
        return false;
    }

    // Caller holds amu.  Issues the buckets as ONE list replay on queue q and hands
    // their Works to the completer.
    void launch_locked(int q, std::vector<std::shared_ptr<Bucket>> buckets) {
        std::vector<mcclx_replay> all;
        std::vector<Span> spans;
        uint64_t first_arrival = ~0ull;
        for (auto& b : buckets) {
            all.insert(all.end(), b->reps.begin(), b->reps.end());
            spans.insert(spans.end(), b->spans.begin(), b->spans.end());
            first_arrival = std::min(first_arrival, b->arrival);
        }
        std::exception_ptr err;
        uint64_t ticket = 0;
        try {
            const int o = 1 - q;
            if (alt) {
                // an earlier bucket still parked for the other queue that touches the same
                // memory goes first ...
                bool earlier = false;
                for (auto& pb : parked[o]) earlier = earlier || (pb->arrival < first_arrival && overlap(pb->spans, spans));
                if (earlier) flush_locked(o);
                // ... and this queue waits for the other queue's unfinished launches that do
                bool wait_other = false;
                for (const Flight& f : flights[o]) wait_other = wait_other || overlap(f.spans, spans);
                if (q == 1 && main_touched) {
                    wait_other = true;
                    main_touched = false;
                }
                if (wait_other) check_rc(mcclx_queue_wait_stream(queue(q), mcclx_queue_stream(queue(o))));
            }
            // an event-based launch runs beside whatever the ranks enqueue next and beside the
            // other queue's launches, and a launch that does not have the memory system to
            // itself should not time its stores (mcclx_set_hold; measured beside a stream of
            // copies: 27.7 us with the hold form, 24.1 us without)
            check_rc(mcclx_set_hold(queue(q), 0));
            {
                phases::Span ph(phases::kLaunch);
                check_rc(mcclx_allreduce_replay_many(queue(q), all.data(), static_cast<uint32_t>(all.size())));
            }
            phases::Span ph(phases::kSubmit);
            check_rc(mcclx_event_record(queue(q), &ticket));
        } catch (...) {
            err = std::current_exception();
        }
        const uint64_t id = next_flight++;
        if (!err) newest_flight[q] = id;
        // only now: a rank that waits on one of these Works and finds it not launched takes
        // `amu` (flush_parked) and so gets behind this launch before it orders its stream
        for (auto& b : buckets) {
            b->flight = id;
            b->launched = true;
        }
        if (err) {
            for (auto& b : buckets)
                for (auto& w : b->works) w->finishWithException(err);
            std::rethrow_exception(err);
        }
        flights[q].push_back(Flight{id, std::move(spans)});
        ++async_launches;
        async_buckets += buckets.size();
        phases::Span ph_submit(phases::kSubmit);
        if (!completer) completer = std::make_unique<Progress>();
        mcclx_ctx* c = queue(q);
        // The task keeps this object alive while it runs: settling a Work runs the callbacks of
        // its Future, and one of them may drop the last process group of the mesh.  The object
        // then goes when the task's captures do, with nothing of it in use up the stack (its
        // destructor shuts the completer down from the completer's own thread, which the engine
        // allows).  From the destructor itself there is no owner left to share with: it waits
        // for these tasks before it goes on.
        std::shared_ptr<Shared> self = weak_from_this().lock();
        completer->submit([this, self, c, q, id, ticket, buckets = std::move(buckets)]() mutable {
            std::exception_ptr failure;
            {
                phases::Span ph(phases::kCompleterWait);
                try {
                    check_rc(mcclx_event_wait(c, ticket));
                } catch (...) {
                    failure = std::current_exception();
                }
            }
            phases::Span ph_settle(phases::kSettle);
            {
                std::lock_guard<std::mutex> lk(amu);
                for (auto it = flights[q].begin(); it != flights[q].end(); ++it)
                    if (it->id == id) {
                        flights[q].erase(it);
                        break;
                    }
                try {
                    flush_locked(q);  // first: the queue should not run dry while Works are settled
                } catch (...) {
                    // the Works carry the error
                }
            }
            for (auto& b : buckets)
                for (auto& w : b->works) {
                    if (failure)
                        w->finishWithException(failure);
                    else
                        w->finish();
                }
            {
                std::lock_guard<std::mutex> lk(amu);
                for (auto& b : buckets)
                    if (b->workspace.defined() && workspace_pool.size() < kPooledWorkspaces)
                        workspace_pool.push_back(std::move(b->workspace));
            }
            buckets.clear();  // what the pool did not take goes back to the allocator only now
        });
    }

    void submit_bucket(std::shared_ptr<Bucket> b) {
        std::lock_guard<std::mutex> lk(amu);
        b->arrival = arrivals++;
        const int q = b->queue;
        // (a launch that finishes after this check takes `amu` after us and finds the bucket parked)
        if (parked[q].empty() && flights[q].size() < (b->small ? size_t(1) : kDepth)) {
            launch_locked(q, {std::move(b)});
            return;
        }
        parked[q].push_back(std::move(b));
    }

    // Caller holds amu.
    void flush_locked(int q) {
        if (parked[q].empty()) return;
        std::vector<std::shared_ptr<Bucket>> go(parked[q].begin(), parked[q].end());
        parked[q].clear();
        launch_locked(q, std::move(go));
    }
    void flush_parked(int q) {
        std::lock_guard<std::mutex> lk(amu);
        try {
            flush_locked(q);
        } catch (...) {
            // the Works carry the error
        }
    }

    // Before any other device work on the main queue: what the event-based mode still
    // holds back goes out first (program order), and the main queue waits for the
    // second queue's launches.
    void begin_main_work() {
        std::lock_guard<std::mutex> lk(amu);
        try {
            flush_locked(0);
            flush_locked(1);
        } catch (...) {
            // the Works carry the error
        }
        main_touched = true;
        if (alt && !flights[1].empty()) check_rc(mcclx_queue_wait_stream(ctx, mcclx_queue_stream(alt)));
        // what follows waits for the ranks' streams and is drained before anyone goes on:
        // it has the GPU to itself
        check_rc(mcclx_set_hold(ctx, 1));
    }

    // The drain of a synchronous allreduce.  hipStreamSynchronize hands the host back 9-10 us
    // after the launch's last wave has gone (the completion signal's way through the runtime);
    // a 4-byte copy queued behind the launch that writes a number into pinned host memory,
    // and a host that watches that word, gets there 4 us sooner (a 26 us launch: 36.2 -> 32.2 us
    // from launch call to return).  The copy is issued while the launch runs, so its own launch
    // cost is hidden.  The word only says that the queue has got that far: the results are in
    // device memory, where the ranks' next kernels (launched after this returns) find them,
    // exactly as after the blocking drain.  If the word has not come after MCCL_DRAIN_SPIN_US
    // (default 1000; 0 = always the blocking drain) the blocking drain takes over, which is also
    // what reports a launch that failed.  Caller is the last arrival of a collective (one at a time).
    struct DrainWord {
        void* host = nullptr;       // pinned: the word at offset 0, the numbers 1..kNumbers from offset 1024 on
        void* alias = nullptr;      // the same memory as the device addresses it
        at::Tensor numbers;         // the numbers again, in device memory (the copy's source)
        uint32_t next = 0;
        long spin_us = -1;
        static constexpr uint32_t kNumbers = 512;
    } drain_word;
    void drain_main() {
#ifdef MCCL_NULL_DEVICE
        check_rc(mcclx_queue_drain(ctx));  // (the host stand-in of the queue has no device to write the word)
#else
        DrainWord& w = drain_word;
        if (w.spin_us < 0) {
            const char* e = std::getenv("MCCL_DRAIN_SPIN_US");
            w.spin_us = e ? std::strtol(e, nullptr, 10) : 1000;
            if (w.spin_us < 0) w.spin_us = 0;
            if (w.spin_us > 0) {
                try {
                    check_rc(mcclx_host_alloc(ctx, 4096, &w.host, &w.alias));
                    auto* h = static_cast<uint32_t*>(w.host);
                    h[0] = 0;
                    for (uint32_t i = 0; i < DrainWord::kNumbers; ++i) h[256 + i] = i + 1;
                    w.numbers = dev::empty_bytes(4 * DrainWord::kNumbers, device);
                    order_after_allocator(ctx, device);
                    check_rc(mcclx_copy(ctx, w.numbers.data_ptr(), static_cast<char*>(w.alias) + 1024, 4 * DrainWord::kNumbers));
                    check_rc(mcclx_queue_drain(ctx));
                } catch (const std::exception& e) {  // no pinned memory to be had: the blocking drain serves
                    MCCL_WARN("the synchronous allreduce keeps the blocking drain: %s", e.what());
                    if (w.host) (void)mcclx_host_free(ctx, w.host);
                    w.host = w.alias = nullptr;
                    w.numbers = at::Tensor();
                    w.spin_us = 0;
                }
            }
        }
        if (w.spin_us == 0) {
            check_rc(mcclx_queue_drain(ctx));
            return;
        }
        const uint32_t i = w.next++ % DrainWord::kNumbers;
        check_rc(mcclx_copy(ctx, w.alias, static_cast<char*>(w.numbers.data_ptr()) + 4 * i, 4));
        const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(w.spin_us);
        const volatile uint32_t* word = static_cast<const volatile uint32_t*>(w.host);
        for (;;) {
            for (int k = 0; k < 64; ++k) {
                if (*word == i + 1) {
                    std::atomic_thread_fence(std::memory_order_acquire);
                    return;
                }
                __builtin_ia32_pause();
            }
            if (std::chrono::steady_clock::now() >= until) break;
        }
        check_rc(mcclx_queue_drain(ctx));
#endif
    }

    // Host-blocking: nothing of the event-based mode is left on the device.
    void quiesce() {
        begin_main_work();
        check_rc(mcclx_queue_drain(ctx));
    }
    void drop_graphs() {
        for (auto& kv : graphs)
            if (kv.second.graph) (void)mcclx_graph_destroy(ctx, kv.second.graph);
        graphs.clear();
    }
    void* workspace(uint64_t nbytes) {
        if (nbytes == 0) return nullptr;
        if (!scratch.defined() || static_cast<uint64_t>(scratch.numel()) < nbytes + 256) {
            check_rc(mcclx_queue_drain(ctx));  // nothing may still read the old buffer
            drop_graphs();                     // recorded launches point into it
            scratch = dev::empty_bytes(static_cast<int64_t>(nbytes + 256), device);
            order_after_allocator(ctx, device);
        }
        auto p = reinterpret_cast<uintptr_t>(scratch.data_ptr());
        return reinterpret_cast<void*>((p + 255) / 256 * 256);
    }

    // One allreduce of the group: issued launch by launch and counted the first time;
    // one of many launches is recorded on its second occurrence and replayed from then on.
    void allreduce(const mcclx_replay& rp) {
        if (!graphs_enabled) {
            check_rc(mcclx_allreduce_replay(ctx, &rp));
            return;
        }
        GraphKey key{rp.world, rp.algo, rp.op, rp.dtype, rp.wire_bf16, rp.mode, rp.numel, rp.workspace,
                     std::vector<void*>(rp.tensors, rp.tensors + rp.world)};
        GraphEntry& e = graphs[key];
        e.last_use = ++use_clock;
        ++e.seen;
        if (e.seen == 1) {  // issued eagerly, and counted
            const uint64_t before = mcclx_launch_count(ctx);
            check_rc(mcclx_allreduce_replay(ctx, &rp));
            e.launches = mcclx_launch_count(ctx) - before;
            if (graphs.size() > kMaxGraphs) evict();
            return;
        }
        if (!e.graph && e.launches >= graph_min_launches) {
            check_rc(mcclx_graph_begin(ctx));
            int rc = mcclx_allreduce_replay(ctx, &rp);
            std::string why = rc == MCCLX_OK ? "" : mcclx_last_error();
            mcclx_graph* g = nullptr;
            int rc_end = mcclx_graph_end(ctx, &g);
            if (rc != MCCLX_OK) {
                if (g) (void)mcclx_graph_destroy(ctx, g);
                throw KernelError(why);
            }
            check_rc(rc_end);
            e.graph = g;
            MCCL_DEBUG("allreduce recorded: world %d algo %d op %d dtype %d wire %d numel %llu (%zu graphs kept)",
                       rp.world, rp.algo, rp.op, rp.dtype, rp.wire_bf16, (unsigned long long)rp.numel, graphs.size());
        }
        if (e.graph) {
            check_rc(mcclx_graph_launch(ctx, e.graph));
            ++graph_hits;
        } else {
            check_rc(mcclx_allreduce_replay(ctx, &rp));
        }
        if (graphs.size() > kMaxGraphs) evict();
    }
    void evict() {  // drop the least recently used half
        std::vector<std::pair<uint64_t, const GraphKey*>> order;
        for (auto& kv : graphs) order.emplace_back(kv.second.last_use, &kv.first);
        std::sort(order.begin(), order.end());
        std::vector<GraphKey> victims;
        for (size_t i = 0; i < order.size() / 2; ++i) victims.push_back(*order[i].second);
        for (auto& k : victims) {
            auto it = graphs.find(k);
            if (it->second.graph) (void)mcclx_graph_destroy(ctx, it->second.graph);
            graphs.erase(it);
        }
    }
};

namespace {
std::mutex g_shared_mu;
std::map<std::string, std::weak_ptr<void>> g_shared;  // mesh key -> Shared (type-erased)
}  // namespace

ProcessGroupMCCL::ProcessGroupMCCL(c10::intrusive_ptr<c10d::Store> store, int rank, int size, Options opts)
    : c10d::Backend(rank, size), store_(std::move(store)), opts_(opts) {
    MCCL_CHECK(rank >= 0 && rank < size, "rank/size invalid");
    try {
        device_ = dev::current_device();
    } catch (const std::exception& e) {
        // the reference fails in metal_kernels_init() when there is no Metal device
        throw MCCLError(std::string("no usable GPU for the mccl backend: ") + e.what());
    }
    if (size == 1) {
        // metal_kernels_init() (ProcessGroupMCCL.cpp:93): fails loudly without a GPU
        shared_ = std::make_shared<Shared>();
        shared_->device = device_;
        check_rc(mcclx_init(device_, &shared_->ctx));
        ctx_ = shared_->ctx;
        return;
    }
    // Rendezvous through the store (the reference exchanges TCP endpoints here,
    // runtime/Rendezvous.cpp:23-79): rank 0 publishes the key of the in-process mesh.
    const std::string store_key = "mccl/local_mesh";
    if (rank == 0) {
        mesh_key_ = LocalMesh::fresh_key();
        mesh_ = LocalMesh::create(mesh_key_, size);
        auto sh = std::make_shared<Shared>();
        sh->device = device_;
        check_rc(mcclx_init(device_, &sh->ctx));
        {
            std::lock_guard<std::mutex> lk(g_shared_mu);
            g_shared[mesh_key_] = sh;
        }
        shared_ = sh;
        store_->set(store_key, std::vector<uint8_t>(mesh_key_.begin(), mesh_key_.end()));
    } else {
        auto raw = store_->get(store_key);  // blocks until rank 0 has set it (store timeout applies)
        mesh_key_.assign(raw.begin(), raw.end());
        mesh_ = LocalMesh::find(mesh_key_);
        MCCL_CHECK(mesh_ != nullptr,
                   "rank 0 of this group is not in this process: this build runs all ranks of a "
                   "group in one process on one GPU");
        MCCL_CHECK(mesh_->world() == size, "mesh size differs from group size");
        std::lock_guard<std::mutex> lk(g_shared_mu);
        shared_ = std::static_pointer_cast<Shared>(g_shared[mesh_key_].lock());
        MCCL_CHECK(shared_ != nullptr, "mesh context already destroyed");
    }
    ctx_ = shared_->ctx;
    wait_marks_ = std::make_shared<WaitMarks>();
    engine_ = std::make_unique<Progress>();
    MCCL_INFO("rank %d of %d joined in-process mesh %s on GPU %d (%d CUs)", rank, size, mesh_key_.c_str(), device_,
              mcclx_device_cus(ctx_));
}

ProcessGroupMCCL::~ProcessGroupMCCL() {
    // (shutdown runs what is queued; called on the engine's own thread -- a callback there
    // dropped the last reference to this group -- it does so in place instead of joining)
    if (engine_) engine_->shutdown();
    host_wire_.reset();
    mesh_.reset();
    shared_.reset();
    if (!mesh_key_.empty()) {
        LocalMesh::forget(mesh_key_);
        std::lock_guard<std::mutex> lk(g_shared_mu);
        auto it = g_shared.find(mesh_key_);
        if (it != g_shared.end() && it->second.expired()) g_shared.erase(it);  // the last rank of the mesh
    }
}

uint64_t ProcessGroupMCCL::graphHits() const { return shared_ ? shared_->graph_hits : 0; }
std::pair<uint64_t, uint64_t> ProcessGroupMCCL::asyncStats() const {
    if (!shared_) return {0, 0};
    return {shared_->async_launches.load(), shared_->async_buckets.load()};
}
uint64_t ProcessGroupMCCL::launchCount() const {
    if (!ctx_) return 0;
    uint64_t n = mcclx_launch_count(ctx_);
    if (shared_) {
        std::lock_guard<std::mutex> lk(shared_->amu);
        if (shared_->alt) n += mcclx_launch_count(shared_->alt);
    }
    return n;
}
std::vector<double> ProcessGroupMCCL::wireStats() const {
    if (!host_wire_) return {};
    const HostWire::Stats& s = host_wire_->stats();
    return {static_cast<double>(s.calls), static_cast<double>(s.fold_elems), static_cast<double>(s.fold_peer_bytes),
            static_cast<double>(s.fold_hbm_bytes), s.fold_ms, static_cast<double>(s.wire_bytes_sent),
            s.leg_ms[0], s.leg_ms[1], s.leg_ms[2], s.leg_ms[3], s.leg_ms[4]};
}

void* ProcessGroupMCCL::my_stream() const {
    return dev::current_stream(device_);
}

void ProcessGroupMCCL::meet(Contribution c, const LocalMesh::Leader& leader) {
    mesh_->rendezvous(getRank(), std::move(c), opts_.timeout, leader);
}

// Builds this rank's contribution and meets the peers.  A rank whose own
// argument checks fail still arrives, carrying the message, so that the whole
// group fails at once (in the reference such a rank simply never sends and its
// peers block on their sockets).
void ProcessGroupMCCL::meet_built(int kind, void* stream, const std::function<void(Contribution&)>& build,
                                  const LocalMesh::Leader& leader) {
    Contribution c;
    try {
        build(c);
    } catch (const std::exception& e) {
        c = Contribution{};
        c.error = e.what();
    }
    c.kind = kind;
    c.stream = stream;
    meet(std::move(c), leader);
}

// The allreduce runs on the caller's thread while every other collective runs
// on the engine thread (as in the reference); a rank must not enter the
// allreduce's meeting point while its own engine still owes an earlier
// collective, or the ranks would meet in different collectives.
void ProcessGroupMCCL::flush_engine_() {
    if (!engine_ || engine_->idle()) return;  // only this thread submits: nothing can slip in behind the check
    std::mutex mu;
    std::condition_variable cv;
    bool done = false;
    engine_->submit([&] {
        std::lock_guard<std::mutex> lk(mu);
        done = true;
        cv.notify_all();
    });
    BlockingRegion unlocked;
    std::unique_lock<std::mutex> lk(mu);
    cv.wait(lk, [&] { return done; });
}

namespace {

// Asynchronous shell of the reference (async_submit_, ProcessGroupMCCL.cpp:45-70):
// the issuing thread orders the reduce queue after its own stream (the
// reference records an event on torch's stream there), the engine thread runs
// the body and completes the Work; the sync callback drains the queue first.
c10::intrusive_ptr<c10d::Work> async_submit_(Progress& engine, mcclx_ctx* ctx, void* issuing_stream,
                                             c10d::OpType op, std::vector<at::Tensor> outputs,
                                             const char* title, std::function<void()> body) {
    auto work = c10::make_intrusive<WorkMCCL>(op, std::move(outputs), title);
    try {
        check_rc(mcclx_queue_wait_stream(ctx, issuing_stream));
    } catch (...) {
        work->finishWithException(std::current_exception());
        return work;
    }
    work->setSyncCallback([ctx] { check_rc(mcclx_queue_drain(ctx)); });
    engine.submit([work, ctx, title, body = std::move(body)]() mutable {
        try {
            body();
            // The captured tensors go back before anyone is told the work is done -- but not
            // before the device has finished with them: a block freed here belongs to the
            // stream it was allocated on, the launches ran on the reduce queue, and torch's
            // allocator would hand the block to the next request on that stream at once.
            check_rc(mcclx_queue_drain(ctx));
            body = nullptr;
            work->finish();
        } catch (...) {
            body = nullptr;
            try {
                throw;
            } catch (const std::exception& e) {
                MCCL_ERROR("%s failed: %s", title, e.what());
            } catch (...) {
                MCCL_ERROR("%s failed with a non-standard exception", title);
            }
            work->finishWithException(std::current_exception());
        }
    });
    return work;
}

bool env_wire_bf16() {
    const char* w = std::getenv("MCCL_WIRE_DTYPE");  // re-read on every call (ProcessGroupMCCL.cpp:117-120)
    return w && std::strcmp(w, "bf16") == 0;
}

int64_t env_tree_below() {
    const char* e = std::getenv("MCCL_TREE_BELOW");  // :138-139
    return e ? static_cast<int64_t>(std::strtoull(e, nullptr, 10)) : -1;
}

}  // namespace

namespace {
bool env_async_allreduce() {
    const char* e = std::getenv("MCCL_ALLREDUCE_ASYNC");  // re-read on every call, like the other knobs
    return e && e[0] == '1';
}
bool env_direct() {
    const char* e = std::getenv("MCCL_DIRECT");
    return !(e && e[0] == '0');
}
// MCCL_WIRE: unset / "device" = peers' chunks are read where they lie in HBM;
// "host" = through pinned, device-mapped host memory; "staged" = through the staging pool.
int env_transport() {
    const char* e = std::getenv("MCCL_WIRE");
    if (!e || !*e || std::strcmp(e, "device") == 0) return 0;
    if (std::strcmp(e, "host") == 0) return 1;
    if (std::strcmp(e, "staged") == 0) return 2;
    throw MCCLError(std::string("MCCL_WIRE=") + e + " is not one of device, host, staged");
}
}  // namespace

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::allreduce(std::vector<at::Tensor>& tensors,
                                                           const c10d::AllreduceOptions& opts) {
    if (getSize() == 1) return make_completed(c10d::OpType::ALLREDUCE, tensors, "mccl:allreduce");
    phases::Span ph_build(phases::kBuild);
    const int world = getSize();
    int transport = 0;
    bool async = false;
    std::string knob_error;
    try {
        transport = env_transport();
        async = transport == 0 && env_async_allreduce();  // the wire modes are synchronous, like the reference
    } catch (const std::exception& e) {
        knob_error = e.what();
    }
    c10::intrusive_ptr<WorkMCCL> work;
    if (async) {
        phases::Span ph(phases::kWorkMake);
        work = c10::make_intrusive<WorkMCCL>(c10d::OpType::ALLREDUCE, tensors, "mccl:allreduce");
    }

    // A rank whose own checks fail still goes to the meeting point, carrying the
    // message, so that the whole group fails at once instead of waiting for it.
    Contribution c;
    try {
        if (!knob_error.empty()) throw MCCLError(knob_error);
        MCCL_CHECK(!tensors.empty(), "allreduce: empty tensor list");
        const int op = reduce_op_code(opts.reduceOp);
        const bool wire = env_wire_bf16();
        const char* env_alg = std::getenv("MCCL_ALLREDUCE_ALGO");
        const int64_t tree_below = env_tree_below();
        c.op = op;
        c.wire_bf16 = wire ? 1 : 0;
        for (auto& t : tensors) {
            check_gpu_(t, "allreduce");
            const int dt = need_reduce_dtype(t, "allreduce");
            MCCL_CHECK(t.numel() > 0, "MCCL does not accept empty tensors");  // TensorChecks.hpp:31-34
            const bool use_wire = wire && dt == MCCLX_F32;  // :131
            const uint64_t bytes = static_cast<uint64_t>(t.numel()) * (use_wire ? 2u : t.element_size());
            c.dst.push_back(t.data_ptr());
            c.numel.push_back(static_cast<uint64_t>(t.numel()));
            c.dtype.push_back(dt);
            c.algo.push_back(mcclx_select_algo(env_alg, tree_below, bytes, t.numel(), world));  // :134-145
        }
        last_algo_ = c.algo.back();
        MCCL_DEBUG("rank %d allreduce: %zu tensor(s), first numel %llu, op %d, algo %d, wire %s%s", getRank(),
                   tensors.size(), (unsigned long long)c.numel[0], op, last_algo_, wire ? "bf16" : "native",
                   async ? ", event-based completion" : "");
    } catch (const std::exception& e) {
        c = Contribution{};
        c.error = e.what();
    }
    c.kind = K_ALLREDUCE;
    c.stream = my_stream();
    c.async = async ? 1 : 0;
    c.direct = env_direct() ? 1 : 0;
    c.transport = transport;
    c.work = work.get();
    c.marks = wait_marks_;
    flush_engine_();

    if (transport != 0) {
        // Rank by rank over the byte transport.  The ranks first meet to agree on what
        // they are about to do (a rank that disagrees, or failed its own checks, fails
        // everyone at once instead of leaving peers blocked in recv).
        const std::vector<uint64_t> numel = c.numel;
        const std::vector<int> dtype = c.dtype, algo = c.algo;
        const int op = c.op;
        const bool wire = c.wire_bf16 != 0;
        void* stream = c.stream;
        meet(std::move(c), [world](const std::vector<Contribution>& all) {
            for (int r = 1; r < world; ++r) {
                MCCL_CHECK(all[r].transport == all[0].transport, "allreduce: ranks disagree on MCCL_WIRE");
                MCCL_CHECK(all[r].op == all[0].op && all[r].wire_bf16 == all[0].wire_bf16,
                           "allreduce: ranks disagree on the reduce op or MCCL_WIRE_DTYPE");
                MCCL_CHECK(all[r].numel == all[0].numel && all[r].dtype == all[0].dtype,
                           "allreduce: ranks passed tensors of different size or dtype");
                MCCL_CHECK(all[r].algo == all[0].algo,
                           "allreduce: ranks resolved different algorithms (MCCL_ALLREDUCE_ALGO / MCCL_TREE_BELOW differ)");
            }
        });
        shared_->quiesce();  // the wire runs on queues of its own: nothing of this group may still be in flight
        if (!host_wire_) host_wire_ = std::make_unique<HostWire>(mesh_, getRank(), device_, opts_.timeout);
        for (size_t i = 0; i < tensors.size(); ++i)  // one after another (ProcessGroupMCCL.cpp:122-168)
            host_wire_->allreduce(tensors[i].data_ptr(), dtype[i], numel[i], op, algo[i], wire,
                                  transport == 1 ? HostWire::Mode::Pinned : HostWire::Mode::Staged, stream);
        return make_completed(c10d::OpType::ALLREDUCE, tensors, "mccl:allreduce");
    }

    auto shared = shared_;
    const int device = device_;
    ph_build.stop();
    phases::Span ph_meet(phases::kMeet);
    meet(std::move(c), [shared, world, device](const std::vector<Contribution>& all) {
        const auto leader_t0 = std::chrono::steady_clock::now();
        struct OffMeet {  // what the last arrival does here is not time spent meeting
            std::chrono::steady_clock::time_point t0;
            ~OffMeet() { phases::discount(phases::kMeet, std::chrono::steady_clock::now() - t0); }
        } off_meet{leader_t0};
        phases::Span ph_checks(phases::kLeaderChecks);
        const size_t nt = all[0].dst.size();
        const bool async = all[0].async != 0;
        int qsel = 0;
        mcclx_ctx* ctx = shared->ctx;
        bool small = false;
        if (async) {
            uint64_t bytes = 0;
            for (size_t i = 0; i < nt && i < all[0].numel.size() && i < all[0].dtype.size(); ++i)
                bytes += all[0].numel[i] * (all[0].dtype[i] == MCCLX_F32 ? 4u : 2u);
            small = bytes < shared->coalesce_below;
            ctx = shared->pick_queue(&qsel, small);
        } else {
            shared->begin_main_work();
        }
        for (int r = 0; r < world; ++r) {
            MCCL_CHECK(all[r].dst.size() == nt, "allreduce: ranks passed different numbers of tensors");
            MCCL_CHECK(all[r].op == all[0].op && all[r].wire_bf16 == all[0].wire_bf16,
                       "allreduce: ranks disagree on the reduce op or MCCL_WIRE_DTYPE");
            MCCL_CHECK((all[r].async != 0) == async, "allreduce: ranks disagree on MCCL_ALLREDUCE_ASYNC");
        }
        // mps_stream_sync, :172 -- once per distinct stream: ranks on one stream (threads
        // that all use torch's default stream) are covered by one wait, and a wait costs
        // the host about ten microseconds
        {
            ph_checks.stop();
            phases::Span ph(phases::kStreamWait);
            for (int r = 0; r < world; ++r) {
                bool seen = false;
                for (int q = 0; q < r; ++q) seen = seen || all[q].stream == all[r].stream;
                if (!seen) check_rc(mcclx_queue_wait_stream(ctx, all[r].stream));
            }
        }
        phases::Span ph_checks2(phases::kLeaderChecks);
        // one replay per tensor of the list; the reference runs them one after another
        // (ProcessGroupMCCL.cpp:122-168), here a list is issued together so that
        // entries sharing a plan need one launch per phase for all of them
        auto bucket = std::make_shared<Shared::Bucket>();
        auto& ptrs = bucket->ptrs;
        auto& reps = bucket->reps;
        ptrs.assign(nt, std::vector<void*>(static_cast<size_t>(world)));
        reps.resize(nt);
        std::vector<uint64_t> need(nt), offset(nt);
        uint64_t total = 0;
        for (size_t i = 0; i < nt; ++i) {
            for (int r = 0; r < world; ++r) {
                MCCL_CHECK(all[r].numel[i] == all[0].numel[i] && all[r].dtype[i] == all[0].dtype[i],
                           "allreduce: ranks passed tensors of different size or dtype");
                MCCL_CHECK(all[r].algo[i] == all[0].algo[i],
                           "allreduce: ranks resolved different algorithms (MCCL_ALLREDUCE_ALGO / MCCL_TREE_BELOW differ)");
                ptrs[i][static_cast<size_t>(r)] = all[r].dst[i];
            }
            mcclx_replay& rp = reps[i];
            std::memset(&rp, 0, sizeof rp);
            rp.world = world;
            rp.algo = all[0].algo[i];
            rp.op = all[0].op;
            rp.dtype = all[0].dtype[i];
            rp.wire_bf16 = all[0].wire_bf16;
            // all ranks of this build share one GPU: over the wire codec the fold reads the
            // peers' fp32 tensors where they lie (MCCL_DIRECT=0: through bf16 copies, the
            // shape the same schedule has across GPUs)
            rp.mode = all[0].direct ? MCCLX_REPLAY_DIRECT : MCCLX_REPLAY_FUSED;
            rp.acc = MCCLX_ACC_STEP;
            rp.numel = all[0].numel[i];
            rp.tensors = ptrs[i].data();
            need[i] = (mcclx_replay_workspace_bytes(&rp) + 255) / 256 * 256;
            offset[i] = total;
            total += need[i];
        }
        char* ws = nullptr;
        if (async && total) {
            // several calls may be in flight: each keeps a workspace of its own until it has finished
            bucket->workspace = shared->take_workspace(total + 256, ctx);
            auto p = reinterpret_cast<uintptr_t>(bucket->workspace.data_ptr());
            ws = reinterpret_cast<char*>((p + 255) / 256 * 256);
        } else {
            ws = static_cast<char*>(shared->workspace(total));
        }
        for (size_t i = 0; i < nt; ++i) {
            reps[i].workspace = need[i] ? ws + offset[i] : nullptr;
            reps[i].workspace_bytes = need[i];
        }
        if (async) {
            bucket->queue = qsel;
            bucket->small = small;
            for (size_t i = 0; i < nt; ++i) {
                const uint64_t tb = reps[i].numel * (reps[i].dtype == MCCLX_F32 ? 4u : 2u);
                for (int r = 0; r < world; ++r) {
                    const auto p = reinterpret_cast<uintptr_t>(ptrs[i][static_cast<size_t>(r)]);
                    bucket->spans.push_back(Shared::Span{p, p + tb});
                }
            }
            if (total) {
                const auto p = reinterpret_cast<uintptr_t>(ws);
                bucket->spans.push_back(Shared::Span{p, p + total});
            }
            for (int r = 0; r < world; ++r) {
                MCCL_CHECK(all[r].work != nullptr, "allreduce: a rank arrived without its Work");
                bucket->works.push_back(
                    c10::intrusive_ptr<WorkMCCL>::reclaim_copy(static_cast<WorkMCCL*>(all[r].work)));
            }
            // wait() on any rank's Work: make sure the launch is out, then let the
            // rank's current stream wait for the queue on the device
            // (weak references: a Work may outlive the group, and the last Work of a launch is
            // released on the completer thread, which must never be the one to tear the group down)
            std::weak_ptr<Shared::Bucket> weak = bucket;
            std::weak_ptr<Shared> weak_shared = shared;
            for (int r = 0; r < world; ++r) {
                // A stream that was put behind a launch of a queue is behind every earlier launch
                // of that queue as well: a rank that waits for its buckets one after another pays
                // for one event per queue, not one per bucket (an event record plus a wait of
                // torch's legacy stream cost the host 20-35 us).
                std::shared_ptr<WaitMarks> marks = all[r].marks;
                bucket->works[static_cast<size_t>(r)]->setWaitHook([weak_shared, weak, device, marks] {
                    phases::Span ph(phases::kWaitHook);
                    auto sh = weak_shared.lock();
                    if (!sh) return;  // the group is gone: its destructor has drained the queue
                    auto b = weak.lock();
                    if (!b) return;   // settled and released: nothing left to order against
                    if (!b->launched) sh->flush_parked(b->queue);
                    const int q = b->queue;
                    const uint64_t id = b->flight.load();
                    void* stream = dev::current_stream(device);
                    if (marks) {
                        std::lock_guard<std::mutex> lk(marks->mu);
                        if (id != 0 && marks->stream[q] == stream && marks->valid[q] && marks->upto[q] >= id) return;
                    }
                    const uint64_t newest = sh->newest_on(q);  // enqueued before the event below is
                    check_rc(mcclx_stream_wait_queue(sh->queue(q), stream));
                    if (marks) {
                        std::lock_guard<std::mutex> lk(marks->mu);
                        marks->stream[q] = stream;
                        marks->valid[q] = true;
                        marks->upto[q] = std::max(newest, id);
                    }
                });
            }
            ph_checks2.stop();
            shared->submit_bucket(bucket);
            return;
        }
        ph_checks2.stop();
        // The reference's allreduce is synchronous (ProcessGroupMCCL.cpp:170-185): when
        // it returns, every rank's tensor holds the result and the queue is drained.
        {
            phases::Span ph(phases::kLaunch);
            if (nt == 1)
                shared->allreduce(reps[0]);  // a single bucket: recorded and replayed when it comes again
            else
                check_rc(mcclx_allreduce_replay_many(ctx, reps.data(), static_cast<uint32_t>(nt)));
        }
        phases::Span ph(phases::kDrain);
        shared->drain_main();  // mccl_queue_drain, :178
    });
    ph_meet.stop();
    if (async) return work;
    phases::Span ph_work(phases::kWorkMake);
    return make_completed(c10d::OpType::ALLREDUCE, tensors, "mccl:allreduce");
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::broadcast(std::vector<at::Tensor>& tensors,
                                                           const c10d::BroadcastOptions& opts) {
    if (getSize() == 1) return make_completed(c10d::OpType::BROADCAST, tensors, "mccl:broadcast");
    MCCL_CHECK(!tensors.empty(), "broadcast: empty tensor list");
    auto tensors_copy = tensors;
    const int root = static_cast<int>(opts.rootRank);
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::BROADCAST, tensors, "mccl:broadcast",
                         [this, shared, tensors_copy, root, world, stream]() mutable {
        meet_built(K_BROADCAST, stream, [&](Contribution& c) {
            c.root = root;
            for (auto& t : tensors_copy) {
                check_gpu_(t, "broadcast");
                c.dst.push_back(t.data_ptr());
                c.nbytes.push_back(static_cast<uint64_t>(t.nbytes()));
            }
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            const int root = all[0].root;
            MCCL_CHECK(root >= 0 && root < world, "broadcast: root outside the group");
            for (int r = 0; r < world; ++r) {
                MCCL_CHECK(all[r].root == root && all[r].dst.size() == all[0].dst.size(),
                           "broadcast: ranks disagree on root or tensor count");
                check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            }
            for (size_t i = 0; i < all[0].dst.size(); ++i)
                for (int r = 0; r < world; ++r) {
                    if (r == root) continue;
                    MCCL_CHECK(all[r].nbytes[i] == all[root].nbytes[i], "broadcast: size mismatch");
                    check_rc(mcclx_copy(shared->ctx, all[r].dst[i], all[root].dst[i], all[root].nbytes[i]));
                }
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::_allgather_base(at::Tensor& output_tensor,
                                                                 at::Tensor& input_tensor,
                                                                 const c10d::AllgatherOptions&) {
    if (getSize() == 1) {
        output_tensor.copy_(input_tensor);
        return make_completed(c10d::OpType::_ALLGATHER_BASE, {output_tensor}, "mccl:_allgather_base");
    }
    at::Tensor out = output_tensor, in = input_tensor;
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::_ALLGATHER_BASE, {output_tensor},
                         "mccl:_allgather_base", [this, shared, out, in, world, stream]() mutable {
        meet_built(K_ALLGATHER_BASE, stream, [&](Contribution& c) {
            check_gpu_(in, "_allgather_base");
            check_gpu_(out, "_allgather_base");
            const uint64_t chunk = static_cast<uint64_t>(in.nbytes());
            MCCL_CHECK(static_cast<uint64_t>(out.nbytes()) == chunk * static_cast<uint64_t>(world),
                       "_allgather_base: output size != input * world");
            c.dst = {out.data_ptr()};
            c.src = {in.data_ptr()};
            c.nbytes = {chunk};
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            std::vector<void*> outs(static_cast<size_t>(world));
            std::vector<const void*> ins(static_cast<size_t>(world));
            for (int r = 0; r < world; ++r) {
                MCCL_CHECK(all[r].nbytes[0] == all[0].nbytes[0], "_allgather_base: ranks pass different sizes");
                outs[static_cast<size_t>(r)] = all[r].dst[0];
                ins[static_cast<size_t>(r)] = all[r].src[0];
                check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            }
            check_rc(mcclx_allgather_replay(shared->ctx, world, outs.data(), ins.data(), all[0].nbytes[0]));
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::allgather(
    std::vector<std::vector<at::Tensor>>& output_tensors, std::vector<at::Tensor>& input_tensors,
    const c10d::AllgatherOptions&) {
    if (getSize() == 1) {
        MCCL_CHECK(!output_tensors.empty() && !output_tensors[0].empty(), "allgather output empty");
        output_tensors[0][0].copy_(input_tensors[0]);
        return make_completed(c10d::OpType::ALLGATHER, output_tensors[0], "mccl:allgather");
    }
    auto outs_copy = output_tensors;
    auto ins_copy = input_tensors;
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::ALLGATHER, input_tensors, "mccl:allgather",
                         [this, shared, outs_copy, ins_copy, world, stream]() mutable {
        meet_built(K_ALLGATHER, stream, [&](Contribution& c) {
            MCCL_CHECK(ins_copy.size() == outs_copy.size(), "allgather: input/output count mismatch");
            for (size_t i = 0; i < ins_copy.size(); ++i) {
                MCCL_CHECK(static_cast<int>(outs_copy[i].size()) == world, "allgather: output list size != world");
                check_gpu_(ins_copy[i], "allgather");
                c.src.push_back(ins_copy[i].data_ptr());
                c.nbytes.push_back(static_cast<uint64_t>(ins_copy[i].nbytes()));
                for (auto& o : outs_copy[i]) {
                    check_gpu_(o, "allgather");
                    MCCL_CHECK(o.nbytes() == ins_copy[i].nbytes(), "allgather: output size != input size");
                    c.dst.push_back(o.data_ptr());
                }
            }
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            for (int r = 0; r < world; ++r) check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            const size_t nt = all[0].src.size();
            for (size_t i = 0; i < nt; ++i)
                for (int r = 0; r < world; ++r) {
                    MCCL_CHECK(all[r].src.size() == nt && all[r].nbytes[i] == all[0].nbytes[i],
                               "allgather: ranks pass different tensors");
                    for (int p = 0; p < world; ++p)
                        check_rc(mcclx_copy(shared->ctx, all[r].dst[i * static_cast<size_t>(world) + p],
                                            all[p].src[i], all[0].nbytes[i]));
                }
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::_reduce_scatter_base(at::Tensor& output_tensor,
                                                                      at::Tensor& input_tensor,
                                                                      const c10d::ReduceScatterOptions& opts) {
    if (getSize() == 1) {
        output_tensor.copy_(input_tensor);
        return make_completed(c10d::OpType::_REDUCE_SCATTER_BASE, {output_tensor}, "mccl:_reduce_scatter_base");
    }
    const int op = reduce_op_code(opts.reduceOp);
    at::Tensor out = output_tensor, in = input_tensor;
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::_REDUCE_SCATTER_BASE, {output_tensor},
                         "mccl:_reduce_scatter_base", [this, shared, out, in, op, world, stream]() mutable {
        meet_built(K_REDUCE_SCATTER_BASE, stream, [&](Contribution& c) {
            check_gpu_(in, "_reduce_scatter_base");
            check_gpu_(out, "_reduce_scatter_base");
            MCCL_CHECK(static_cast<uint64_t>(in.nbytes()) == static_cast<uint64_t>(out.nbytes()) * world,
                       "_reduce_scatter_base: input size != output * world");
            c.op = op;
            c.dst = {out.data_ptr()};
            c.src = {in.data_ptr()};
            c.numel = {static_cast<uint64_t>(out.numel())};
            c.dtype = {need_reduce_dtype(out, "_reduce_scatter_base")};
            MCCL_CHECK(in.scalar_type() == out.scalar_type(), "_reduce_scatter_base: dtype mismatch");
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            std::vector<void*> outs(static_cast<size_t>(world));
            std::vector<const void*> ins(static_cast<size_t>(world));
            for (int r = 0; r < world; ++r) {
                MCCL_CHECK(all[r].numel[0] == all[0].numel[0] && all[r].dtype[0] == all[0].dtype[0] &&
                               all[r].op == all[0].op,
                           "_reduce_scatter_base: ranks disagree on size, dtype or op");
                outs[static_cast<size_t>(r)] = all[r].dst[0];
                ins[static_cast<size_t>(r)] = all[r].src[0];
                check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            }
            // one launch for the whole group (the reference batches its N-1 binary
            // launches per rank into one command buffer, :378-387)
            check_rc(mcclx_batch_begin(shared->ctx, "mccl:_reduce_scatter_base"));
            int rc = mcclx_reduce_scatter_replay(shared->ctx, world, outs.data(), ins.data(), all[0].dtype[0],
                                                 all[0].numel[0], all[0].op, MCCLX_REPLAY_FUSED, MCCLX_ACC_STEP);
            mcclx_batch_end(shared->ctx);
            check_rc(rc);
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::reduce_scatter(
    std::vector<at::Tensor>& output_tensors, std::vector<std::vector<at::Tensor>>& input_tensors,
    const c10d::ReduceScatterOptions& opts) {
    if (getSize() == 1) {
        MCCL_CHECK(!input_tensors.empty() && !input_tensors[0].empty(), "reduce_scatter input empty");
        output_tensors[0].copy_(input_tensors[0][0]);
        return make_completed(c10d::OpType::REDUCE_SCATTER, output_tensors, "mccl:reduce_scatter");
    }
    const int op = reduce_op_code(opts.reduceOp);
    auto outs_copy = output_tensors;
    auto ins_copy = input_tensors;
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::REDUCE_SCATTER, output_tensors,
                         "mccl:reduce_scatter", [this, shared, outs_copy, ins_copy, op, world, stream]() mutable {
        meet_built(K_REDUCE_SCATTER, stream, [&](Contribution& c) {
            MCCL_CHECK(outs_copy.size() == ins_copy.size(), "reduce_scatter: count mismatch");
            c.op = op;
            for (size_t i = 0; i < outs_copy.size(); ++i) {
                auto& out = outs_copy[i];
                auto& ins = ins_copy[i];
                MCCL_CHECK(static_cast<int>(ins.size()) == world, "reduce_scatter: input list size != world");
                check_gpu_(out, "reduce_scatter");
                c.dst.push_back(out.data_ptr());
                c.numel.push_back(static_cast<uint64_t>(out.numel()));
                c.dtype.push_back(need_reduce_dtype(out, "reduce_scatter"));
                for (auto& t : ins) {
                    check_gpu_(t, "reduce_scatter");
                    MCCL_CHECK(t.nbytes() == out.nbytes() && t.scalar_type() == out.scalar_type(),
                               "reduce_scatter: output size != input chunk size");
                    c.src.push_back(t.data_ptr());
                }
            }
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            for (int r = 0; r < world; ++r) check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            const size_t nt = all[0].dst.size();
            const size_t W = static_cast<size_t>(world);
            for (size_t i = 0; i < nt; ++i) {
                std::vector<void*> outs(W);
                std::vector<const void*> shares(W * W);
                for (size_t r = 0; r < W; ++r) {
                    MCCL_CHECK(all[r].dst.size() == nt && all[r].numel[i] == all[0].numel[i] &&
                                   all[r].dtype[i] == all[0].dtype[i] && all[r].op == all[0].op,
                               "reduce_scatter: ranks disagree on size, dtype or op");
                    outs[r] = all[r].dst[i];
                    // rank p's list entry r is its contribution to rank r's output
                    for (size_t p = 0; p < W; ++p) shares[r * W + p] = all[p].src[i * W + r];
                }
                check_rc(mcclx_reduce_scatter_shares(shared->ctx, world, outs.data(), shares.data(),
                                                     all[0].dtype[i], all[0].numel[i], all[0].op,
                                                     MCCLX_REPLAY_FUSED, MCCLX_ACC_STEP));
            }
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::barrier(const c10d::BarrierOptions&) {
    if (getSize() == 1) return make_completed(c10d::OpType::BARRIER, {}, "mccl:barrier");
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::BARRIER, {}, "mccl:barrier",
                         [this, shared, stream]() {
        // the Work's sync callback drains the main queue: it must be behind everything of the group
        meet_built(K_BARRIER, stream, [](Contribution&) {},
                   [shared](const std::vector<Contribution>&) { shared->begin_main_work(); });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::alltoall_base(at::Tensor& output_tensor, at::Tensor& input_tensor,
                                                               std::vector<int64_t>& output_split_sizes,
                                                               std::vector<int64_t>& input_split_sizes,
                                                               const c10d::AllToAllOptions&) {
    if (getSize() == 1) {
        output_tensor.copy_(input_tensor);
        return make_completed(c10d::OpType::ALLTOALL_BASE, {output_tensor}, "mccl:alltoall_base");
    }
    at::Tensor out = output_tensor, in = input_tensor;
    auto out_splits = output_split_sizes;
    auto in_splits = input_split_sizes;
    const int world = getSize();
    const int rank = getRank();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::ALLTOALL_BASE, {output_tensor},
                         "mccl:alltoall_base",
                         [this, shared, out, in, out_splits, in_splits, world, rank, stream]() mutable {
        meet_built(K_ALLTOALL_BASE, stream, [&](Contribution& c) {
            check_gpu_(in, "alltoall_base");
            check_gpu_(out, "alltoall_base");
            const uint64_t esize = static_cast<uint64_t>(in.element_size());
            MCCL_CHECK(esize == static_cast<uint64_t>(out.element_size()), "alltoall_base: dtype mismatch");
            const size_t W = static_cast<size_t>(world);
            // byte offsets of the W pieces (ProcessGroupMCCL.cpp:498-521); split sizes
            // count rows of dim 0, as c10d defines them
            auto offsets = [&](const at::Tensor& t, const std::vector<int64_t>& splits, const char* what) {
                std::vector<uint64_t> off(W + 1, 0);
                if (splits.empty()) {
                    const uint64_t per = static_cast<uint64_t>(t.numel()) / W * esize;
                    MCCL_CHECK(per * W == static_cast<uint64_t>(t.nbytes()),
                               std::string("alltoall_base: ") + what + " not divisible by world");
                    for (size_t p = 0; p < W; ++p) off[p + 1] = off[p] + per;
                } else {
                    MCCL_CHECK(splits.size() == W, std::string("alltoall_base: ") + what + "_split_sizes wrong length");
                    const uint64_t row = t.dim() > 0 && t.size(0) > 0
                                             ? static_cast<uint64_t>(t.nbytes()) / static_cast<uint64_t>(t.size(0))
                                             : esize;
                    for (size_t p = 0; p < W; ++p) {
                        MCCL_CHECK(splits[p] >= 0, std::string("alltoall_base: negative ") + what + " split");
                        off[p + 1] = off[p] + static_cast<uint64_t>(splits[p]) * row;
                    }
                    MCCL_CHECK(off[W] == static_cast<uint64_t>(t.nbytes()),
                               std::string("alltoall_base: ") + what + "_split_sizes do not add up to the tensor");
                }
                return off;
            };
            c.in_off = offsets(in, in_splits, "input");
            c.out_off = offsets(out, out_splits, "output");
            const size_t r = static_cast<size_t>(rank);
            MCCL_CHECK(c.in_off[r + 1] - c.in_off[r] == c.out_off[r + 1] - c.out_off[r],
                       "alltoall_base: self chunk size mismatch");
            c.src = {in.data_ptr()};
            c.dst = {out.data_ptr()};
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            const size_t W = static_cast<size_t>(world);
            for (size_t r = 0; r < W; ++r) check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            for (size_t r = 0; r < W; ++r)        // sender
                for (size_t p = 0; p < W; ++p) {  // receiver
                    const uint64_t slen = all[r].in_off[p + 1] - all[r].in_off[p];
                    const uint64_t rlen = all[p].out_off[r + 1] - all[p].out_off[r];
                    MCCL_CHECK(slen == rlen, "alltoall_base: rank " + std::to_string(r) + " sends " +
                                                 std::to_string(slen) + " bytes to rank " + std::to_string(p) +
                                                 ", which expects " + std::to_string(rlen));
                }
            // A rank may pass the same buffer as input and output (the reference stages
            // through host memory, so that works there): then the inputs are first
            // copied aside, since the pieces are moved one after another on the queue.
            bool aliased = false;
            uint64_t total_in = 0;
            std::vector<uint64_t> base(W + 1, 0);
            for (size_t r = 0; r < W; ++r) {
                base[r + 1] = base[r] + (all[r].in_off[W] + 255) / 256 * 256;
                for (size_t q = 0; q < W; ++q) {
                    auto a = reinterpret_cast<uintptr_t>(all[r].src[0]);
                    auto b = reinterpret_cast<uintptr_t>(all[q].dst[0]);
                    if (a < b + all[q].out_off[W] && b < a + all[r].in_off[W]) aliased = true;
                }
            }
            total_in = base[W];
            char* aside = aliased ? static_cast<char*>(shared->workspace(total_in)) : nullptr;
            if (aliased)
                for (size_t r = 0; r < W; ++r)
                    if (all[r].in_off[W])
                        check_rc(mcclx_copy(shared->ctx, aside + base[r], all[r].src[0], all[r].in_off[W]));
            for (size_t r = 0; r < W; ++r)
                for (size_t p = 0; p < W; ++p) {
                    const uint64_t len = all[r].in_off[p + 1] - all[r].in_off[p];
                    if (len == 0) continue;
                    const char* from = aliased ? aside + base[r] : static_cast<const char*>(all[r].src[0]);
                    check_rc(mcclx_copy(shared->ctx, static_cast<char*>(all[p].dst[0]) + all[p].out_off[r],
                                        from + all[r].in_off[p], len));
                }
        });
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::alltoall(std::vector<at::Tensor>& output_tensors,
                                                          std::vector<at::Tensor>& input_tensors,
                                                          const c10d::AllToAllOptions&) {
    MCCL_CHECK(static_cast<int>(input_tensors.size()) == getSize() &&
                   static_cast<int>(output_tensors.size()) == getSize(),
               "alltoall: list size != world");  // ProcessGroupMCCL.cpp:555-557
    if (getSize() == 1) {
        output_tensors[0].copy_(input_tensors[0]);
        return make_completed(c10d::OpType::ALLTOALL, output_tensors, "mccl:alltoall");
    }
    auto outs_copy = output_tensors;
    auto ins_copy = input_tensors;
    const int world = getSize();
    auto shared = shared_;
    void* stream = my_stream();
    return async_submit_(*engine_, ctx_, stream, c10d::OpType::ALLTOALL, output_tensors, "mccl:alltoall",
                         [this, shared, outs_copy, ins_copy, world, stream]() mutable {
        meet_built(K_ALLTOALL, stream, [&](Contribution& c) {
            for (int p = 0; p < world; ++p) {
                check_gpu_(ins_copy[static_cast<size_t>(p)], "alltoall");
                check_gpu_(outs_copy[static_cast<size_t>(p)], "alltoall");
                c.src.push_back(ins_copy[static_cast<size_t>(p)].data_ptr());
                c.dst.push_back(outs_copy[static_cast<size_t>(p)].data_ptr());
                c.in_off.push_back(static_cast<uint64_t>(ins_copy[static_cast<size_t>(p)].nbytes()));    // sizes here
                c.out_off.push_back(static_cast<uint64_t>(outs_copy[static_cast<size_t>(p)].nbytes()));
            }
        }, [shared, world](const std::vector<Contribution>& all) {
            shared->begin_main_work();
            const size_t W = static_cast<size_t>(world);
            for (size_t r = 0; r < W; ++r) check_rc(mcclx_queue_wait_stream(shared->ctx, all[r].stream));
            for (size_t r = 0; r < W; ++r)
                for (size_t p = 0; p < W; ++p)
                    MCCL_CHECK(all[r].in_off[p] == all[p].out_off[r],
                               "alltoall: rank " + std::to_string(r) + " sends " + std::to_string(all[r].in_off[p]) +
                                   " bytes to rank " + std::to_string(p) + ", which expects " +
                                   std::to_string(all[p].out_off[r]));
            for (size_t r = 0; r < W; ++r)
                for (size_t p = 0; p < W; ++p)
                    if (all[r].in_off[p])
                        check_rc(mcclx_copy(shared->ctx, all[p].dst[r], all[r].src[p], all[r].in_off[p]));
        });
    });
}

// Point-to-point.  The reference writes an 8-byte {tag, nbytes} header and then
// the payload to the peer's socket (ProcessGroupMCCL.cpp:614-631); the socket
// buffers what the receiver has not asked for yet.  Here the sender copies the
// payload into a device buffer owned by the parcel (so the Work completes
// without waiting for the receiver, and the sender may reuse its tensor), and
// the receiver copies it out.  All ranks of a mesh share one reduce queue, so
// the two copies are ordered by the queue itself.
c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::send(std::vector<at::Tensor>& tensors, int dst_rank, int tag) {
    MCCL_CHECK(dst_rank >= 0 && dst_rank < getSize() && dst_rank != getRank(), "send: bad dst_rank");
    auto tensors_copy = tensors;
    auto shared = shared_;
    auto mesh = mesh_;
    const int rank = getRank();
    return async_submit_(*engine_, ctx_, my_stream(), c10d::OpType::SEND, tensors, "mccl:send",
                         [shared, mesh, tensors_copy, rank, dst_rank, tag]() mutable {
        shared->begin_main_work();
        for (auto& t : tensors_copy) {
            check_gpu_(t, "send");
            Parcel p;
            p.tag = static_cast<int32_t>(tag);
            p.nbytes = static_cast<uint64_t>(t.nbytes());
            if (p.nbytes) {
                auto hold = std::make_shared<at::Tensor>(dev::empty_bytes(static_cast<int64_t>(p.nbytes), shared->device));
                order_after_allocator(shared->ctx, shared->device);
                check_rc(mcclx_copy(shared->ctx, hold->data_ptr(), t.data_ptr(), p.nbytes));
                p.data = hold->data_ptr();
                p.keep = hold;
            }
            mesh->post(rank, dst_rank, std::move(p));
        }
    });
}

c10::intrusive_ptr<c10d::Work> ProcessGroupMCCL::recv(std::vector<at::Tensor>& tensors, int src_rank, int tag) {
    MCCL_CHECK(src_rank >= 0 && src_rank < getSize() && src_rank != getRank(), "recv: bad src_rank");
    auto tensors_copy = tensors;
    auto shared = shared_;
    auto mesh = mesh_;
    const int rank = getRank();
    const auto timeout = opts_.timeout;
    return async_submit_(*engine_, ctx_, my_stream(), c10d::OpType::RECV, tensors, "mccl:recv",
                         [shared, mesh, tensors_copy, rank, src_rank, tag, timeout]() mutable {
        shared->begin_main_work();
        for (auto& t : tensors_copy) {
            check_gpu_(t, "recv");
            Parcel p = mesh->take(src_rank, rank, timeout);
            // header checks of the reference (ProcessGroupMCCL.cpp:645-651)
            MCCL_CHECK(tag < 0 || p.tag == tag, "recv: tag mismatch (expected " + std::to_string(tag) + " got " +
                                                    std::to_string(p.tag) + ")");
            MCCL_CHECK(p.nbytes == static_cast<uint64_t>(t.nbytes()),
                       "recv: size mismatch (expected " + std::to_string(t.nbytes()) + " got " +
                           std::to_string(p.nbytes) + ")");
            if (p.nbytes) {
                check_rc(mcclx_copy(shared->ctx, t.data_ptr(), p.data, p.nbytes));
                // the parcel's buffer goes back to torch's allocator when `p` dies:
                // nothing may still be reading it then
                check_rc(mcclx_queue_drain(shared->ctx));
            }
        }
    });
}

}  // namespace mccl
