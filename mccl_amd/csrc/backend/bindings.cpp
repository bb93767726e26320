// bindings.cpp -- the `mccl_amd._C` extension module.
//
// Exposes the factory torch.distributed needs, mirroring the reference's
// csrc/backend/Registration.cpp:22-39 (`_create_process_group_mccl(store, rank,
// size, timeout)`), plus small host-only hooks the CPU tests drive (the FIFO
// engine, the Work object, the in-process mesh).
#include <torch/extension.h>

#include <pybind11/chrono.h>
#include <pybind11/functional.h>
#include <pybind11/stl.h>

#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/HashStore.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>

#include <execinfo.h>
#include <fcntl.h>
#include <signal.h>
#include <unistd.h>

#include <cstring>
#include <exception>

#include <atomic>
#include <chrono>
#include <cstdlib>
#include <thread>

#include "backend/Errors.hpp"
#include "backend/LocalMesh.hpp"
#include "backend/Logging.hpp"
#include "backend/Phases.hpp"
#include "backend/ProcessGroupMCCL.hpp"
#include "backend/Progress.hpp"
#include "backend/WorkMCCL.hpp"

namespace py = pybind11;

namespace {

// Blocking hooks for the engine (Progress.hpp): give the GIL up while a caller
// waits for the worker thread, if this thread holds it.
void* gil_release_if_held() {
    if (!Py_IsInitialized() || !PyGILState_Check()) return nullptr;
    return PyEval_SaveThread();
}
void gil_take_back(void* token) {
    if (token) PyEval_RestoreThread(static_cast<PyThreadState*>(token));
}

// MCCL_ABORT_BACKTRACE: when the process aborts, the native stack of the aborting thread is
// written out before the handler that was installed before runs (Python's faulthandler prints
// the interpreter's side), and an uncaught C++ exception is named before it ends the process.
// An abort raised on one of the backend's worker threads is otherwise anonymous.  The value
// is "1" for stderr or the path of a file to append to -- under a test runner that captures
// file descriptor 2, what goes to stderr dies with the process, a file does not.
struct sigaction g_previous_abort_action;
int g_abort_fd = 2;
std::terminate_handler g_previous_terminate = nullptr;

void write_all(int fd, const char* text) { (void)!write(fd, text, strlen(text)); }

void abort_backtrace(int sig, siginfo_t* info, void* uctx) {
    write_all(g_abort_fd, "\n[MCCL] SIGABRT: native stack of the aborting thread\n");
    void* frames[64];
    const int n = backtrace(frames, 64);
    backtrace_symbols_fd(frames, n, g_abort_fd);
    sigaction(SIGABRT, &g_previous_abort_action, nullptr);
    if (g_previous_abort_action.sa_flags & SA_SIGINFO) {
        if (g_previous_abort_action.sa_sigaction) g_previous_abort_action.sa_sigaction(sig, info, uctx);
    } else if (g_previous_abort_action.sa_handler != SIG_DFL && g_previous_abort_action.sa_handler != SIG_IGN) {
        g_previous_abort_action.sa_handler(sig);
    }
    raise(sig);
}

// std::terminate: say which exception it was (and that there was none, if so) where the
// abort handler's stack will follow, then go on to whoever was installed before (abort).
void terminate_with_message() {
    write_all(g_abort_fd, "\n[MCCL] std::terminate called");
    if (std::exception_ptr e = std::current_exception()) {
        try {
            std::rethrow_exception(e);
        } catch (const std::exception& ex) {
            write_all(g_abort_fd, " with an uncaught exception: ");
            write_all(g_abort_fd, ex.what());
        } catch (...) {
            write_all(g_abort_fd, " with an uncaught exception of a non-standard type");
        }
    } else {
        write_all(g_abort_fd, " without an active exception (a joinable std::thread destroyed, or a throw from a noexcept function)");
    }
    write_all(g_abort_fd, "\n");
    if (g_previous_terminate) g_previous_terminate();
    abort();
}

void install_abort_backtrace() {
    const char* e = std::getenv("MCCL_ABORT_BACKTRACE");
    if (!e || !*e || (e[0] == '0' && !e[1])) return;
    if (!(e[0] == '1' && !e[1])) {
        const int fd = open(e, O_WRONLY | O_CREAT | O_APPEND | O_CLOEXEC, 0644);
        if (fd >= 0) g_abort_fd = fd;
    }
    void* warm[2];
    (void)backtrace(warm, 2);  // loads the unwinder now, not inside the handler
    struct sigaction sa;
    sa.sa_sigaction = &abort_backtrace;
    sigemptyset(&sa.sa_mask);
    sa.sa_flags = SA_SIGINFO | SA_NODEFER;
    sigaction(SIGABRT, &sa, &g_previous_abort_action);
    g_previous_terminate = std::set_terminate(&terminate_with_message);
}

// The engine shut down from its own worker thread.
//  "task_owns_engine": a task holds the last reference to the engine it runs on; two more
//      tasks are queued behind it.  Returns the order in which the three ran.
//  "callback_drops_owner": an owner of an engine (as a process group is) is kept alive only
//      by a Future callback; the engine's task completes the Work, the callback runs on the
//      engine thread and is destroyed there, and with it the owner and its engine.
std::vector<int> progress_self_shutdown(const std::string& mode) {
    auto order = std::make_shared<std::vector<int>>();
    auto mu = std::make_shared<std::mutex>();
    auto push = [order, mu](int v) {
        std::lock_guard<std::mutex> lk(*mu);
        order->push_back(v);
    };
    auto settled = [&](size_t want) {
        for (int i = 0; i < 500; ++i) {
            {
                std::lock_guard<std::mutex> lk(*mu);
                if (order->size() >= want) break;
            }
            std::this_thread::sleep_for(std::chrono::milliseconds(10));
        }
        std::this_thread::sleep_for(std::chrono::milliseconds(30));  // lets the worker leave its loop
        std::lock_guard<std::mutex> lk(*mu);
        return *order;
    };
    if (mode == "task_owns_engine") {
        auto engine = std::make_shared<mccl::Progress>();
        engine->submit([engine, push] {
            std::this_thread::sleep_for(std::chrono::milliseconds(40));  // until the caller has let go
            push(1);
        });
        engine->submit([push] { push(2); });
        engine->submit([push] { push(3); });
        engine.reset();
        return settled(3);
    }
    if (mode == "callback_drops_owner") {
        struct Owner {
            std::unique_ptr<mccl::Progress> engine = std::make_unique<mccl::Progress>();
            std::function<void(int)> push;
            ~Owner() {
                engine->shutdown();
                push(9);  // the owner's members are still whole here
            }
        };
        auto owner = std::make_shared<Owner>();
        owner->push = push;
        auto work = c10::make_intrusive<mccl::WorkMCCL>(c10d::OpType::ALLREDUCE, std::vector<at::Tensor>{}, "mccl:test");
        work->getFuture()->addCallback([owner, push](c10::ivalue::Future&) { push(1); });
        mccl::Progress* engine = owner->engine.get();
        engine->submit([work, push] {
            std::this_thread::sleep_for(std::chrono::milliseconds(40));
            work->finish();  // runs the callback here; the Future then drops it, and the owner with it
            push(2);
        });
        engine->submit([push] { push(3); });
        owner.reset();
        work.reset();
        return settled(4);
    }
    throw mccl::MCCLError("unknown mode " + mode);
}

// Submits n tasks; task i throws when bit i of throw_mask is set (i < 64).
// Returns the order in which the non-throwing tasks ran.
std::vector<int> progress_order(int n, uint64_t throw_mask, bool use_destructor) {
    std::vector<int> order;
    std::mutex mu;
    {
        mccl::Progress p;
        for (int i = 0; i < n; ++i) {
            const bool thr = i < 64 && ((throw_mask >> i) & 1u);
            p.submit([i, thr, &order, &mu] {
                if (thr) throw std::runtime_error("boom");
                std::lock_guard<std::mutex> lk(mu);
                order.push_back(i);
            });
        }
        if (!use_destructor) {
            p.shutdown();
            p.shutdown();  // idempotent
        }
    }
    return order;
}

// Called WITH the GIL held: a task that needs the GIL (as one that drops the last
// reference to a Python-created tensor does) must not dead-lock the shutdown.
int progress_shutdown_while_task_needs_gil() {
    int ran = 0;
    mccl::Progress p;
    p.submit([&ran] {
        std::this_thread::sleep_for(std::chrono::milliseconds(20));
        py::gil_scoped_acquire gil;
        ran = 1;
    });
    p.shutdown();
    return ran;
}

// Microseconds a submit() takes while the worker is busy with a 50 ms task.
long progress_submit_latency_us() {
    mccl::Progress p;
    p.submit([] { std::this_thread::sleep_for(std::chrono::milliseconds(50)); });
    auto t0 = std::chrono::steady_clock::now();
    p.submit([] {});
    auto t1 = std::chrono::steady_clock::now();
    p.shutdown();
    return static_cast<long>(std::chrono::duration_cast<std::chrono::microseconds>(t1 - t0).count());
}

// Exercises WorkMCCL without any device: returns (completed, success, message).
std::tuple<bool, bool, std::string> work_probe(const std::string& mode, int wait_ms) {
    auto w = c10::make_intrusive<mccl::WorkMCCL>(c10d::OpType::ALLREDUCE, std::vector<at::Tensor>{}, "mccl:test");
    std::string msg;
    if (mode == "finish") {
        w->finish();
        w->finish();
    } else if (mode == "fail") {
        w->finishWithException(std::make_exception_ptr(mccl::MCCLError("engine task failed")));
        w->finish();  // too late: the first completion stands
    } else if (mode == "sync_cb_throws") {
        w->setSyncCallback([] { throw mccl::MCCLError("drain failed"); });
        w->finish();
    } else if (mode == "late") {
        std::thread([w] {
            std::this_thread::sleep_for(std::chrono::milliseconds(30));
            w->finish();
        }).detach();
    }
    bool ok = false;
    try {
        ok = w->wait(std::chrono::milliseconds(wait_ms));
        if (!ok) msg = "timeout";
    } catch (const std::exception& e) {
        msg = e.what();
    }
    if (mode == "late") w->wait();
    bool future_err = w->getFuture()->completed() && w->getFuture()->hasError();
    return {w->isCompleted(), w->isSuccess() && !future_err, msg};
}

// N threads meet `rounds` times in a LocalMesh; rank `absent` (if >= 0) never
// shows up -- or shows up `late_ms` milliseconds after the others, if that is given --,
// `leader_throws` makes the leader throw.  Returns per-rank messages; a leader that ran
// although a rank had already left with a timeout shows as a count in the late rank's message.
std::vector<std::string> mesh_probe(int world, int rounds, int absent, int timeout_ms, bool leader_throws, int late_ms) {
    auto mesh = mccl::LocalMesh::create(mccl::LocalMesh::fresh_key(), world);
    std::vector<std::string> out(static_cast<size_t>(world));
    std::vector<std::thread> ts;
    std::atomic<int> leader_runs{0};
    for (int r = 0; r < world; ++r) {
        if (r == absent && late_ms < 0) {
            out[static_cast<size_t>(r)] = "absent";
            continue;
        }
        ts.emplace_back([&, r] {
            try {
                if (r == absent) std::this_thread::sleep_for(std::chrono::milliseconds(late_ms));
                for (int i = 0; i < rounds; ++i) {
                    mccl::Contribution c;
                    c.kind = 100 + i;
                    c.numel = {static_cast<uint64_t>(r)};
                    mesh->rendezvous(r, c, std::chrono::milliseconds(timeout_ms),
                                     [&](const std::vector<mccl::Contribution>& all) {
                                         for (int q = 0; q < world; ++q)
                                             if (all[static_cast<size_t>(q)].numel[0] != static_cast<uint64_t>(q))
                                                 throw mccl::MCCLError("slot mix-up");
                                         ++leader_runs;
                                         if (leader_throws) throw mccl::MCCLError("leader failed");
                                     });
                }
                out[static_cast<size_t>(r)] = "ok:" + std::to_string(leader_runs.load());
            } catch (const std::exception& e) {
                out[static_cast<size_t>(r)] = e.what();
            }
        });
    }
    for (auto& t : ts) t.join();
    return out;
}

// `world` ranks as native threads, each with its own process group on device 0,
// issue `buckets` allreduces of `numel` floats back to back and wait for them;
// the best of `rounds` rounds, in microseconds per bucket, for every rank.  What
// the c10d surface costs without an interpreter in the ranks' way (the knobs are
// read from the environment as always).
std::vector<double> allreduce_rate_probe(int world, int64_t numel, int buckets, int rounds) {
    auto store = c10::make_intrusive<c10d::HashStore>();
    std::vector<double> best(static_cast<size_t>(world), 1e30);
    std::vector<std::string> errs(static_cast<size_t>(world));
    std::vector<std::thread> ts;
    for (int r = 0; r < world; ++r)
        ts.emplace_back([&, r] {
            try {
                c10::hip::set_device(0);
                mccl::ProcessGroupMCCL::Options opts;
                opts.timeout = std::chrono::milliseconds(120000);
                auto pg = c10::make_intrusive<mccl::ProcessGroupMCCL>(store, r, world, opts);
                std::vector<std::vector<at::Tensor>> lists;
                for (int b = 0; b < buckets; ++b)
                    lists.push_back({at::randn({numel}, at::TensorOptions().device(at::kCUDA, 0)) * 1e-3});
                c10d::AllreduceOptions o;
                o.reduceOp = c10d::ReduceOp::AVG;
                auto stream = c10::hip::getCurrentHIPStream(0);
                for (int rep = 0; rep < rounds; ++rep) {
                    stream.synchronize();
                    pg->barrier()->wait();
                    const auto t0 = std::chrono::steady_clock::now();
                    std::vector<c10::intrusive_ptr<c10d::Work>> works;
                    for (auto& l : lists) works.push_back(pg->allreduce(l, o));
                    for (auto& w : works) w->wait();
                    stream.synchronize();
                    const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
                    best[static_cast<size_t>(r)] = std::min(best[static_cast<size_t>(r)], us / buckets);
                }
                stream.synchronize();
                pg->barrier()->wait();
            } catch (const std::exception& e) {
                errs[static_cast<size_t>(r)] = e.what();
            }
        });
    for (auto& t : ts) t.join();
    for (auto& e : errs)
        if (!e.empty()) throw mccl::MCCLError(e);
    return best;
}

// The byte transport with PeerMesh's interface, between `world` threads.
//  "ring":    `rounds` ring steps as the reference's allreduce_ring issues them (send to
//             the right neighbour, receive from the left; AllreduceAlgos.cpp:62-69) with
//             messages of growing length; every rank checks what it received byte by byte.
//  "kept":    the same with send_kept: the payload is not copied, and the receiver's copy
//             must release the transport's hold on the buffer.
//  "short":   the receiver expects more bytes than were sent.
//  "silent":  nobody sends; recv must time out and leave the mesh usable for a later exchange.
std::vector<std::string> peer_wire_probe(const std::string& mode, int world, int rounds, int timeout_ms) {
    auto mesh = mccl::LocalMesh::create(mccl::LocalMesh::fresh_key(), world);
    std::vector<std::string> out(static_cast<size_t>(world));
    std::vector<std::thread> ts;
    auto pattern = [](int from, int round, size_t i) { return static_cast<uint8_t>(from * 31 + round * 7 + i * 13 + 1); };
    for (int r = 0; r < world; ++r)
        ts.emplace_back([&, r] {
            mccl::LocalPeer peer(mesh, r, std::chrono::milliseconds(timeout_ms));
            const int right = (r + 1) % world, left = (r + world - 1) % world;
            try {
                if (mode == "silent") {
                    std::string first;
                    uint8_t b = 0;
                    try {
                        peer.recv(left, &b, 1);
                        first = "received";
                    } catch (const mccl::TimeoutError& e) {
                        first = "timeout";
                    }
                    // nobody sends before everybody has seen the silence
                    mesh->rendezvous(r, mccl::Contribution{}, std::chrono::milliseconds(20000),
                                     [](const std::vector<mccl::Contribution>&) {});
                    uint8_t mine = static_cast<uint8_t>(r + 1), theirs = 0;
                    mccl::LocalPeer patient(mesh, r, std::chrono::milliseconds(20000));
                    patient.send(right, &mine, 1);
                    patient.recv(left, &theirs, 1);
                    out[static_cast<size_t>(r)] = first + ":" + std::to_string(theirs);
                    return;
                }
                if (mode == "short") {
                    uint8_t three[3] = {1, 2, 3}, four[4] = {0, 0, 0, 0};
                    peer.send(right, three, 3);
                    peer.recv(left, four, 4);
                    out[static_cast<size_t>(r)] = "accepted";
                    return;
                }
                long held = 0;
                std::vector<std::shared_ptr<std::vector<uint8_t>>> sent;
                for (int i = 0; i < rounds; ++i) {
                    const size_t len = static_cast<size_t>(i) * 1000 + (i == 0 ? 0 : 17);  // the first message is empty
                    auto buf = std::make_shared<std::vector<uint8_t>>(len);
                    for (size_t k = 0; k < len; ++k) (*buf)[k] = pattern(r, i, k);
                    if (mode == "kept")
                        peer.send_kept(right, buf->data(), len, buf);
                    else
                        peer.send(right, buf->data(), len);
                    if (mode != "kept") std::fill(buf->begin(), buf->end(), 0);  // a copy was taken: ours to reuse
                    std::vector<uint8_t> got(len, 0xEE);
                    peer.recv(left, got.data(), len);
                    for (size_t k = 0; k < len; ++k)
                        if (got[k] != pattern(left, i, k)) throw mccl::MCCLError("wrong byte in message " + std::to_string(i));
                    if (mode == "kept") sent.push_back(buf);
                }
                if (mode == "kept") {
                    // a message is released when its receiver's recv returns: once every rank
                    // has finished its rounds nobody but the sender may hold one
                    mesh->rendezvous(r, mccl::Contribution{}, std::chrono::milliseconds(20000),
                                     [](const std::vector<mccl::Contribution>&) {});
                    for (auto& b : sent)
                        if (b.use_count() != 1) ++held;
                }
                out[static_cast<size_t>(r)] = "ok:" + std::to_string(held);
            } catch (const std::exception& e) {
                out[static_cast<size_t>(r)] = e.what();
            }
        });
    for (auto& t : ts) t.join();
    return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "mccl_amd native backend: c10d ProcessGroup over libmcclx";
    py::register_exception<mccl::MCCLError>(m, "MCCLError", PyExc_RuntimeError);
    mccl::set_blocking_hooks({&gil_release_if_held, &gil_take_back});
    install_abort_backtrace();

    m.def("_create_process_group_mccl",
          [](const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
             std::chrono::milliseconds timeout) -> c10::intrusive_ptr<c10d::Backend> {
              mccl::ProcessGroupMCCL::Options opts;
              opts.timeout = timeout;
              return c10::make_intrusive<mccl::ProcessGroupMCCL>(store, rank, size, opts);
          },
          py::arg("store"), py::arg("rank"), py::arg("size"),
          py::arg("timeout") = std::chrono::milliseconds(30 * 60 * 1000),
          py::call_guard<py::gil_scoped_release>(),
          "Factory used by torch.distributed.Backend.register_backend('mccl').");

    m.def("_last_algo", [](const c10::intrusive_ptr<c10d::Backend>& pg) {
        auto* p = dynamic_cast<mccl::ProcessGroupMCCL*>(pg.get());
        return p ? p->lastAlgo() : -1;
    });
    m.def("_graph_hits", [](const c10::intrusive_ptr<c10d::Backend>& pg) {
        auto* p = dynamic_cast<mccl::ProcessGroupMCCL*>(pg.get());
        return p ? p->graphHits() : uint64_t(0);
    });

    m.def("_async_stats", [](const c10::intrusive_ptr<c10d::Backend>& pg) {
        auto* p = dynamic_cast<mccl::ProcessGroupMCCL*>(pg.get());
        return p ? p->asyncStats() : std::pair<uint64_t, uint64_t>(0, 0);
    });
    m.def("_wire_stats", [](const c10::intrusive_ptr<c10d::Backend>& pg) {
        auto* p = dynamic_cast<mccl::ProcessGroupMCCL*>(pg.get());
        return p ? p->wireStats() : std::vector<double>{};
    });
    m.def("_launch_count", [](const c10::intrusive_ptr<c10d::Backend>& pg) {
        auto* p = dynamic_cast<mccl::ProcessGroupMCCL*>(pg.get());
        return p ? p->launchCount() : uint64_t(0);
    });

    m.def("_phase_stats", [](bool reset) {
        // phase -> (calls, total microseconds) since the last reset; all zero unless MCCL_PHASE_STATS=1
        py::dict d;
        for (int p = 0; p < mccl::phases::kCount; ++p)
            d[mccl::phases::name(p)] = py::make_tuple(mccl::phases::totals().calls[p].load(),
                                                      static_cast<double>(static_cast<int64_t>(mccl::phases::totals().ns[p].load())) * 1e-3);
        if (reset) mccl::phases::reset();
        return d;
    }, py::arg("reset") = false);
    m.def("_test_progress_order", &progress_order, py::arg("n"), py::arg("throw_mask") = 0,
          py::arg("use_destructor") = false, py::call_guard<py::gil_scoped_release>());
    m.def("_test_log", [](int level, const std::string& text) {
        mccl::log::emit(level, "bindings.cpp", 0, "%s", text.c_str());
        return mccl::log::enabled(level);
    });
    m.def("_test_progress_shutdown_while_task_needs_gil", &progress_shutdown_while_task_needs_gil);
    m.def("_test_progress_self_shutdown", &progress_self_shutdown, py::arg("mode"),
          py::call_guard<py::gil_scoped_release>());
    m.def("_test_terminate", [](const std::string& what) {
        // ends the process (tests run it in a child): an exception nobody catches, on a native thread
        std::thread t([what] { throw mccl::MCCLError(what); });
        t.join();
    }, py::call_guard<py::gil_scoped_release>());
    m.def("_test_progress_submit_latency_us", &progress_submit_latency_us,
          py::call_guard<py::gil_scoped_release>());
    m.def("_test_work", &work_probe, py::arg("mode"), py::arg("wait_ms") = 1000,
          py::call_guard<py::gil_scoped_release>());
    m.def("_allreduce_rate", &allreduce_rate_probe, py::arg("world"), py::arg("numel"), py::arg("buckets") = 8,
          py::arg("rounds") = 4, py::call_guard<py::gil_scoped_release>(),
          "Microseconds per allreduce, per rank, with the ranks as native threads of this process.");
    m.def("_test_peer_wire", &peer_wire_probe, py::arg("mode"), py::arg("world") = 3, py::arg("rounds") = 6,
          py::arg("timeout_ms") = 5000, py::call_guard<py::gil_scoped_release>());
    m.def("_test_mesh", &mesh_probe, py::arg("world"), py::arg("rounds") = 3, py::arg("absent") = -1,
          py::arg("timeout_ms") = 2000, py::arg("leader_throws") = false, py::arg("late_ms") = -1,
          py::call_guard<py::gil_scoped_release>());
}
