// null_mcclx.cpp -- a HOST stand-in of the kernel layer of include/mcclx.h, for sanitizer runs of
// the c10d backend without a GPU (tests/native/pg_stress.cpp).  The chunk scheduler
// (mccl_amd/csrc/mcclx_sched.cpp) is the real one and sits on top of this file.
//
// A context is a reduce queue as the library's is: launches return at once and run later, in order,
// on a thread of the context's own (the "device"); tickets, drains and cross-queue waits order the
// host and other queues against it.  Arithmetic is done on host memory for what the stress test
// checks -- fp32 sums with scale and fan-out, copies -- and skipped for everything else.  This is
// test infrastructure: nothing in the product builds or loads it.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "mcclx.h"

namespace {
thread_local std::string g_err;

struct Marker {
    std::mutex mu;
    std::condition_variable cv;
    bool done = false;
    void set() {
        {
            std::lock_guard<std::mutex> lk(mu);
            done = true;
        }
        cv.notify_all();
    }
    void wait() {
        std::unique_lock<std::mutex> lk(mu);
        cv.wait(lk, [&] { return done; });
    }
    bool test() {
        std::lock_guard<std::mutex> lk(mu);
        return done;
    }
};
}  // namespace

struct mcclx_graph {
    std::vector<std::function<void()>> work;
};

struct mcclx_ctx {
    std::mutex mu;
    std::condition_variable wake;
    std::deque<std::function<void()>> queue;
    bool closing = false;
    std::thread device;
    std::atomic<uint64_t> launches{0};
    std::map<uint64_t, std::shared_ptr<Marker>> tickets;
    uint64_t next_ticket = 1;
    bool recording = false;
    std::vector<std::function<void()>> recorded;
    std::map<void*, uint64_t> host_allocs;

    mcclx_ctx() {
        device = std::thread([this] {
            std::unique_lock<std::mutex> lk(mu);
            for (;;) {
                wake.wait(lk, [&] { return closing || !queue.empty(); });
                if (queue.empty()) return;
                auto f = std::move(queue.front());
                queue.pop_front();
                lk.unlock();
                f();
                f = nullptr;
                lk.lock();
            }
        });
    }
    ~mcclx_ctx() {
        {
            std::lock_guard<std::mutex> lk(mu);
            closing = true;
        }
        wake.notify_all();
        device.join();
    }
    void launch(std::function<void()> f, bool counts = true) {
        if (counts) ++launches;
        std::lock_guard<std::mutex> lk(mu);
        if (recording) {
            recorded.push_back(std::move(f));
            return;
        }
        queue.push_back(std::move(f));
        wake.notify_one();
    }
    std::shared_ptr<Marker> marker() {
        auto m = std::make_shared<Marker>();
        {
            std::lock_guard<std::mutex> lk(mu);
            queue.push_back([m] { m->set(); });
        }
        wake.notify_one();
        return m;
    }
};

namespace {
std::mutex g_ctx_mu;
std::map<void*, mcclx_ctx*> g_streams;  // a context's "stream" is its own address

bool known_stream(void* s, mcclx_ctx** out) {
    std::lock_guard<std::mutex> lk(g_ctx_mu);
    auto it = g_streams.find(s);
    if (it == g_streams.end()) return false;
    *out = it->second;
    return true;
}

size_t esize(int dtype) { return dtype == MCCLX_F32 ? 4 : 2; }
}  // namespace

extern "C" {

int mcclx_fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = std::string("[MCCL] ") + buf;
    return code;
}
const char* mcclx_last_error(void) { return g_err.c_str(); }
int mcclx_abi_version(void) { return MCCLX_ABI_VERSION; }

int mcclx_init(int device, mcclx_ctx** out) {
    if (device != 0) return mcclx_fail(MCCLX_ERR_INVALID, "device %d out of range (1 visible)", device);
    auto* c = new mcclx_ctx();
    std::lock_guard<std::mutex> lk(g_ctx_mu);
    g_streams[c] = c;
    *out = c;
    return MCCLX_OK;
}
int mcclx_init_on_stream(int device, void*, mcclx_ctx** out) { return mcclx_init(device, out); }
int mcclx_destroy(mcclx_ctx* c) {
    if (!c) return MCCLX_OK;
    {
        std::lock_guard<std::mutex> lk(g_ctx_mu);
        g_streams.erase(c);
    }
    for (auto& kv : c->host_allocs) free(kv.first);
    delete c;  // joins the device thread: everything queued has run
    return MCCLX_OK;
}
void* mcclx_queue_stream(mcclx_ctx* c) { return c; }
int mcclx_device_cus(mcclx_ctx*) { return 256; }
uint64_t mcclx_launch_count(mcclx_ctx* c) { return c ? c->launches.load() : 0; }
uint64_t mcclx_hold_launch_count(mcclx_ctx*) { return 0; }
int mcclx_set_hold(mcclx_ctx*, int) { return MCCLX_OK; }
int mcclx_hold_model(mcclx_ctx*, uint32_t* a, uint32_t* b) {
    if (a) *a = 40;
    if (b) *b = 72000;
    return 0;
}

int mcclx_fold_batched(mcclx_ctx* c, const mcclx_plan* plan, const mcclx_seg* segs, uint32_t nseg) {
    if (!c || !plan) return mcclx_fail(MCCLX_ERR_STATE, "context is null");
    const mcclx_plan p = *plan;
    std::vector<mcclx_seg> s(segs, segs + nseg);
    c->launch([p, s] {
        if (p.dtype != MCCLX_F32 || (p.op != MCCLX_SUM && p.op != MCCLX_AVG)) return;  // not checked by the test
        const int fan = (p.flags & MCCLX_PLAN_FANOUT_MASK) >> MCCLX_PLAN_FANOUT_SHIFT;
        const float scale = (float)p.scale;
        for (const mcclx_seg& g : s)
            for (uint64_t i = 0; i < g.count; ++i) {
                float acc = static_cast<const float*>(g.in[0])[i];
                for (int k = 1; k < p.k; ++k) acc += static_cast<const float*>(g.in[k])[i];
                if (p.scale_mode != MCCLX_SCALE_NONE) acc *= scale;
                if (g.out) static_cast<float*>(g.out)[i] = acc;
                for (int f = 0; f < fan; ++f) static_cast<float*>(const_cast<void*>(g.in[p.k + f]))[i] = acc;
            }
    });
    return MCCLX_OK;
}
int mcclx_fold(mcclx_ctx* c, const mcclx_plan* plan, const mcclx_seg* seg) { return mcclx_fold_batched(c, plan, seg, 1); }
int mcclx_fold_batched_noalloc(mcclx_ctx* c, const mcclx_plan* plan, const mcclx_seg* segs, uint32_t nseg) {
    return mcclx_fold_batched(c, plan, segs, nseg);
}
int mcclx_reduce(mcclx_ctx* c, void* dst, const void* src, int dtype, uint64_t count, int op) {
    mcclx_plan p;
    memset(&p, 0, sizeof p);
    p.dtype = dtype;
    p.k = 2;
    p.op = op;
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = dst;
    s.in[0] = dst;
    s.in[1] = src;
    s.count = count;
    return mcclx_fold_batched(c, &p, &s, 1);
}
int mcclx_scale(mcclx_ctx* c, void* buf, int dtype, uint64_t count, double scale, int scale_mode) {
    mcclx_plan p;
    memset(&p, 0, sizeof p);
    p.dtype = dtype;
    p.k = 1;
    p.scale = scale;
    p.scale_mode = scale_mode;
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = buf;
    s.in[0] = buf;
    s.count = count;
    return mcclx_fold_batched(c, &p, &s, 1);
}
int mcclx_accumulate_scale(mcclx_ctx* c, void* dst, const void* src, int dtype, uint64_t count, double scale) {
    mcclx_plan p;
    memset(&p, 0, sizeof p);
    p.dtype = dtype;
    p.k = 2;
    p.scale = scale;
    p.scale_mode = MCCLX_SCALE_TENSOR;
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = dst;
    s.in[0] = dst;
    s.in[1] = src;
    s.count = count;
    return mcclx_fold_batched(c, &p, &s, 1);
}
int mcclx_encode_bf16(mcclx_ctx* c, void*, const void*, uint64_t) {
    c->launch([] {});
    return MCCLX_OK;
}
int mcclx_decode_bf16(mcclx_ctx* c, void*, const void*, uint64_t) {
    c->launch([] {});
    return MCCLX_OK;
}
int mcclx_batch_begin(mcclx_ctx*, const char*) { return MCCLX_OK; }
int mcclx_batch_end(mcclx_ctx*) { return MCCLX_OK; }

int mcclx_copy(mcclx_ctx* c, void* dst, const void* src, uint64_t nbytes) {
    if (!c) return mcclx_fail(MCCLX_ERR_STATE, "context is null");
    if (nbytes == 0 || dst == src) return MCCLX_OK;
    c->launch([dst, src, nbytes] { memmove(dst, src, nbytes); });
    return MCCLX_OK;
}
int mcclx_copy_batched(mcclx_ctx* c, const mcclx_copy_desc* d, uint32_t n) {
    std::vector<mcclx_copy_desc> v(d, d + n);
    c->launch([v] {
        for (auto& x : v)
            if (x.nbytes && x.dst != x.src) memmove(x.dst, x.src, x.nbytes);
    });
    return MCCLX_OK;
}

int mcclx_queue_drain(mcclx_ctx* c) {
    if (!c) return mcclx_fail(MCCLX_ERR_STATE, "context is null");
    c->marker()->wait();
    return MCCLX_OK;
}
int mcclx_queue_wait_stream(mcclx_ctx* c, void* producer) {
    mcclx_ctx* p = nullptr;
    if (!producer || producer == c || !known_stream(producer, &p)) return MCCLX_OK;  // the null stream: host code, already done
    auto m = p->marker();
    c->launch([m] { m->wait(); }, false);
    return MCCLX_OK;
}
int mcclx_stream_wait_queue(mcclx_ctx* c, void* consumer) {
    mcclx_ctx* q = nullptr;
    if (!consumer || consumer == c || !known_stream(consumer, &q)) return MCCLX_OK;
    auto m = c->marker();
    q->launch([m] { m->wait(); }, false);
    return MCCLX_OK;
}
int mcclx_event_record(mcclx_ctx* c, uint64_t* ticket) {
    auto m = c->marker();
    std::lock_guard<std::mutex> lk(c->mu);
    *ticket = c->next_ticket++;
    c->tickets[*ticket] = m;
    return MCCLX_OK;
}
int mcclx_event_query(mcclx_ctx* c, uint64_t ticket, int* done) {
    std::shared_ptr<Marker> m;
    {
        std::lock_guard<std::mutex> lk(c->mu);
        auto it = c->tickets.find(ticket);
        if (it == c->tickets.end()) {
            *done = 1;
            return MCCLX_OK;
        }
        m = it->second;
    }
    *done = m->test() ? 1 : 0;
    return MCCLX_OK;
}
int mcclx_event_wait(mcclx_ctx* c, uint64_t ticket) {
    if (ticket == 0) return MCCLX_OK;
    std::shared_ptr<Marker> m;
    {
        std::lock_guard<std::mutex> lk(c->mu);
        auto it = c->tickets.find(ticket);
        if (it == c->tickets.end()) return MCCLX_OK;
        m = it->second;
    }
    m->wait();
    std::lock_guard<std::mutex> lk(c->mu);
    c->tickets.erase(ticket);
    return MCCLX_OK;
}

int mcclx_graph_begin(mcclx_ctx* c) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (c->recording) return mcclx_fail(MCCLX_ERR_STATE, "graph recording already active");
    c->recording = true;
    return MCCLX_OK;
}
int mcclx_graph_end(mcclx_ctx* c, mcclx_graph** out) {
    std::lock_guard<std::mutex> lk(c->mu);
    if (!c->recording) return mcclx_fail(MCCLX_ERR_STATE, "graph_end without graph_begin");
    c->recording = false;
    auto* g = new mcclx_graph();
    g->work.swap(c->recorded);
    *out = g;
    return MCCLX_OK;
}
int mcclx_graph_launch(mcclx_ctx* c, mcclx_graph* g) {
    for (auto& f : g->work) c->launch(f, false);
    return MCCLX_OK;
}
int mcclx_graph_destroy(mcclx_ctx* c, mcclx_graph* g) {
    if (c) mcclx_queue_drain(c);
    delete g;
    return MCCLX_OK;
}

int mcclx_host_alloc(mcclx_ctx* c, uint64_t nbytes, void** host_ptr, void** device_ptr) {
    void* p = malloc(nbytes);
    if (!p) return mcclx_fail(MCCLX_ERR_NOMEM, "malloc(%llu) failed", (unsigned long long)nbytes);
    std::lock_guard<std::mutex> lk(c->mu);
    c->host_allocs[p] = nbytes;
    *host_ptr = *device_ptr = p;
    return MCCLX_OK;
}
int mcclx_host_free(mcclx_ctx* c, void* p) {
    if (!p) return MCCLX_OK;
    mcclx_queue_drain(c);
    std::lock_guard<std::mutex> lk(c->mu);
    c->host_allocs.erase(p);
    free(p);
    return MCCLX_OK;
}
int mcclx_stage_for_send(mcclx_ctx* c, const void* src, uint64_t, void** host_ptr) {
    mcclx_queue_drain(c);
    *host_ptr = const_cast<void*>(src);
    return MCCLX_OK;
}
int mcclx_unstage_from_recv(mcclx_ctx* c, void* dst, const void* src, uint64_t nbytes) {
    std::vector<char> keep(static_cast<const char*>(src), static_cast<const char*>(src) + nbytes);
    c->launch([dst, keep] { memcpy(dst, keep.data(), keep.size()); });
    return MCCLX_OK;
}

}  // extern "C"
