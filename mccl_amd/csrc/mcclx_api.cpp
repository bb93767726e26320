// mcclx_api.cpp -- the C ABI (include/mcclx.h): context, reduce queue, launch
// validation, host-buffer interop.  Host-only code; kernels live in
// fold_kernels.hip / copy_kernel.hip behind fold_launch.h.

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <chrono>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "fold_launch.h"
#include "mcclx.h"
#include "mcclx_internal.h"

namespace {
thread_local std::string g_err;
}

extern "C" int mcclx_fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    // same prefix as the reference's MCCLError (csrc/common/Errors.hpp:9-13)
    g_err = std::string("[MCCL] ") + buf;
    return code;
}

namespace {

#define fail mcclx_fail

#define HIP_TRY(expr)                                                                  \
    do {                                                                               \
        hipError_t _e = (expr);                                                        \
        if (_e != hipSuccess)                                                          \
            return fail(MCCLX_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

constexpr int kTableSlots = 4;
constexpr uint64_t kMaxMappedItems = 1u << 20;  // work items up to which a launch carries an item -> segment map (8 B each)

struct TableSlot {
    void* host = nullptr;  // pinned staging
    void* dev = nullptr;
    size_t cap = 0;
    hipEvent_t done = nullptr;  // recorded after the launch that read `dev`
    bool pending = false;
};

}  // namespace

struct mcclx_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<void*> tables;  // descriptor tables recorded launches read
};

struct mcclx_ctx {
    bool capturing = false;
    std::vector<void*> capture_tables;
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    int cus = 0;
    uint32_t max_blocks = 0;
    std::atomic<uint64_t> launches{0};  // kernel launches issued (diagnostic)
    uint32_t few_max = mcclx::kFewSegs;  // segments up to which descriptors travel in the kernel arguments
    bool validate = false;
    // reads-then-writes launches (LaunchParams): least bytes read, and the gate's model
    uint64_t hold_min_read_bytes = 10ull << 20;
    uint32_t hold_latency_ticks = 40, hold_bytes_per_tick = 72000;  // in ticks of 100 MHz
    uint32_t wall_khz = 100000;                                      // the device's wall clock
    bool hold_measured = false;        // the gate's rate was measured on this device (not the default)
    std::atomic<bool> hold_enabled{true};  // a completer thread may switch it while ranks launch
    std::atomic<uint64_t> hold_launches{0};
    bool batch_active = false;
    std::string batch_label;
    std::mutex mu;
    struct Ticket {
        hipEvent_t ev = nullptr;
        int waiters = 0;  // threads inside hipEventSynchronize on `ev`
    };
    std::unordered_map<uint64_t, Ticket> tickets;
    std::vector<hipEvent_t> free_events;
    uint64_t next_ticket = 1;
    TableSlot slots[kTableSlots];
    int next_slot = 0;
    std::unordered_map<void*, uint64_t> host_allocs;
    // cross-stream ordering events, used round robin so that an event is not
    // re-recorded until 15 later waits have been issued
    hipEvent_t xev[16] = {};
    int xnext = 0;
    hipStream_t upload_stream = nullptr;  // blocking table uploads while the queue is recording
    // staging pool (MPSInterop.mm:47-204): one grow-only pinned buffer for sends,
    // two fixed pinned chunks + events for pipelined receives from pageable memory
    void* stage_send = nullptr;
    size_t stage_send_cap = 0;
    void* stage_recv[2] = {nullptr, nullptr};
    hipEvent_t stage_recv_done[2] = {nullptr, nullptr};
    bool stage_recv_pending[2] = {false, false};
    void* static_table = nullptr;  // this device's copy of the static descriptor table (static_table.hip)
};

namespace {

bool dtype_ok(int d) { return d == MCCLX_F32 || d == MCCLX_F16 || d == MCCLX_BF16; }

struct DeviceGuard {
    int prev = -1;
    bool ok = true;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        if (prev != dev) ok = (hipSetDevice(dev) == hipSuccess);
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

// binary16 <- binary64 in one rounding (the `(__fp16)scale` of
// MetalKernels.mm:387,656): scale into the target's quantum, round to nearest
// even with nearbyint (exact in double), rebuild the pattern.
uint16_t f64_to_f16_bits(double x) {
    uint16_t sign = std::signbit(x) ? 0x8000u : 0u;
    double a = std::fabs(x);
    if (std::isnan(x)) return (uint16_t)(sign | 0x7E00u);
    if (std::isinf(x)) return (uint16_t)(sign | 0x7C00u);
    if (a == 0.0) return sign;
    int e;
    double m = std::frexp(a, &e);  // a = m * 2^e, m in [0.5, 1)
    if (e < -13) {                 // below the smallest normal 2^-14: fixed quantum 2^-24
        double q = std::nearbyint(std::ldexp(a, 24));
        return (uint16_t)(sign | (uint16_t)q);  // q == 1024 is the smallest normal
    }
    double q = std::nearbyint(std::ldexp(m, 11));  // 11 significant bits: [1024, 2048]
    if (q == 2048.0) {
        q = 1024.0;
        e += 1;
    }
    int field = e + 14;
    if (field >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | (field << 10) | ((int)q - 1024));
}

float f16_bits_to_f32(uint16_t h) {
    int ex = (h >> 10) & 0x1F, man = h & 0x3FF;
    double v;
    if (ex == 0)
        v = std::ldexp((double)man, -24);
    else if (ex == 31)
        v = man ? NAN : INFINITY;
    else
        v = std::ldexp((double)(man | 0x400), ex - 25);
    return (float)((h & 0x8000) ? -v : v);
}

// The multiplier each scale kernel receives, as an fp32 value
// (MetalKernels.mm:384-398 tensor variant, :655-666 view variant).
int scale_value(int dtype, double scale, int mode, float* out) {
    float f = (float)scale;
    uint32_t bits;
    memcpy(&bits, &f, 4);
    if (dtype == MCCLX_F32) {
        *out = f;
    } else if (dtype == MCCLX_F16) {
        *out = f16_bits_to_f32(f64_to_f16_bits(scale));
    } else if (mode == MCCLX_SCALE_VIEW) {
        bits &= 0xFFFF0000u;  // bits >> 16, truncation
        memcpy(out, &bits, 4);
    } else if (mode == MCCLX_SCALE_TENSOR) {
        if ((bits & 0x7FFFFFFFu) > 0x7F800000u)
            bits = 0x7FC00000u;
        else
            bits = (bits + 0x7FFFu + ((bits >> 16) & 1u)) & 0xFFFF0000u;
        memcpy(out, &bits, 4);
    } else {
        return fail(MCCLX_ERR_INVALID, "scale_mode %d is not VIEW or TENSOR", mode);
    }
    return MCCLX_OK;
}

int normalize_op(int op, int* out) {
    switch (op) {
        case MCCLX_SUM:
        case MCCLX_AVG: *out = MCCLX_SUM; return MCCLX_OK;  // select_op_pipeline, MetalKernels.mm:609-611
        case MCCLX_PRODUCT:
        case MCCLX_MIN:
        case MCCLX_MAX: *out = op; return MCCLX_OK;
        default:
            // MetalKernels.mm:546-548
            return fail(MCCLX_ERR_UNSUPPORTED, "Unsupported ReduceOp: %d", op);
    }
}

int check_plan(const mcclx_plan* p, mcclx::PlanKey* key, float* scale_f, int* has_scale, int* fan) {
    if (!p) return fail(MCCLX_ERR_INVALID, "plan is null");
    if (p->flags & ~(MCCLX_PLAN_ACC_IS_SRC | MCCLX_PLAN_FANOUT_MASK))
        return fail(MCCLX_ERR_INVALID, "plan.flags=%d has unknown bits", p->flags);
    *fan = (p->flags & MCCLX_PLAN_FANOUT_MASK) >> MCCLX_PLAN_FANOUT_SHIFT;
    if (!dtype_ok(p->dtype))
        return fail(MCCLX_ERR_UNSUPPORTED, "No kernel for dtype code %d", p->dtype);
    if (p->k < 1 || p->k > MCCLX_MAX_INPUTS)
        return fail(MCCLX_ERR_INVALID, "plan.k=%d outside 1..%d", p->k, MCCLX_MAX_INPUTS);
    int op;
    if (int rc = normalize_op(p->op, &op)) return rc;
    if (p->io < MCCLX_IO_PURE || p->io > MCCLX_IO_ALL_F32)
        return fail(MCCLX_ERR_INVALID, "plan.io=%d unknown", p->io);
    if (p->io != MCCLX_IO_PURE && p->dtype != MCCLX_BF16)
        return fail(MCCLX_ERR_UNSUPPORTED, "fp32 operands/outputs need the bf16 wire dtype");
    if (p->topo != MCCLX_TOPO_FOLD && p->topo != MCCLX_TOPO_BINOMIAL)
        return fail(MCCLX_ERR_INVALID, "plan.topo=%d unknown", p->topo);
    if (p->acc != MCCLX_ACC_STEP && p->acc != MCCLX_ACC_F32)
        return fail(MCCLX_ERR_INVALID, "plan.acc=%d unknown", p->acc);
    if (op != MCCLX_SUM && (p->io != MCCLX_IO_PURE || p->acc != MCCLX_ACC_STEP))
        return fail(MCCLX_ERR_UNSUPPORTED,
                    "MIN/MAX/PRODUCT fold same-dtype operands with per-step rounding only (PURE, STEP)");
    if (p->dtype == MCCLX_F16 && p->acc != MCCLX_ACC_STEP)
        return fail(MCCLX_ERR_UNSUPPORTED, "fp16 folds round after every step (STEP) only");
    if (p->io == MCCLX_IO_OWN_LAST_F32 && p->topo == MCCLX_TOPO_BINOMIAL)
        return fail(MCCLX_ERR_UNSUPPORTED, "the tree reduces into rank 0: own operand is first");
    if ((p->flags & MCCLX_PLAN_ACC_IS_SRC) && p->topo == MCCLX_TOPO_BINOMIAL && p->k >= 4)
        return fail(MCCLX_ERR_UNSUPPORTED, "the tree reduces into the surviving rank: its partial result is dst");
    // SUM and PRODUCT do not depend on the operand roles; MIN and MAX do
    if ((p->flags & MCCLX_PLAN_ACC_IS_SRC) && (op == MCCLX_MIN || op == MCCLX_MAX))
        op = (op == MCCLX_MIN) ? mcclx::MCCLX_MIN_ACC_SRC : mcclx::MCCLX_MAX_ACC_SRC;
    int acc = (p->dtype == MCCLX_F32) ? MCCLX_ACC_STEP : p->acc;  // fp32 has no rounding to skip
    *key = mcclx::PlanKey{p->dtype, p->io, p->k, (p->k >= 4) ? p->topo : MCCLX_TOPO_FOLD, op, acc};
    if (*fan && (!mcclx::fan_plan_ok(*key) || p->k + *fan > MCCLX_MAX_INPUTS))
        return fail(MCCLX_ERR_UNSUPPORTED,
                    "fan-out (%d further destinations) needs a sum with per-step rounding, an output of the "
                    "operands' form or fp32 next to an fp32 operand, and k + fan <= %d (k=%d)",
                    *fan, MCCLX_MAX_INPUTS, p->k);
    *has_scale = p->scale_mode != MCCLX_SCALE_NONE;
    *scale_f = 1.0f;
    if (*has_scale) {
        if (int rc = scale_value(p->dtype, p->scale, p->scale_mode, scale_f)) return rc;
        // fp32 accumulation keeps everything before its one rounding in fp32, the factor included
        if (acc == MCCLX_ACC_F32) *scale_f = (float)p->scale;
    }
    return MCCLX_OK;
}

bool in_is_f32(const mcclx::PlanKey& k, int i) {
    return k.dtype == MCCLX_F32 || k.io == MCCLX_IO_ALL_F32 || (k.io == MCCLX_IO_OWN_FIRST_F32 && i == 0) ||
           (k.io == MCCLX_IO_OWN_LAST_F32 && i == k.k - 1);
}

// Is [p, p+nbytes) inside one allocation the GPU can address?
int check_range(const void* p, uint64_t nbytes, const char* what, uint32_t seg) {
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(MCCLX_ERR_INVALID, "segment %u: %s=%p is not GPU-accessible memory", seg, what, p);
    }
    void* base = nullptr;
    size_t size = 0;
    if (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged) {
        if (hipMemGetAddressRange((hipDeviceptr_t*)&base, &size, (hipDeviceptr_t)p) != hipSuccess) {
            (void)hipGetLastError();
            return MCCLX_OK;  // range unknown: accept
        }
        const char* lo = static_cast<const char*>(base);
        const char* q = static_cast<const char*>(p);
        if (q < lo || q + nbytes > lo + size)
            return fail(MCCLX_ERR_INVALID,
                        "segment %u: %s=%p + %llu bytes runs past its allocation (%zu bytes at %p)",
                        seg, what, p, (unsigned long long)nbytes, size, base);
    }
    return MCCLX_OK;
}

int check_segs(mcclx_ctx* ctx, const mcclx::PlanKey& key, const mcclx_seg* segs, uint32_t nseg, int fan) {
    if (!segs && nseg) return fail(MCCLX_ERR_INVALID, "segment array is null");
    const bool out_f32 = key.dtype == MCCLX_F32 || key.io != MCCLX_IO_PURE;
    for (uint32_t s = 0; s < nseg; ++s) {
        const mcclx_seg& g = segs[s];
        if (g.count == 0) continue;
        if (!g.out && !g.wire_out) return fail(MCCLX_ERR_INVALID, "segment %u has no output", s);
        if (g.wire_out && key.dtype == MCCLX_F32)
            return fail(MCCLX_ERR_INVALID, "segment %u: wire_out needs a 16-bit arithmetic dtype", s);
        for (int i = 0; i < key.k; ++i) {
            if (!g.in[i]) return fail(MCCLX_ERR_INVALID, "segment %u: in[%d] is null", s, i);
            size_t al = in_is_f32(key, i) ? 4 : 2;
            if ((uintptr_t)g.in[i] % al)
                return fail(MCCLX_ERR_INVALID, "segment %u: in[%d]=%p is not element aligned", s, i,
                            g.in[i]);
        }
        if (g.out && (uintptr_t)g.out % (out_f32 ? 4 : 2))
            return fail(MCCLX_ERR_INVALID, "segment %u: out=%p is not element aligned", s, g.out);
        if (g.wire_out && (uintptr_t)g.wire_out % 2)
            return fail(MCCLX_ERR_INVALID, "segment %u: wire_out=%p is not element aligned", s,
                        g.wire_out);
        if (fan && !g.out) return fail(MCCLX_ERR_INVALID, "segment %u: fan-out needs `out`", s);
        for (int f = 0; f < fan; ++f) {
            const void* d = g.in[key.k + f];
            if (!d) return fail(MCCLX_ERR_INVALID, "segment %u: fan-out destination in[%d] is null", s, key.k + f);
            if ((uintptr_t)d % (out_f32 ? 4 : 2))
                return fail(MCCLX_ERR_INVALID, "segment %u: fan-out destination in[%d]=%p is not element aligned", s,
                            key.k + f, d);
            if (ctx->validate) {
                if (int rc = check_range(d, g.count * (out_f32 ? 4 : 2), "fan-out destination", s)) return rc;
                // a destination may BE one of the operands (each lane reads a packet before it
                // writes it); one that overlaps an operand at another offset would be read by
                // some lanes after other lanes have written it
                const char* d0 = static_cast<const char*>(d);
                const char* d1 = d0 + g.count * (out_f32 ? 4 : 2);
                for (int i = 0; i < key.k; ++i) {
                    const char* i0 = static_cast<const char*>(g.in[i]);
                    const char* i1 = i0 + g.count * (in_is_f32(key, i) ? 4 : 2);
                    if (d0 != i0 && d0 < i1 && i0 < d1)
                        return fail(MCCLX_ERR_INVALID,
                                    "segment %u: fan-out destination in[%d]=%p overlaps operand in[%d]=%p at another offset",
                                    s, key.k + f, d, i, g.in[i]);
                }
            }
        }
        if (ctx->validate) {
            for (int i = 0; i < key.k; ++i)
                if (int rc = check_range(g.in[i], g.count * (in_is_f32(key, i) ? 4 : 2), "in", s))
                    return rc;
            if (g.out)
                if (int rc = check_range(g.out, g.count * (out_f32 ? 4 : 2), "out", s)) return rc;
            if (g.wire_out)
                if (int rc = check_range(g.wire_out, g.count * 2, "wire_out", s)) return rc;
        }
    }
    return MCCLX_OK;
}

int launch_error(hipError_t e, const mcclx::PlanKey& k) {
    if (e == hipErrorInvalidValue)
        return fail(MCCLX_ERR_UNSUPPORTED, "No kernel for plan dtype=%d io=%d k=%d topo=%d op=%d acc=%d",
                    k.dtype, k.io, k.k, k.topo, k.op, k.acc);
    return fail(MCCLX_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
}

int ensure_slot(mcclx_ctx* ctx, TableSlot& sl, size_t need) {
    if (sl.pending) {
        HIP_TRY(hipEventSynchronize(sl.done));
        sl.pending = false;
    }
    if (sl.cap >= need) return MCCLX_OK;
    size_t cap = 1 << 16;
    while (cap < need) cap <<= 1;
    if (sl.host) HIP_TRY(hipHostFree(sl.host));
    if (sl.dev) HIP_TRY(hipFree(sl.dev));
    sl.host = sl.dev = nullptr;
    sl.cap = 0;
    HIP_TRY(hipHostMalloc(&sl.host, cap, hipHostMallocDefault));
    HIP_TRY(hipMalloc(&sl.dev, cap));
    if (!sl.done) HIP_TRY(hipEventCreateWithFlags(&sl.done, hipEventDisableTiming));
    sl.cap = cap;
    (void)ctx;
    return MCCLX_OK;
}

// Puts a descriptor table where a kernel can read it (caller holds ctx->mu).
// Outside a recording: the next slot of the pinned staging ring, copied to its
// device twin on the queue (`*slot` names it).  While recording: the launch needs a table that outlives this
// call, so it gets its own device buffer, filled now with a blocking copy
// (outside the recording) and owned by the graph; `*slot` stays null.
int stage_table(mcclx_ctx* ctx, const void* bytes, size_t nbytes, void** dev, TableSlot** slot) {
    *slot = nullptr;
    if (ctx->capturing) {
        void* d = nullptr;
        HIP_TRY(hipMalloc(&d, nbytes));
        // not the legacy stream: that one may not be touched while another stream records
        if (!ctx->upload_stream)
            HIP_TRY(hipStreamCreateWithFlags(&ctx->upload_stream, hipStreamNonBlocking));
        hipError_t ce = hipMemcpyAsync(d, bytes, nbytes, hipMemcpyHostToDevice, ctx->upload_stream);
        if (ce == hipSuccess) ce = hipStreamSynchronize(ctx->upload_stream);
        if (ce != hipSuccess) {
            (void)hipFree(d);
            return fail(MCCLX_ERR_HIP, "table upload failed: %s", hipGetErrorString(ce));
        }
        ctx->capture_tables.push_back(d);
        *dev = d;
        return MCCLX_OK;
    }
    // The queue may be a stream the caller owns (mcclx_init_on_stream) and is recording
    // into a graph of its own: a table upload recorded there would replay whatever the
    // staging ring holds at that time.  Such callers record through mcclx_graph_begin or
    // use the allocation-free entry point, whose table travels in kernel arguments.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone)
        return fail(MCCLX_ERR_STATE,
                    "a launch with a descriptor table cannot be recorded by a stream capture the library did not "
                    "start: record with mcclx_graph_begin, or use mcclx_fold_batched_noalloc");
    TableSlot& sl = ctx->slots[ctx->next_slot];
    ctx->next_slot = (ctx->next_slot + 1) % kTableSlots;
    if (int rc = ensure_slot(ctx, sl, nbytes)) return rc;
    memcpy(sl.host, bytes, nbytes);
    HIP_TRY(hipMemcpyAsync(sl.dev, sl.host, nbytes, hipMemcpyHostToDevice, ctx->stream));
    // The slot's pinned half is busy until this copy has run; its device half is only
    // touched on the queue, whose order keeps the next upload behind the launch that
    // reads this one.  Recorded here, so that no exit path of the caller can skip it.
    HIP_TRY(hipEventRecord(sl.done, ctx->stream));
    sl.pending = true;
    *dev = sl.dev;
    *slot = &sl;
    return MCCLX_OK;
}

// Descriptors in the kernel arguments (nseg <= kFewSegs).
int launch_by_value(mcclx_ctx* ctx, const mcclx::PlanKey& key, float scale_f, int has_scale,
                    const mcclx_seg* segs, uint32_t nseg, int fan) {
    mcclx::LaunchParams lp;
    lp.max_blocks = ctx->max_blocks;
    lp.fan = fan;
    lp.cus = ctx->cus;
    bool held = false;
    lp.held = &held;
    lp.hold_min_read_bytes = ctx->hold_enabled.load(std::memory_order_relaxed) ? ctx->hold_min_read_bytes : 0;
    lp.hold_latency_ticks = (uint32_t)((uint64_t)ctx->hold_latency_ticks * ctx->wall_khz / 100000);
    lp.hold_bytes_per_tick = (uint32_t)((uint64_t)ctx->hold_bytes_per_tick * 100000 / ctx->wall_khz);
    if (lp.hold_bytes_per_tick == 0) lp.hold_bytes_per_tick = 1;
    mcclx::FewArgs a;
    memset(&a, 0, sizeof a);
    for (uint32_t s = 0; s < nseg; ++s) memcpy(&a.seg[s], &segs[s], sizeof(mcclx_seg));
    a.scale = scale_f;
    a.has_scale = has_scale;
    a.nseg = (int32_t)nseg;
    lp.few = &a;
    hipError_t e = mcclx::launch_fold(ctx->stream, key, lp);
    if (e != hipSuccess) return launch_error(e, key);
    ++ctx->launches;
    if (held) ++ctx->hold_launches;
    return MCCLX_OK;
}

// By value the grid is (tiles of the longest segment) x (segments), so a launch whose
// segments differ wildly in length would consist mostly of blocks with nothing to do;
// such a launch takes a table, which has one block per tile.
bool even_enough(const mcclx::PlanKey& key, const mcclx_seg* segs, uint32_t nseg) {
    if (nseg <= 4) return true;
    uint64_t longest = 0, total = 0;
    for (uint32_t s = 0; s < nseg; ++s) {
        const uint64_t n = mcclx::items_for(key, segs[s].count);
        total += n;
        if (n > longest) longest = n;
    }
    return longest * nseg <= 4 * total + 64;
}

int fold_impl(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* segs, uint32_t nseg) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    mcclx::PlanKey key;
    float scale_f;
    int has_scale, fan;
    if (int rc = check_plan(plan, &key, &scale_f, &has_scale, &fan)) return rc;
    if (int rc = check_segs(ctx, key, segs, nseg, fan)) return rc;
    if (nseg == 0) return MCCLX_OK;
    DeviceGuard guard(ctx->device);
    if (!guard.ok) return fail(MCCLX_ERR_HIP, "hipSetDevice(%d) failed", ctx->device);

    mcclx::LaunchParams lp;
    lp.max_blocks = ctx->max_blocks;
    if (nseg <= ctx->few_max && even_enough(key, segs, nseg))
        return launch_by_value(ctx, key, scale_f, has_scale, segs, nseg, fan);

    // descriptor table: segs, then nseg+1 work-item prefix sums
    std::lock_guard<std::mutex> lk(ctx->mu);
    size_t seg_bytes = (size_t)nseg * sizeof(mcclx_seg);
    size_t pre_bytes = ((size_t)nseg + 1) * sizeof(uint64_t);
    std::vector<char> host(seg_bytes + pre_bytes);
    memcpy(host.data(), segs, seg_bytes);
    uint64_t* pre = reinterpret_cast<uint64_t*>(host.data() + seg_bytes);
    uint64_t total = 0, uniform = mcclx::items_for(key, segs[0].count);
    for (uint32_t s = 0; s < nseg; ++s) {
        pre[s] = total;
        uint64_t n = mcclx::items_for(key, segs[s].count);
        if (n != uniform) uniform = 0;
        total += n;
    }
    pre[nseg] = total;
    if (total == 0) return MCCLX_OK;
    if (total >> 31) return fail(MCCLX_ERR_INVALID, "fold: more than 2^31 work items in one launch");
    // Ragged segments: spell out (segment, tile) per work item, so that a block finds
    // its work with one load instead of a binary search through device memory
    // (measured on 4096 ragged messages: 3.9 -> 6.3 TB/s).
    const bool mapped = uniform == 0 && total <= kMaxMappedItems;
    const size_t map_off = host.size();
    if (mapped) {
        host.resize(map_off + (size_t)total * sizeof(uint2));
        pre = reinterpret_cast<uint64_t*>(host.data() + seg_bytes);
        uint2* map = reinterpret_cast<uint2*>(host.data() + map_off);
        for (uint32_t s = 0; s < nseg; ++s)
            for (uint64_t w = pre[s]; w < pre[s + 1]; ++w) map[w] = make_uint2(s, (uint32_t)(w - pre[s]));
    }
    void* dev = nullptr;
    TableSlot* slot = nullptr;
    if (int rc = stage_table(ctx, host.data(), host.size(), &dev, &slot)) return rc;
    mcclx::TableArgs t;
    t.segs = static_cast<const mcclx::SegArgs*>(dev);
    t.first_item = reinterpret_cast<const uint64_t*>(static_cast<char*>(dev) + seg_bytes);
    t.item_map = mapped ? reinterpret_cast<const uint2*>(static_cast<char*>(dev) + map_off) : nullptr;
    t.total_items = total;
    t.uniform_items = uniform;
    t.nseg = nseg;
    t.scale = scale_f;
    t.has_scale = has_scale;
    lp.table = &t;
    lp.fan = fan;
    hipError_t e = mcclx::launch_fold(ctx->stream, key, lp);
    if (e != hipSuccess) return launch_error(e, key);
    ++ctx->launches;
    return MCCLX_OK;
}

// The hold form's gate follows the device.  Its model -- no store before
// latency + bytes read / rate -- has one constant that differs from part to part and from
// one memory configuration to the next: the rate at which a launch's reads come in.  It is
// measured once per device and process, when the first context is made: read-only launches of
// two sizes (24 and 96 MiB) over a scratch buffer larger than the Infinity Cache (so they read
// HBM, as a gradient bucket does), the difference of their times over the difference of their
// sizes, after 20 ms of the same probe (a device that has been idle needs that long to reach its
// steady clocks); the figure repeats within 1 % from process to process.  On MI355X the best gate
// of a 25 MiB bucket, swept, sits at 760-775 ticks after a block's start, flat within 0.05 us
// across that range, 0.2 us worse 3 % earlier and 0.15 us worse 6 % later: 1.005 of the rate
// this probe measures, and that ratio is what carries over to another device.
// MCCLX_HOLD_CALIBRATE=0 keeps the defaults; the MCCLX_HOLD_* knobs override either.
struct HoldModel {
    uint32_t latency_ticks = 40;      // ticks of 100 MHz
    uint32_t bytes_per_tick = 72000;  // per tick of 100 MHz
    bool measured = false;
};
constexpr double kHoldGateRatio = 1.005;

HoldModel measure_hold_model() {  // the device is current
    HoldModel m;
    if (const char* v = getenv("MCCLX_HOLD_CALIBRATE"))
        if (v[0] == '0') return m;
    constexpr size_t kBig = 96u << 20, kMid = 60u << 20, kSmall = 24u << 20;  // the launches that hold read 10-100 MB
    constexpr int kCopies = 4;  // 384 MiB: more than the 256 MiB Infinity Cache
    char* buf = nullptr;
    hipStream_t st = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto cleanup = [&] {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        if (st) (void)hipStreamDestroy(st);
        if (buf) (void)hipFree(buf);
        (void)hipGetLastError();
    };
    if (hipMalloc(reinterpret_cast<void**>(&buf), kBig * kCopies) != hipSuccess ||
        hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        cleanup();
        return m;
    }
    bool ok = true;
    for (int i = 0; i < kCopies && ok; ++i)  // a payload of mixed bits (zero-filled memory reads faster)
        ok = mcclx::launch_stream_probe(st, buf + (size_t)i * kBig, kBig, true) == hipSuccess;
    // A device that has been idle takes some tens of milliseconds of work to reach its steady
    // clocks, and the first context of a process is often its first work: 20 ms of the probe first.
    for (const auto until = std::chrono::steady_clock::now() + std::chrono::milliseconds(20);
         ok && std::chrono::steady_clock::now() < until;) {
        for (int i = 0; i < 16 && ok; ++i)
            ok = mcclx::launch_stream_probe(st, buf + (size_t)(i % kCopies) * kBig, kBig, false) == hipSuccess;
        ok = ok && hipStreamSynchronize(st) == hipSuccess;
    }
    auto timed = [&](size_t nbytes) -> double {  // microseconds per launch, best of five rounds
        double best = 1e30;
        for (int round = 0; round < 5 && ok; ++round) {
            constexpr int kReps = 32;
            for (int i = 0; i < 4 && ok; ++i)
                ok = mcclx::launch_stream_probe(st, buf + (size_t)(i % kCopies) * kBig, nbytes, false) == hipSuccess;
            ok = ok && hipEventRecord(e0, st) == hipSuccess;
            for (int i = 0; i < kReps && ok; ++i)
                ok = mcclx::launch_stream_probe(st, buf + (size_t)((i + 4) % kCopies) * kBig, nbytes, false) == hipSuccess;
            ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
            float ms = 0.f;
            ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
            if (ok && ms * 1e3 / kReps < best) best = ms * 1e3 / kReps;
        }
        return best;
    };
    const double t_small = timed(kSmall), t_mid = timed(kMid), t_big = timed(kBig);
    cleanup();
    if (!ok || !(t_mid > t_small) || !(t_big > t_mid)) return m;
    const double probe_rate = (double)(kBig - kSmall) / ((t_big - t_small) * 100.0);  // bytes per 10 ns
    const double rate = probe_rate * kHoldGateRatio;
    // A device busy with someone else's work while this ran, or a tool that stretches launches and
    // event times (a profiler: 111,000 B per tick was once "measured" under one), gives nonsense:
    // the two halves of the size range must agree on the rate within 15 % (undisturbed, the lower half
    // reads 5-8 % faster than the upper; under a profiler the shortest launch takes twice its time and
    // the halves differ by a factor of two to four), and the rate must be one a part of this family
    // can have; otherwise the built-in constants stay.
    const double lower = (double)(kMid - kSmall) / (t_mid - t_small), upper = (double)(kBig - kMid) / (t_big - t_mid);
    if (const char* v = getenv("MCCLX_HOLD_CALIBRATE"))
        if (v[0] == '2')  // say what was measured
            fprintf(stderr, "[mcclx] gate calibration: %.2f / %.2f / %.2f us for 24 / 60 / 96 MiB read; %.0f B per 10 ns "
                            "(lower half %.0f, upper half %.0f)\n", t_small, t_mid, t_big, probe_rate, lower / 100.0, upper / 100.0);
    if (lower > 1.15 * upper || upper > 1.15 * lower) return m;
    if (rate < 0.6 * m.bytes_per_tick || rate > 1.4 * m.bytes_per_tick) return m;
    m.bytes_per_tick = (uint32_t)rate;
    m.measured = true;
    return m;
}

HoldModel device_hold_model(int device) {  // `device` is current
    static std::mutex mu;
    static std::map<int, HoldModel> cache;
    std::lock_guard<std::mutex> lk(mu);
    auto it = cache.find(device);
    if (it != cache.end()) return it->second;
    const HoldModel m = measure_hold_model();
    cache[device] = m;
    return m;
}

int make_ctx(int device, hipStream_t borrowed, bool borrow, mcclx_ctx** out) {
    if (!out) return fail(MCCLX_ERR_INVALID, "out is null");
    *out = nullptr;
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (device < 0 || device >= n)
        return fail(MCCLX_ERR_INVALID, "device %d out of range (%d visible)", device, n);
    DeviceGuard guard(device);
    if (!guard.ok) return fail(MCCLX_ERR_HIP, "hipSetDevice(%d) failed", device);
    auto* ctx = new mcclx_ctx();
    ctx->device = device;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) {
        delete ctx;
        return fail(MCCLX_ERR_HIP, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    }
    ctx->cus = prop.multiProcessorCount;
    // the gate of the hold form is counted in ticks of the device's wall clock: the model's
    // constants are in ticks of 100 MHz (what gfx950 runs it at) and scaled if the device differs
    int wall_khz = 0;
    if (hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || wall_khz <= 0) {
        (void)hipGetLastError();
        wall_khz = 100000;
    }
    ctx->wall_khz = (uint32_t)wall_khz;
    // Grid cap of the table launches.  Default: effectively none -- one block per
    // tile measured fastest (blocks are dispatched in address order; a capped,
    // grid-striding launch loses 5-20 %).  MCCLX_BLOCKS_PER_CU forces a
    // persistent-style cap there; by-value launches always run one block per tile.
    ctx->max_blocks = 1u << 22;
    if (const char* v = getenv("MCCLX_BLOCKS_PER_CU")) {
        int x = atoi(v);
        if (x >= 1 && x <= 16384) ctx->max_blocks = (uint32_t)ctx->cus * (uint32_t)x;
    }
    if (const char* v = getenv("MCCLX_FEW_SEGS")) {  // tuning: 0 sends every launch through the table kernel
        int x = atoi(v);
        if (x >= 0 && x <= mcclx::kFewSegs) ctx->few_max = (uint32_t)x;
    }
    if (const char* v = getenv("MCCLX_VALIDATE")) ctx->validate = (v[0] == '1');
    {
        const HoldModel hm = device_hold_model(device);
        ctx->hold_latency_ticks = hm.latency_ticks;
        ctx->hold_bytes_per_tick = hm.bytes_per_tick;
        ctx->hold_measured = hm.measured;
    }
    // MCCLX_HOLD=0 switches the reads-then-writes launches off; the other three are tuning knobs
    if (const char* v = getenv("MCCLX_HOLD")) ctx->hold_enabled.store(v[0] != '0');
    if (const char* v = getenv("MCCLX_HOLD_MIN_BYTES")) {
        const unsigned long long x = strtoull(v, nullptr, 10);
        ctx->hold_min_read_bytes = x ? x : 1;
    }
    if (const char* v = getenv("MCCLX_HOLD_LATENCY_TICKS")) ctx->hold_latency_ticks = (uint32_t)strtoul(v, nullptr, 10);
    if (const char* v = getenv("MCCLX_HOLD_BYTES_PER_TICK")) {
        const unsigned long x = strtoul(v, nullptr, 10);
        if (x >= 1000 && x <= 1000000) {
            ctx->hold_bytes_per_tick = (uint32_t)x;
            ctx->hold_measured = false;
        }
    }
    e = mcclx::static_table_resolve(device, &ctx->static_table);  // `device` is current (guard above)
    if (e != hipSuccess) {
        delete ctx;
        return fail(MCCLX_ERR_HIP, "hipGetSymbolAddress(static table) failed: %s", hipGetErrorString(e));
    }
    if (borrow) {
        ctx->stream = borrowed;
    } else {
        e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);  // default priority
        if (e != hipSuccess) {
            delete ctx;
            return fail(MCCLX_ERR_HIP, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
        }
        ctx->own_stream = true;
    }
    *out = ctx;
    return MCCLX_OK;
}

// Host-side guard of a GPU's static descriptor table: held for the duration of one
// allocation-free call.
constexpr int kMaxGuardedDevices = 64;
std::atomic<bool> g_static_table_busy[kMaxGuardedDevices];
struct StaticTableUse {
    int dev;
    bool mine;
    explicit StaticTableUse(int device) : dev(device), mine(true) {
        if (dev >= 0 && dev < kMaxGuardedDevices) mine = !g_static_table_busy[dev].exchange(true, std::memory_order_acquire);
    }
    ~StaticTableUse() {
        if (mine && dev >= 0 && dev < kMaxGuardedDevices) g_static_table_busy[dev].store(false, std::memory_order_release);
    }
};

int get_event(mcclx_ctx* ctx, hipEvent_t* ev) {
    if (!ctx->free_events.empty()) {
        *ev = ctx->free_events.back();
        ctx->free_events.pop_back();
        return MCCLX_OK;
    }
    HIP_TRY(hipEventCreateWithFlags(ev, hipEventDisableTiming));
    return MCCLX_OK;
}

}  // namespace

extern "C" {

const char* mcclx_last_error(void) { return g_err.c_str(); }
int mcclx_abi_version(void) { return MCCLX_ABI_VERSION; }

int mcclx_init(int device, mcclx_ctx** out) { return make_ctx(device, nullptr, false, out); }

int mcclx_init_on_stream(int device, void* hip_stream, mcclx_ctx** out) {
    return make_ctx(device, static_cast<hipStream_t>(hip_stream), true, out);
}

int mcclx_destroy(mcclx_ctx* ctx) {
    if (!ctx) return MCCLX_OK;
    DeviceGuard guard(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto& kv : ctx->tickets) (void)hipEventDestroy(kv.second.ev);
    for (auto ev : ctx->free_events) (void)hipEventDestroy(ev);
    for (auto ev : ctx->xev)
        if (ev) (void)hipEventDestroy(ev);
    for (auto& sl : ctx->slots) {
        if (sl.host) (void)hipHostFree(sl.host);
        if (sl.dev) (void)hipFree(sl.dev);
        if (sl.done) (void)hipEventDestroy(sl.done);
    }
    for (auto& kv : ctx->host_allocs) (void)hipHostFree(kv.first);
    if (ctx->stage_send) (void)hipHostFree(ctx->stage_send);
    for (int i = 0; i < 2; ++i) {
        if (ctx->stage_recv[i]) (void)hipHostFree(ctx->stage_recv[i]);
        if (ctx->stage_recv_done[i]) (void)hipEventDestroy(ctx->stage_recv_done[i]);
    }
    if (ctx->upload_stream) (void)hipStreamDestroy(ctx->upload_stream);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return MCCLX_OK;
}

void* mcclx_queue_stream(mcclx_ctx* ctx) { return ctx ? (void*)ctx->stream : nullptr; }
int mcclx_device_cus(mcclx_ctx* ctx) { return ctx ? ctx->cus : 0; }
uint64_t mcclx_launch_count(mcclx_ctx* ctx) { return ctx ? ctx->launches.load() : 0; }
uint64_t mcclx_hold_launch_count(mcclx_ctx* ctx) { return ctx ? ctx->hold_launches.load() : 0; }
int mcclx_hold_model(mcclx_ctx* ctx, uint32_t* latency_ticks, uint32_t* bytes_per_tick) {
    if (!ctx) return 0;
    if (latency_ticks) *latency_ticks = ctx->hold_latency_ticks;
    if (bytes_per_tick) *bytes_per_tick = ctx->hold_bytes_per_tick;
    return ctx->hold_measured ? 1 : 0;
}
int mcclx_set_hold(mcclx_ctx* ctx, int enabled) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    ctx->hold_enabled.store(enabled != 0, std::memory_order_relaxed);
    return MCCLX_OK;
}

int mcclx_fold(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* seg) {
    return fold_impl(ctx, plan, seg, 1);
}

int mcclx_fold_batched(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* segs, uint32_t nseg) {
    return fold_impl(ctx, plan, segs, nseg);
}

int mcclx_fold_batched_noalloc(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* segs, uint32_t nseg) {
    static_assert(sizeof(mcclx_seg) % 8 == 0, "descriptors are uploaded as 8-byte words");
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (nseg > MCCLX_NOALLOC_MAX_SEGS)
        return fail(MCCLX_ERR_INVALID, "fold_batched_noalloc: %u segments, the static table holds at most %d",
                    nseg, MCCLX_NOALLOC_MAX_SEGS);
    mcclx::PlanKey key;
    float scale_f;
    int has_scale, fan;
    if (int rc = check_plan(plan, &key, &scale_f, &has_scale, &fan)) return rc;
    if (int rc = check_segs(ctx, key, segs, nseg, fan)) return rc;
    if (nseg == 0) return MCCLX_OK;
    DeviceGuard guard(ctx->device);
    if (!guard.ok) return fail(MCCLX_ERR_HIP, "hipSetDevice(%d) failed", ctx->device);
    if (nseg <= (uint32_t)mcclx::kFewSegs && even_enough(key, segs, nseg))
        return launch_by_value(ctx, key, scale_f, has_scale, segs, nseg, fan);

    // One table per GPU, shared by every context on it: a second call that enters while this
    // one is still writing its descriptors would mix the two tables.  (Calls on one context
    // are ordered by its queue; launches of different contexts that are both already queued
    // and overlap on the device still race -- the host cannot see that.)
    StaticTableUse use(ctx->device);
    if (!use.mine)
        return fail(MCCLX_ERR_STATE,
                    "fold_batched_noalloc: another call is filling GPU %d's static descriptor table", ctx->device);

    uint64_t total = 0, uniform = mcclx::items_for(key, segs[0].count);
    for (uint32_t s = 0; s < nseg; ++s) {
        const uint64_t n = mcclx::items_for(key, segs[s].count);
        if (n != uniform) uniform = 0;
        total += n;
    }
    if (total == 0) return MCCLX_OK;
    if (total >> 31) return fail(MCCLX_ERR_INVALID, "fold: more than 2^31 work items in one launch");

    // Table layout, in 8-byte words: nseg descriptors, then nseg+1 work-item prefix
    // sums.  It is produced a writer launch's worth at a time, on the stack.
    std::lock_guard<std::mutex> lk(ctx->mu);
    constexpr uint32_t kSegWords = sizeof(mcclx_seg) / 8;
    const uint32_t seg_words = nseg * kSegWords, words = seg_words + nseg + 1;
    uint64_t* const table = static_cast<uint64_t*>(ctx->static_table);
    uint64_t running = 0;  // work items of the segments before `next_prefix`
    uint32_t next_prefix = 0;
    for (uint32_t off = 0; off < words; off += mcclx::kUploadWords) {
        uint64_t buf[mcclx::kUploadWords];
        const uint32_t n = words - off < mcclx::kUploadWords ? words - off : mcclx::kUploadWords;
        for (uint32_t i = 0; i < n; ++i) {
            const uint32_t g = off + i;
            if (g < seg_words) {
                memcpy(&buf[i], reinterpret_cast<const char*>(segs) + (size_t)g * 8, 8);
            } else {
                buf[i] = running;
                if (next_prefix < nseg) running += mcclx::items_for(key, segs[next_prefix].count);
                ++next_prefix;
            }
        }
        hipError_t e = mcclx::launch_table_write(ctx->stream, table + off, buf, n);
        if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "table write launch failed: %s", hipGetErrorString(e));
        ++ctx->launches;
    }
    mcclx::TableArgs t;
    t.segs = reinterpret_cast<const mcclx::SegArgs*>(table);
    t.first_item = table + seg_words;
    t.item_map = nullptr;  // ragged segments: a block finds its segment by bisection over first_item
    t.total_items = total;
    t.uniform_items = uniform;
    t.nseg = nseg;
    t.scale = scale_f;
    t.has_scale = has_scale;
    mcclx::LaunchParams lp;
    lp.max_blocks = ctx->max_blocks;
    lp.table = &t;
    lp.fan = fan;
    hipError_t e = mcclx::launch_fold(ctx->stream, key, lp);
    if (e != hipSuccess) return launch_error(e, key);
    ++ctx->launches;
    return MCCLX_OK;
}

int mcclx_reduce(mcclx_ctx* ctx, void* dst, const void* src, int dtype, uint64_t count, int op) {
    mcclx_plan p = {dtype, MCCLX_IO_PURE, 2, MCCLX_TOPO_FOLD, op, MCCLX_ACC_STEP, MCCLX_SCALE_NONE, 0, 0.0};
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = dst;
    s.in[0] = dst;
    s.in[1] = src;
    s.count = count;
    return fold_impl(ctx, &p, &s, 1);
}

int mcclx_scale(mcclx_ctx* ctx, void* buf, int dtype, uint64_t count, double scale, int scale_mode) {
    if (scale_mode != MCCLX_SCALE_VIEW && scale_mode != MCCLX_SCALE_TENSOR)
        return fail(MCCLX_ERR_INVALID, "scale_mode %d is not VIEW or TENSOR", scale_mode);
    mcclx_plan p = {dtype, MCCLX_IO_PURE, 1, MCCLX_TOPO_FOLD, MCCLX_SUM, MCCLX_ACC_STEP, scale_mode, 0, scale};
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = buf;
    s.in[0] = buf;
    s.count = count;
    return fold_impl(ctx, &p, &s, 1);
}

int mcclx_accumulate_scale(mcclx_ctx* ctx, void* dst, const void* src, int dtype, uint64_t count,
                           double scale) {
    mcclx_plan p = {dtype, MCCLX_IO_PURE, 2, MCCLX_TOPO_FOLD, MCCLX_SUM, MCCLX_ACC_STEP,
                    MCCLX_SCALE_TENSOR, 0, scale};
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = dst;
    s.in[0] = dst;
    s.in[1] = src;
    s.count = count;
    return fold_impl(ctx, &p, &s, 1);
}

int mcclx_encode_bf16(mcclx_ctx* ctx, void* dst_bf16, const void* src_f32, uint64_t count) {
    mcclx_plan p = {MCCLX_BF16, MCCLX_IO_OWN_FIRST_F32, 1, MCCLX_TOPO_FOLD, MCCLX_SUM, MCCLX_ACC_STEP,
                    MCCLX_SCALE_NONE, 0, 0.0};
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.wire_out = dst_bf16;
    s.in[0] = src_f32;
    s.count = count;
    return fold_impl(ctx, &p, &s, 1);
}

int mcclx_decode_bf16(mcclx_ctx* ctx, void* dst_f32, const void* src_bf16, uint64_t count) {
    mcclx_plan p = {MCCLX_BF16, MCCLX_IO_OUT_F32, 1, MCCLX_TOPO_FOLD, MCCLX_SUM, MCCLX_ACC_STEP,
                    MCCLX_SCALE_NONE, 0, 0.0};
    mcclx_seg s;
    memset(&s, 0, sizeof s);
    s.out = dst_f32;
    s.in[0] = src_bf16;
    s.count = count;
    return fold_impl(ctx, &p, &s, 1);
}

int mcclx_copy(mcclx_ctx* ctx, void* dst, const void* src, uint64_t nbytes) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (nbytes == 0 || dst == src) return MCCLX_OK;
    if (!dst || !src) return fail(MCCLX_ERR_INVALID, "copy: null pointer");
    if (ctx->validate) {
        if (int rc = check_range(src, nbytes, "src", 0)) return rc;
        if (int rc = check_range(dst, nbytes, "dst", 0)) return rc;
    }
    DeviceGuard guard(ctx->device);
    hipError_t e = mcclx::launch_copy(ctx->stream, dst, src, nbytes, ctx->max_blocks);
    if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "copy launch failed: %s", hipGetErrorString(e));
    ++ctx->launches;
    return MCCLX_OK;
}

int mcclx_copy_batched(mcclx_ctx* ctx, const mcclx_copy_desc* descs, uint32_t n) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (n == 0) return MCCLX_OK;
    if (!descs) return fail(MCCLX_ERR_INVALID, "copy_batched: descriptor array is null");
    uintptr_t both = 0;
    uint64_t bytes = 0;
    uint32_t live = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const mcclx_copy_desc& d = descs[i];
        if (d.nbytes == 0 || d.dst == d.src) continue;
        if (!d.dst || !d.src) return fail(MCCLX_ERR_INVALID, "copy_batched: descriptor %u has a null pointer", i);
        if (ctx->validate) {
            if (int rc = check_range(d.src, d.nbytes, "src", i)) return rc;
            if (int rc = check_range(d.dst, d.nbytes, "dst", i)) return rc;
        }
        both |= reinterpret_cast<uintptr_t>(d.dst) | reinterpret_cast<uintptr_t>(d.src);
        bytes += d.nbytes;
        ++live;
    }
    if (live == 0) return MCCLX_OK;
    DeviceGuard guard(ctx->device);
    if (!guard.ok) return fail(MCCLX_ERR_HIP, "hipSetDevice(%d) failed", ctx->device);
    const int align = (both % 4 == 0) ? 4 : (both % 2 == 0) ? 2 : 1;
    // Few or large copies: descriptors in the kernel arguments, up to 32 copies per
    // grid (a block of the table kernel first has to fetch its descriptor from
    // memory, which costs large copies 5-10 %); the grid is as wide as the longest
    // copy of a group, so groups are cut where lengths differ wildly.  Many small
    // ones: one table launch.
    if (live <= (uint32_t)mcclx::kFewCopies || bytes / live >= (1u << 20)) {
        mcclx::CopyFew few;
        few.n = 0;
        uint64_t longest = 0, sum = 0;
        auto flush = [&]() -> int {
            if (few.n == 0) return MCCLX_OK;
            hipError_t e = mcclx::launch_copy_few(ctx->stream, few, align);
            if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "copy_batched launch failed: %s", hipGetErrorString(e));
            ++ctx->launches;
            few.n = 0;
            longest = sum = 0;
            return MCCLX_OK;
        };
        for (uint32_t i = 0; i < n; ++i) {
            const mcclx_copy_desc& d = descs[i];
            if (d.nbytes == 0 || d.dst == d.src) continue;
            const uint64_t lg = d.nbytes > longest ? d.nbytes : longest;
            // blocks with nothing to do: more than 3 in 4 -> start a new group
            if (few.n == (uint32_t)mcclx::kFewCopies || (few.n && lg * (few.n + 1) > 4 * (sum + d.nbytes) + (1u << 16)))
                if (int rc = flush()) return rc;
            few.d[few.n++] = mcclx::CopyDesc{d.dst, d.src, d.nbytes};
            longest = d.nbytes > longest ? d.nbytes : longest;
            sum += d.nbytes;
        }
        return flush();
    }
    std::lock_guard<std::mutex> lk(ctx->mu);
    const size_t desc_bytes = (size_t)live * sizeof(mcclx::CopyDesc);
    std::vector<char> host(desc_bytes + ((size_t)live + 1) * sizeof(uint64_t));
    auto* hd = reinterpret_cast<mcclx::CopyDesc*>(host.data());
    auto* pre = reinterpret_cast<uint64_t*>(host.data() + desc_bytes);
    uint64_t total = 0, uniform = 0;
    uint32_t j = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const mcclx_copy_desc& d = descs[i];
        if (d.nbytes == 0 || d.dst == d.src) continue;
        hd[j] = mcclx::CopyDesc{d.dst, d.src, d.nbytes};
        pre[j] = total;
        const uint64_t items = mcclx::copy_items(d.nbytes);
        if (j == 0) uniform = items;
        if (items != uniform) uniform = 0;
        total += items;
        ++j;
    }
    pre[live] = total;
    if (total >> 31) return fail(MCCLX_ERR_INVALID, "copy_batched: more than 2^31 work items in one launch");
    const bool mapped = uniform == 0 && total <= kMaxMappedItems;
    const size_t map_off = host.size();
    if (mapped) {
        host.resize(map_off + (size_t)total * sizeof(uint2));
        pre = reinterpret_cast<uint64_t*>(host.data() + desc_bytes);
        uint2* map = reinterpret_cast<uint2*>(host.data() + map_off);
        for (uint32_t c = 0; c < live; ++c)
            for (uint64_t w = pre[c]; w < pre[c + 1]; ++w) map[w] = make_uint2(c, (uint32_t)(w - pre[c]));
    }
    void* dev = nullptr;
    TableSlot* slot = nullptr;
    if (int rc = stage_table(ctx, host.data(), host.size(), &dev, &slot)) return rc;
    mcclx::CopyTable t;
    t.descs = static_cast<const mcclx::CopyDesc*>(dev);
    t.first_item = reinterpret_cast<const uint64_t*>(static_cast<char*>(dev) + desc_bytes);
    t.item_map = mapped ? reinterpret_cast<const uint2*>(static_cast<char*>(dev) + map_off) : nullptr;
    t.total_items = (uint32_t)total;
    t.uniform_items = (uint32_t)uniform;
    t.n = live;
    hipError_t e = mcclx::launch_copy_many(ctx->stream, t, align, ctx->max_blocks);
    if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "copy_batched launch failed: %s", hipGetErrorString(e));
    ++ctx->launches;
    return MCCLX_OK;
}

int mcclx_batch_begin(mcclx_ctx* ctx, const char* label) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (ctx->batch_active) return fail(MCCLX_ERR_STATE, "batch already active");  // MetalKernels.mm:562
    ctx->batch_active = true;
    ctx->batch_label = label ? label : "mccl_batch";
    return MCCLX_OK;
}

int mcclx_batch_end(mcclx_ctx* ctx) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    ctx->batch_active = false;  // no-op when none is open (MetalKernels.mm:571)
    return MCCLX_OK;
}

#define REFUSE_WHILE_RECORDING(ctx, what)                                                     \
    if ((ctx)->capturing)                                                                    \
    return fail(MCCLX_ERR_STATE, what " is not allowed between graph_begin and graph_end")

int mcclx_queue_drain(mcclx_ctx* ctx) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    REFUSE_WHILE_RECORDING(ctx, "queue_drain");
    DeviceGuard guard(ctx->device);
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return MCCLX_OK;
}

static int stream_wait(mcclx_ctx* ctx, hipStream_t waiter, hipStream_t producer) {
    if (waiter == producer) return MCCLX_OK;
    REFUSE_WHILE_RECORDING(ctx, "cross-stream ordering");
    DeviceGuard guard(ctx->device);
    // A producer that has nothing in flight needs no event: everything enqueued on it so far is
    // complete, which is all the wait would establish (an event record plus a stream wait cost
    // the host 10-20 us on torch's legacy stream, a query a fraction of that).
    const hipError_t idle = hipStreamQuery(producer);
    if (idle == hipSuccess) return MCCLX_OK;
    (void)hipGetLastError();  // hipErrorNotReady, or a state the record below reports properly
    std::lock_guard<std::mutex> lk(ctx->mu);
    hipEvent_t& ev = ctx->xev[ctx->xnext];
    ctx->xnext = (ctx->xnext + 1) % 16;
    if (!ev) HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    HIP_TRY(hipEventRecord(ev, producer));
    HIP_TRY(hipStreamWaitEvent(waiter, ev, 0));
    return MCCLX_OK;
}

int mcclx_queue_wait_stream(mcclx_ctx* ctx, void* producer_stream) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    return stream_wait(ctx, ctx->stream, static_cast<hipStream_t>(producer_stream));
}

int mcclx_stream_wait_queue(mcclx_ctx* ctx, void* consumer_stream) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    return stream_wait(ctx, static_cast<hipStream_t>(consumer_stream), ctx->stream);
}

int mcclx_event_record(mcclx_ctx* ctx, uint64_t* ticket) {
    if (!ctx || !ticket) return fail(MCCLX_ERR_INVALID, "event_record: null argument");
    REFUSE_WHILE_RECORDING(ctx, "event_record");
    DeviceGuard guard(ctx->device);
    std::lock_guard<std::mutex> lk(ctx->mu);
    hipEvent_t ev;
    if (int rc = get_event(ctx, &ev)) return rc;
    HIP_TRY(hipEventRecord(ev, ctx->stream));
    *ticket = ctx->next_ticket++;
    ctx->tickets[*ticket].ev = ev;
    return MCCLX_OK;
}

int mcclx_event_query(mcclx_ctx* ctx, uint64_t ticket, int* done) {
    if (!ctx || !done) return fail(MCCLX_ERR_INVALID, "event_query: null argument");
    std::lock_guard<std::mutex> lk(ctx->mu);
    auto it = ctx->tickets.find(ticket);
    if (it == ctx->tickets.end()) {
        // already waited for (or never issued): tickets below the counter are complete
        if (ticket == 0 || ticket >= ctx->next_ticket) return fail(MCCLX_ERR_INVALID, "unknown ticket");
        *done = 1;
        return MCCLX_OK;
    }
    hipError_t e = hipEventQuery(it->second.ev);
    if (e == hipSuccess) {
        *done = 1;
    } else if (e == hipErrorNotReady) {
        (void)hipGetLastError();
        *done = 0;
    } else {
        return fail(MCCLX_ERR_HIP, "hipEventQuery failed: %s", hipGetErrorString(e));
    }
    return MCCLX_OK;
}

int mcclx_event_wait(mcclx_ctx* ctx, uint64_t ticket) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (ticket == 0) return MCCLX_OK;  // "fell back to blocking sync", MPSInterop.mm:352-355
    hipEvent_t ev;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        auto it = ctx->tickets.find(ticket);
        if (it == ctx->tickets.end()) {
            if (ticket >= ctx->next_ticket) return fail(MCCLX_ERR_INVALID, "unknown ticket");
            return MCCLX_OK;  // waited for before: complete
        }
        ev = it->second.ev;
        ++it->second.waiters;  // the ticket stays known (and pollable) until the wait is over
    }
    hipError_t e = hipEventSynchronize(ev);
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        auto it = ctx->tickets.find(ticket);
        if (it != ctx->tickets.end() && --it->second.waiters == 0) {
            ctx->free_events.push_back(ev);  // the last waiter retires the ticket
            ctx->tickets.erase(it);
        }
    }
    if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "hipEventSynchronize failed: %s", hipGetErrorString(e));
    return MCCLX_OK;
}

int mcclx_graph_begin(mcclx_ctx* ctx) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (ctx->capturing) return fail(MCCLX_ERR_STATE, "graph recording already active");
    DeviceGuard guard(ctx->device);
    // relaxed mode: the blocking table uploads above stay legal while recording
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    ctx->capturing = true;
    return MCCLX_OK;
}

int mcclx_graph_end(mcclx_ctx* ctx, mcclx_graph** out) {
    if (!ctx || !out) return fail(MCCLX_ERR_INVALID, "graph_end: null argument");
    if (!ctx->capturing) return fail(MCCLX_ERR_STATE, "graph_end without graph_begin");
    DeviceGuard guard(ctx->device);
    ctx->capturing = false;
    auto* g = new mcclx_graph();
    g->tables.swap(ctx->capture_tables);
    hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    // stage the launch's kernel arguments on the device now rather than during the first replay
    if (e == hipSuccess) e = hipGraphUpload(g->exec, ctx->stream);
    if (e != hipSuccess) {
        if (g->exec) (void)hipGraphExecDestroy(g->exec);
        if (g->graph) (void)hipGraphDestroy(g->graph);
        for (void* t : g->tables) (void)hipFree(t);
        delete g;
        return fail(MCCLX_ERR_HIP, "graph_end failed: %s", hipGetErrorString(e));
    }
    *out = g;
    return MCCLX_OK;
}

int mcclx_graph_launch(mcclx_ctx* ctx, mcclx_graph* graph) {
    if (!ctx || !graph) return fail(MCCLX_ERR_INVALID, "graph_launch: null argument");
    REFUSE_WHILE_RECORDING(ctx, "graph_launch");
    DeviceGuard guard(ctx->device);
    HIP_TRY(hipGraphLaunch(graph->exec, ctx->stream));
    return MCCLX_OK;
}

int mcclx_graph_destroy(mcclx_ctx* ctx, mcclx_graph* graph) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (!graph) return MCCLX_OK;
    DeviceGuard guard(ctx->device);
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    for (void* t : graph->tables) (void)hipFree(t);
    delete graph;
    return MCCLX_OK;
}

int mcclx_host_alloc(mcclx_ctx* ctx, uint64_t nbytes, void** host_ptr, void** device_ptr) {
    if (!ctx || !host_ptr || !device_ptr) return fail(MCCLX_ERR_INVALID, "host_alloc: null argument");
    if (nbytes == 0) return fail(MCCLX_ERR_INVALID, "host_alloc: zero bytes");
    DeviceGuard guard(ctx->device);
    void* h = nullptr;
    hipError_t e = hipHostMalloc(&h, nbytes, hipHostMallocMapped | hipHostMallocPortable);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(MCCLX_ERR_NOMEM, "hipHostMalloc(%llu) failed: %s", (unsigned long long)nbytes,
                    hipGetErrorString(e));
    }
    void* d = nullptr;
    e = hipHostGetDevicePointer(&d, h, 0);
    if (e != hipSuccess) {
        (void)hipHostFree(h);
        return fail(MCCLX_ERR_HIP, "hipHostGetDevicePointer failed: %s", hipGetErrorString(e));
    }
    std::lock_guard<std::mutex> lk(ctx->mu);
    ctx->host_allocs[h] = nbytes;
    *host_ptr = h;
    *device_ptr = d;
    return MCCLX_OK;
}

namespace {
constexpr size_t kRecvChunk = 8u << 20;  // pinned chunk of the pipelined receive path

// Host-addressable?  (pinned allocations of this library or of anyone else; on
// ROCm a pinned allocation has one address for host and device)
bool host_visible(const void* p, void** host_alias) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (attr.type != hipMemoryTypeHost) return false;
    *host_alias = const_cast<void*>(p);
    return true;
}
}  // namespace

int mcclx_stage_for_send(mcclx_ctx* ctx, const void* device_src, uint64_t nbytes, void** host_ptr) {
    if (!ctx || !host_ptr) return fail(MCCLX_ERR_INVALID, "stage_for_send: null argument");
    if (!device_src || nbytes == 0) return fail(MCCLX_ERR_INVALID, "stage_for_send: empty source");
    REFUSE_WHILE_RECORDING(ctx, "stage_for_send");
    DeviceGuard guard(ctx->device);
    void* alias = nullptr;
    if (host_visible(device_src, &alias)) {  // direct path: no copy
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        *host_ptr = alias;
        return MCCLX_OK;
    }
    std::lock_guard<std::mutex> lk(ctx->mu);
    if (ctx->stage_send_cap < nbytes) {
        if (ctx->stage_send) HIP_TRY(hipHostFree(ctx->stage_send));
        ctx->stage_send = nullptr;
        ctx->stage_send_cap = 0;
        size_t cap = 1u << 20;
        while (cap < nbytes) cap <<= 1;
        hipError_t e = hipHostMalloc(&ctx->stage_send, cap, hipHostMallocDefault);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(MCCLX_ERR_NOMEM, "staging buffer of %zu bytes: %s", cap, hipGetErrorString(e));
        }
        ctx->stage_send_cap = cap;
    }
    HIP_TRY(hipMemcpyAsync(ctx->stage_send, device_src, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    *host_ptr = ctx->stage_send;
    return MCCLX_OK;
}

int mcclx_unstage_from_recv(mcclx_ctx* ctx, void* device_dst, const void* host_src, uint64_t nbytes) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (nbytes == 0) return MCCLX_OK;
    if (!device_dst || !host_src) return fail(MCCLX_ERR_INVALID, "unstage_from_recv: null pointer");
    REFUSE_WHILE_RECORDING(ctx, "unstage_from_recv");
    DeviceGuard guard(ctx->device);
    void* alias = nullptr;
    if (host_visible(host_src, &alias)) {  // pinned source: one asynchronous copy
        HIP_TRY(hipMemcpyAsync(device_dst, alias, nbytes, hipMemcpyHostToDevice, ctx->stream));
        return MCCLX_OK;
    }
    // pageable source: memcpy into one pinned chunk while the other is in flight
    std::lock_guard<std::mutex> lk(ctx->mu);
    for (int i = 0; i < 2; ++i) {
        if (!ctx->stage_recv[i]) {
            hipError_t e = hipHostMalloc(&ctx->stage_recv[i], kRecvChunk, hipHostMallocDefault);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fail(MCCLX_ERR_NOMEM, "staging chunk: %s", hipGetErrorString(e));
            }
            HIP_TRY(hipEventCreateWithFlags(&ctx->stage_recv_done[i], hipEventDisableTiming));
        }
    }
    const char* src = static_cast<const char*>(host_src);
    char* dst = static_cast<char*>(device_dst);
    int slot = 0;
    for (uint64_t off = 0; off < nbytes; off += kRecvChunk, slot ^= 1) {
        size_t n = (size_t)((nbytes - off) < kRecvChunk ? (nbytes - off) : kRecvChunk);
        if (ctx->stage_recv_pending[slot]) {
            HIP_TRY(hipEventSynchronize(ctx->stage_recv_done[slot]));
            ctx->stage_recv_pending[slot] = false;
        }
        memcpy(ctx->stage_recv[slot], src + off, n);
        HIP_TRY(hipMemcpyAsync(dst + off, ctx->stage_recv[slot], n, hipMemcpyHostToDevice, ctx->stream));
        HIP_TRY(hipEventRecord(ctx->stage_recv_done[slot], ctx->stream));
        ctx->stage_recv_pending[slot] = true;
    }
    return MCCLX_OK;
}

int mcclx_host_free(mcclx_ctx* ctx, void* host_ptr) {
    if (!ctx) return fail(MCCLX_ERR_STATE, "context is null (mcclx_init not called)");
    if (!host_ptr) return MCCLX_OK;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        auto it = ctx->host_allocs.find(host_ptr);
        if (it == ctx->host_allocs.end())
            return fail(MCCLX_ERR_INVALID, "host_free: %p was not returned by mcclx_host_alloc", host_ptr);
        ctx->host_allocs.erase(it);
    }
    DeviceGuard guard(ctx->device);
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipHostFree(host_ptr));
    return MCCLX_OK;
}

#if MCCLX_TUNE_TIMELINE
// Measurement build only (include/mcclx_bench.h): one launch that only reads or only
// writes `nbytes` of `buf` on `hip_stream`, with the copy kernel's access shape.
MCCLX_API int mcclx_bench_probe(void* hip_stream, void* buf, uint64_t nbytes, int write) {
    if (nbytes == 0) return MCCLX_OK;
    if (!buf || (uintptr_t)buf % 4) return fail(MCCLX_ERR_INVALID, "bench_probe: buffer is null or not 4-byte aligned");
    hipError_t e = mcclx::launch_stream_probe(static_cast<hipStream_t>(hip_stream), buf, nbytes, write != 0);
    if (e != hipSuccess) return fail(MCCLX_ERR_HIP, "probe launch failed: %s", hipGetErrorString(e));
    return MCCLX_OK;
}
#endif

}  // extern "C"
