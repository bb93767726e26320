#include "backend/HostWire.hpp"

#ifndef MCCL_NULL_DEVICE
#include <hip/hip_runtime_api.h>
#endif

#include <algorithm>
#include <chrono>
#include <cstring>

#include "backend/Device.hpp"
#include "backend/Errors.hpp"
#include "backend/Logging.hpp"

namespace mccl {

// Device-time bracket around the fold launch, for the statistics.
#ifndef MCCL_NULL_DEVICE
struct FoldTimer {
    hipEvent_t t0 = nullptr, t1 = nullptr;
    ~FoldTimer() {
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
    }
    void begin(void* stream) {
        if (!t0)
            MCCL_CHECK(hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess,
                       "host wire: hipEventCreate failed");
        MCCL_CHECK(hipEventRecord(t0, static_cast<hipStream_t>(stream)) == hipSuccess, "host wire: hipEventRecord failed");
    }
    double end_ms(void* stream) {
        float ms = 0.f;
        MCCL_CHECK(hipEventRecord(t1, static_cast<hipStream_t>(stream)) == hipSuccess &&
                       hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&ms, t0, t1) == hipSuccess,
                   "host wire: timing the fold failed");
        return ms;
    }
};
#else
struct FoldTimer {
    void begin(void*) {}
    double end_ms(void*) { return 0.0; }
};
#endif

struct HostWire::Ctx {
    mcclx_ctx* ctx = nullptr;
    FoldTimer timer;
    ~Ctx() {
        if (ctx) mcclx_destroy(ctx);
    }
};

struct HostWire::Pinned {
    std::shared_ptr<Ctx> owner;  // host_free needs the context
    void* host = nullptr;
    void* dev = nullptr;
    uint64_t nbytes = 0;
    ~Pinned() {
        if (host && owner && owner->ctx) (void)mcclx_host_free(owner->ctx, host);
    }
};

namespace {

uint64_t esize(int dtype) { return dtype == MCCLX_F32 ? 4 : 2; }

// One chunk of the tensor, who ends up owning its reduction, and the order in
// which the ranks' operands enter the fold (the schedule's own order).
struct Piece {
    uint64_t start = 0, count = 0;
    int owner = 0;
    std::vector<int> order;
};

std::vector<Piece> pieces_of(int algo, int world, uint64_t numel) {
    std::vector<Piece> out;
    if (algo == MCCLX_ALGO_TREE) {  // allreduce_tree: everything reduces into rank 0 (AllreduceAlgos.cpp:100-114)
        Piece p;
        p.count = numel;
        for (int q = 0; q < world; ++q) p.order.push_back(q);
        out.push_back(std::move(p));
        return out;
    }
    std::vector<mcclx_chunk> c(static_cast<size_t>(world));
    check_rc(mcclx_chunkize(static_cast<int64_t>(numel), 1, world, c.data()));
    const bool ring = algo == MCCLX_ALGO_RING;
    for (int ch = 0; ch < world; ++ch) {
        if (c[static_cast<size_t>(ch)].elem_count == 0) continue;
        Piece p;
        p.start = static_cast<uint64_t>(c[static_cast<size_t>(ch)].elem_start);
        p.count = static_cast<uint64_t>(c[static_cast<size_t>(ch)].elem_count);
        if (ring) {  // chunk ch travels ch, ch+1, ... and ends at rank ch-1 (AllreduceAlgos.cpp:62-75)
            p.owner = (ch - 1 + world) % world;
            for (int j = 0; j < world; ++j) p.order.push_back((ch + j) % world);
        } else {     // butterfly: owner ch, then the peers in ascending order (:151-180)
            p.owner = ch;
            p.order.push_back(ch);
            for (int q = 0; q < world; ++q)
                if (q != ch) p.order.push_back(q);
        }
        out.push_back(std::move(p));
    }
    return out;
}

char* at(void* base, uint64_t off) { return static_cast<char*>(base) + off; }

}  // namespace

HostWire::HostWire(std::shared_ptr<LocalMesh> mesh, int rank, int device, std::chrono::milliseconds timeout)
    : peer_(mesh, rank, timeout), rank_(rank), world_(mesh->world()), device_(device), ctx_(std::make_shared<Ctx>()) {
    check_rc(mcclx_init(device, &ctx_->ctx));
}

HostWire::~HostWire() {
    // messages still in flight keep their buffers (and through them the context) alive
    send_pin_[0].reset();
    send_pin_[1].reset();
    recv_a_pin_.reset();
    recv_b_pin_.reset();
}

std::shared_ptr<HostWire::Pinned> HostWire::pinned(std::shared_ptr<Pinned>& slot, uint64_t nbytes) {
    if (!slot || slot->nbytes < nbytes) {
        auto p = std::make_shared<Pinned>();
        p->owner = ctx_;
        uint64_t cap = 1u << 20;
        while (cap < nbytes) cap <<= 1;
        check_rc(mcclx_host_alloc(ctx_->ctx, cap, &p->host, &p->dev));
        p->nbytes = cap;
        slot = std::move(p);
    }
    return slot;
}

void* HostWire::device_scratch(at::Tensor& slot, uint64_t nbytes) {
    if (!slot.defined() || static_cast<uint64_t>(slot.numel()) < nbytes + 256) {
        check_rc(mcclx_queue_drain(ctx_->ctx));
        slot = dev::empty_bytes(static_cast<int64_t>(nbytes + 256), device_);
        check_rc(mcclx_queue_wait_stream(ctx_->ctx, dev::current_stream(device_)));
    }
    auto p = reinterpret_cast<uintptr_t>(slot.data_ptr());
    return reinterpret_cast<void*>((p + 255) / 256 * 256);
}

void HostWire::allreduce(void* tensor, int dtype, uint64_t numel, int op, int algo, bool wire_bf16, Mode mode,
                         void* torch_stream) {
    MCCL_CHECK(world_ <= MCCLX_MAX_INPUTS,
               "the host-wire allreduce folds one chunk in one pass: at most " + std::to_string(MCCLX_MAX_INPUTS) + " ranks");
    mcclx_ctx* ctx = ctx_->ctx;
    const int N = world_, me = rank_;
    const bool codec = wire_bf16 && dtype == MCCLX_F32;             // ProcessGroupMCCL.cpp:131
    const int W = codec ? MCCLX_BF16 : dtype;                       // dtype on the wire
    const uint64_t es = esize(W), ts = esize(dtype);
    const bool sum_like = op == MCCLX_SUM || op == MCCLX_AVG;
    const bool all_on_wire = codec && !sum_like;  // the fold mixes fp32 and bf16 operands for sums only
    const bool staged = mode == Mode::Staged;
    const std::vector<Piece> pieces = pieces_of(algo, N, numel);
    const Piece* mine = nullptr;
    uint64_t max_count = 0;
    for (const Piece& p : pieces) {
        if (p.owner == me) mine = &p;
        max_count = std::max(max_count, p.count);
    }
    stats_ = Stats{stats_.calls + 1, 0, 0, 0, 0.0, 0, {0, 0, 0, 0, 0}};
    auto leg_t0 = std::chrono::steady_clock::now();
    auto leg_done = [&](int leg) {
        const auto now = std::chrono::steady_clock::now();
        stats_.leg_ms[leg] = std::chrono::duration<double, std::milli>(now - leg_t0).count();
        leg_t0 = now;
    };

    // buffers: what this rank sends (wire form, laid out like the tensor), what it
    // receives for its own chunk (one slot per peer), what it receives in the allgather leg
    const uint64_t send_bytes = numel * es, recv_a_bytes = static_cast<uint64_t>(N - 1) * max_count * es;
    void *send_dev, *recv_a_dev, *recv_b_dev;
    char *send_host = nullptr, *recv_a_host = nullptr, *recv_b_host = nullptr;
    std::shared_ptr<Pinned> send_keep;
    if (staged) {
        send_dev = device_scratch(send_dev_, send_bytes);
        recv_a_dev = device_scratch(recv_a_dev_, recv_a_bytes);
        recv_b_dev = device_scratch(recv_b_dev_, send_bytes);
        if (pageable_.size() < max_count * es) pageable_.resize(max_count * es);
    } else {
        send_keep = pinned(send_pin_[stats_.calls & 1], send_bytes);
        auto a = pinned(recv_a_pin_, recv_a_bytes);
        auto b = pinned(recv_b_pin_, send_bytes);
        send_dev = send_keep->dev;
        recv_a_dev = a->dev;
        recv_b_dev = b->dev;
        send_host = static_cast<char*>(send_keep->host);
        recv_a_host = static_cast<char*>(a->host);
        recv_b_host = static_cast<char*>(b->host);
    }
    auto slot_of = [&](int q) { return q < me ? q : q - 1; };  // peers in ascending order, this rank skipped

    check_rc(mcclx_queue_wait_stream(ctx, torch_stream));  // mps_stream_sync, ProcessGroupMCCL.cpp:172

    // ---- 1. the wire form of what this rank sends: every chunk it does not own
    {
        mcclx_plan enc;
        std::memset(&enc, 0, sizeof enc);
        enc.dtype = MCCLX_BF16;
        enc.io = MCCLX_IO_OWN_FIRST_F32;
        enc.k = 1;
        enc.op = MCCLX_SUM;
        std::vector<mcclx_seg> segs;
        for (const Piece& p : pieces) {
            if (p.owner == me && !all_on_wire) continue;
            if (codec) {
                mcclx_seg s;
                std::memset(&s, 0, sizeof s);
                s.wire_out = at(send_dev, p.start * 2);
                s.in[0] = at(tensor, p.start * 4);
                s.count = p.count;
                segs.push_back(s);
            } else {
                check_rc(mcclx_copy(ctx, at(send_dev, p.start * es), at(tensor, p.start * ts), p.count * es));
            }
        }
        if (!segs.empty()) check_rc(mcclx_fold_batched(ctx, &enc, segs.data(), static_cast<uint32_t>(segs.size())));
        check_rc(mcclx_queue_drain(ctx));  // the bytes are in host memory (Pinned) before the wire reads them
    }
    leg_done(0);

    // ---- 2. reduce-scatter leg of the wire: my operand of every other chunk goes to its owner ...
    auto send_piece = [&](int to, const Piece& p) {
        const uint64_t len = p.count * es;
        if (staged) {
            void* h = nullptr;  // valid until the next staging call: the transport copies it
            check_rc(mcclx_stage_for_send(ctx, at(send_dev, p.start * es), len, &h));
            peer_.send(to, h, len);
        } else {
            peer_.send_kept(to, send_host + p.start * es, len, send_keep);
        }
        stats_.wire_bytes_sent += len;
    };
    auto recv_into = [&](int from, void* dev_dst, char* host_dst, uint64_t len) {
        if (staged) {
            peer_.recv(from, pageable_.data(), len);
            check_rc(mcclx_unstage_from_recv(ctx, dev_dst, pageable_.data(), len));
            check_rc(mcclx_queue_drain(ctx));  // `pageable_` is reused for the next message
        } else {
            peer_.recv(from, host_dst, len);
        }
    };
    for (const Piece& p : pieces)
        if (p.owner != me) send_piece(p.owner, p);
    // ... and the peers' operands of my chunk arrive, one slot per peer
    if (mine)
        for (int q = 0; q < N; ++q) {
            if (q == me) continue;
            const uint64_t off = static_cast<uint64_t>(slot_of(q)) * mine->count * es;
            recv_into(q, at(recv_a_dev, off), recv_a_host ? recv_a_host + off : nullptr, mine->count * es);
        }

    leg_done(1);
    // ---- 3. one fold of all operands of my chunk, in the schedule's order
    if (mine) {
        mcclx_plan plan;
        std::memset(&plan, 0, sizeof plan);
        plan.dtype = W;
        plan.k = N;
        plan.topo = algo == MCCLX_ALGO_TREE ? MCCLX_TOPO_BINOMIAL : MCCLX_TOPO_FOLD;
        plan.op = op;
        plan.acc = MCCLX_ACC_STEP;
        plan.scale_mode = op == MCCLX_AVG ? MCCLX_SCALE_VIEW : MCCLX_SCALE_NONE;  // AllreduceAlgos.cpp:88-91
        plan.scale = 1.0 / static_cast<double>(N);
        plan.flags = algo == MCCLX_ALGO_RING ? MCCLX_PLAN_ACC_IS_SRC : 0;      // :72-74
        plan.io = MCCLX_IO_PURE;
        if (codec && !all_on_wire) plan.io = algo == MCCLX_ALGO_RING ? MCCLX_IO_OWN_LAST_F32 : MCCLX_IO_OWN_FIRST_F32;
        mcclx_seg s;
        std::memset(&s, 0, sizeof s);
        s.count = mine->count;
        for (int j = 0; j < N; ++j) {
            const int q = mine->order[static_cast<size_t>(j)];
            if (q == me)
                s.in[j] = all_on_wire ? at(send_dev, mine->start * 2) : at(tensor, mine->start * ts);
            else
                s.in[j] = at(recv_a_dev, static_cast<uint64_t>(slot_of(q)) * mine->count * es);
        }
        if (all_on_wire) {
            s.out = at(send_dev, mine->start * 2);  // in place over the owner's wire copy; cast back below
        } else {
            s.out = at(tensor, mine->start * ts);
            if (codec) s.wire_out = at(send_dev, mine->start * 2);  // the reduced chunk as it travels on
        }
        ctx_->timer.begin(mcclx_queue_stream(ctx));
        check_rc(mcclx_fold_batched(ctx, &plan, &s, 1));
        stats_.fold_ms = ctx_->timer.end_ms(mcclx_queue_stream(ctx));
        stats_.fold_elems = mine->count;
        stats_.fold_peer_bytes = static_cast<uint64_t>(N - 1) * mine->count * es;
        stats_.fold_hbm_bytes = mine->count * ((all_on_wire ? 0 : 2 * ts));
        if (!codec)  // no codec: the reduced chunk travels in the tensor's own dtype
            check_rc(mcclx_copy(ctx, at(send_dev, mine->start * es), at(tensor, mine->start * ts), mine->count * es));
        check_rc(mcclx_queue_drain(ctx));  // every reduce complete before the next send reads it
    }

    leg_done(2);
    // ---- 4. allgather leg: my reduced chunk goes to every peer, theirs arrive and are cast on arrival
    if (mine) {
        if (staged) {  // staged once, handed to every peer (the transport copies it)
            void* h = nullptr;
            const uint64_t len = mine->count * es;
            check_rc(mcclx_stage_for_send(ctx, at(send_dev, mine->start * es), len, &h));
            for (int q = 0; q < N; ++q)
                if (q != me) {
                    peer_.send(q, h, len);
                    stats_.wire_bytes_sent += len;
                }
        } else {
            for (int q = 0; q < N; ++q)
                if (q != me) send_piece(q, *mine);
        }
    }
    mcclx_plan dec;
    std::memset(&dec, 0, sizeof dec);
    dec.dtype = MCCLX_BF16;
    dec.io = MCCLX_IO_OUT_F32;
    dec.k = 1;
    dec.op = MCCLX_SUM;
    std::vector<mcclx_seg> dsegs;
    for (const Piece& p : pieces) {
        const void* src;
        if (p.owner == me) {
            if (!all_on_wire) continue;  // the fold already wrote this rank's tensor
            src = at(send_dev, p.start * 2);
        } else {
            recv_into(p.owner, at(recv_b_dev, p.start * es), recv_b_host ? recv_b_host + p.start * es : nullptr,
                      p.count * es);
            src = at(recv_b_dev, p.start * es);
        }
        if (codec) {  // ProcessGroupMCCL.cpp:179-183
            mcclx_seg s;
            std::memset(&s, 0, sizeof s);
            s.out = at(tensor, p.start * 4);
            s.in[0] = src;
            s.count = p.count;
            dsegs.push_back(s);
        } else {
            check_rc(mcclx_copy(ctx, at(tensor, p.start * ts), src, p.count * es));
        }
    }
    leg_done(3);
    if (!dsegs.empty()) check_rc(mcclx_fold_batched(ctx, &dec, dsegs.data(), static_cast<uint32_t>(dsegs.size())));
    check_rc(mcclx_queue_drain(ctx));  // mccl_queue_drain, ProcessGroupMCCL.cpp:178
    leg_done(4);
}

}  // namespace mccl
