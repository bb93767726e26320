// mcclx_sched.cpp -- the chunk scheduler: chunkize, algorithm selection and the
// single-process replay of the ring / tree / butterfly allreduce schedules
// (csrc/backend/AllreduceAlgos.cpp) plus reduce_scatter / allgather
// (csrc/backend/ProcessGroupMCCL.cpp) for N virtual ranks on one GPU.
//
// Host C++ on top of the public C ABI only (mcclx_reduce, mcclx_fold_batched,
// mcclx_copy, ...): nothing here touches HIP directly.
//
// STEPWISE mode issues the reference's launches one for one -- every send/recv
// pair becomes a device copy into the receiver's scratch, followed by the
// binary in-place reduce the reference runs on that scratch.
// FUSED mode is the MI355X shape of the same schedule: for every chunk its
// final owner folds all N operands in ONE pass, reading the peers' chunks where
// they already lie (the position xGMI peer reads or a zero-copy host buffer
// would put them in), rounding after each operand exactly as the stepwise
// kernels would, so both modes give bit-identical tensors.

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "mcclx.h"
#include "mcclx_internal.h"

namespace {

constexpr uint64_t kAlign = 256;  // workspace sub-buffers start on 256 B

uint64_t align_up(uint64_t x) { return (x + kAlign - 1) / kAlign * kAlign; }
uint64_t esize(int dtype) { return dtype == MCCLX_F32 ? 4 : 2; }

struct Chunks {
    std::vector<mcclx_chunk> c;
    Chunks(int64_t numel, uint64_t es, int world) : c((size_t)world) {
        mcclx_chunkize(numel, es, world, c.data());
    }
    const mcclx_chunk& operator[](int i) const { return c[(size_t)i]; }
};

char* at(void* base, uint64_t off) { return static_cast<char*>(base) + off; }
const char* at(const void* base, uint64_t off) { return static_cast<const char*>(base) + off; }

#define TRY(x)                 \
    do {                       \
        int _rc = (x);         \
        if (_rc != MCCLX_OK) return _rc; \
    } while (0)

// recv scratch per rank, ProcessGroupMCCL.cpp:152-162
uint64_t scratch_elems(int algo, int world, uint64_t numel) {
    uint64_t per = (numel + (uint64_t)world - 1) / (uint64_t)world;
    if (algo == MCCLX_ALGO_RING) return per;
    if (algo == MCCLX_ALGO_BUTTERFLY) return (uint64_t)(world - 1) * per;
    return numel;
}

struct Layout {
    bool wire;
    int wdtype;
    uint64_t wire_stride;     // bytes between ranks' bf16 copies
    uint64_t scratch_off;     // start of the recv scratch area
    uint64_t scratch_stride;  // bytes between ranks' recv scratch
    uint64_t total;
};

int fan_of(const mcclx_replay* r);
bool direct_applies(const mcclx_replay* r);

Layout layout_of(const mcclx_replay* r) {
    Layout L;
    L.wire = r->wire_bf16 && r->dtype == MCCLX_F32;  // ProcessGroupMCCL.cpp:131
    L.wdtype = L.wire ? MCCLX_BF16 : r->dtype;
    // a DIRECT fold that also hands the result to every rank needs no bf16 copy at all
    const bool no_copies = direct_applies(r) && fan_of(r) > 0;
    L.wire_stride = (L.wire && !no_copies) ? align_up(r->numel * 2) : 0;
    L.scratch_off = L.wire_stride * (uint64_t)r->world;
    bool need_scratch = r->mode == MCCLX_REPLAY_STEPWISE || r->world > MCCLX_MAX_INPUTS;
    L.scratch_stride =
        need_scratch ? align_up(scratch_elems(r->algo, r->world, r->numel) * esize(L.wdtype)) : 0;
    L.total = L.scratch_off + L.scratch_stride * (uint64_t)r->world;
    return L;
}

int bad(const char* msg) { return mcclx_fail(MCCLX_ERR_INVALID, "%s", msg); }

// ---------------------------------------------------------------- STEPWISE

int ring_stepwise(mcclx_ctx* ctx, int N, std::vector<void*>& t, std::vector<void*>& recv, int dtype,
                  uint64_t numel, int op) {
    Chunks c((int64_t)numel, esize(dtype), N);
    for (int k = 0; k < N - 1; ++k) {  // AllreduceAlgos.cpp:62-75
        for (int r = 0; r < N; ++r) {  // the wire: prev's send lands in r's scratch
            int prev = (r - 1 + N) % N;
            int idx = (r - k - 1 + N) % N;  // == prev's send_idx
            TRY(mcclx_copy(ctx, recv[r], at(t[prev], c[idx].byte_off), c[idx].byte_len));
        }
        for (int r = 0; r < N; ++r) {
            int idx = (r - k - 1 + N) % N;
            TRY(mcclx_reduce(ctx, at(t[r], c[idx].byte_off), recv[r], dtype,
                             (uint64_t)c[idx].elem_count, op));
        }
    }
    for (int k = 0; k < N - 1; ++k)  // :77-86
        for (int r = 0; r < N; ++r) {
            int prev = (r - 1 + N) % N;
            int idx = (r - k + N) % N;
            TRY(mcclx_copy(ctx, at(t[r], c[idx].byte_off), at(t[prev], c[idx].byte_off),
                           c[idx].byte_len));
        }
    return MCCLX_OK;
}

int tree_stepwise(mcclx_ctx* ctx, int N, std::vector<void*>& t, std::vector<void*>& recv, int dtype,
                  uint64_t numel, int op) {
    uint64_t nbytes = numel * esize(dtype);
    std::vector<char> active((size_t)N, 1);
    for (int mask = 1; mask < N; mask <<= 1) {  // AllreduceAlgos.cpp:100-114
        for (int r = 0; r < N; ++r)
            if (active[r] && (r & mask)) {
                TRY(mcclx_copy(ctx, recv[r - mask], t[r], nbytes));
                active[r] = 0;
            }
        for (int r = 0; r < N; ++r)
            if (active[r] && !(r & mask) && r + mask < N)
                TRY(mcclx_reduce(ctx, t[r], recv[r], dtype, numel, op));
    }
    int top = 1;
    while (top * 2 < N) top <<= 1;
    for (int mask = top; mask >= 1; mask >>= 1) {  // :119-126
        int two = mask << 1;
        for (int r = 0; r < N; ++r)
            if ((r % two) == 0 && r + mask < N) TRY(mcclx_copy(ctx, t[r + mask], t[r], nbytes));
    }
    return MCCLX_OK;
}

int butterfly_stepwise(mcclx_ctx* ctx, int N, std::vector<void*>& t, std::vector<void*>& recv,
                       int dtype, uint64_t numel, int op) {
    Chunks c((int64_t)numel, esize(dtype), N);
    for (int r = 0; r < N; ++r) {  // AllreduceAlgos.cpp:151-169
        int slot = 0;
        for (int p = 0; p < N; ++p) {
            if (p == r) continue;
            TRY(mcclx_copy(ctx, at(recv[r], (uint64_t)slot * c[r].byte_len),
                           at(t[p], c[r].byte_off), c[r].byte_len));
            slot++;
        }
    }
    for (int r = 0; r < N; ++r)  // :172-180
        for (int slot = 0; slot < N - 1; ++slot)
            TRY(mcclx_reduce(ctx, at(t[r], c[r].byte_off), at(recv[r], (uint64_t)slot * c[r].byte_len),
                             dtype, (uint64_t)c[r].elem_count, op));
    for (int r = 0; r < N; ++r)  // :185-200
        for (int p = 0; p < N; ++p)
            if (p != r)
                TRY(mcclx_copy(ctx, at(t[p], c[r].byte_off), at(t[r], c[r].byte_off), c[r].byte_len));
    return MCCLX_OK;
}

int replay_stepwise(mcclx_ctx* ctx, const mcclx_replay* r, const Layout& L) {
    const int N = r->world;
    std::vector<void*> work((size_t)N), recv((size_t)N);
    for (int i = 0; i < N; ++i) {
        recv[i] = at(r->workspace, L.scratch_off + (uint64_t)i * L.scratch_stride);
        if (L.wire) {
            work[i] = at(r->workspace, (uint64_t)i * L.wire_stride);
            TRY(mcclx_encode_bf16(ctx, work[i], r->tensors[i], r->numel));  // PG.cpp:131-132
        } else {
            work[i] = r->tensors[i];
        }
    }
    if (r->algo == MCCLX_ALGO_RING)
        TRY(ring_stepwise(ctx, N, work, recv, L.wdtype, r->numel, r->op));
    else if (r->algo == MCCLX_ALGO_BUTTERFLY)
        TRY(butterfly_stepwise(ctx, N, work, recv, L.wdtype, r->numel, r->op));
    else
        TRY(tree_stepwise(ctx, N, work, recv, L.wdtype, r->numel, r->op));
    if (r->op == MCCLX_AVG)  // AllreduceAlgos.cpp:88-91,128-131,202-205
        for (int i = 0; i < N; ++i)
            TRY(mcclx_scale(ctx, work[i], L.wdtype, r->numel, 1.0 / (double)N, MCCLX_SCALE_VIEW));
    if (L.wire)
        for (int i = 0; i < N; ++i)  // PG.cpp:179-183
            TRY(mcclx_decode_bf16(ctx, r->tensors[i], work[i], r->numel));
    return MCCLX_OK;
}

// ------------------------------------------------------------------- FUSED

mcclx_plan base_plan(const mcclx_replay* r, const Layout& L, int k) {
    mcclx_plan p;
    memset(&p, 0, sizeof p);
    p.dtype = L.wdtype;
    p.io = MCCLX_IO_PURE;
    p.k = k;
    p.topo = MCCLX_TOPO_FOLD;
    p.op = r->op;
    p.acc = r->acc;
    p.scale_mode = (r->op == MCCLX_AVG) ? MCCLX_SCALE_VIEW : MCCLX_SCALE_NONE;
    p.scale = 1.0 / (double)r->world;
    // the ring reduces the travelling partial result into each receiver's own chunk:
    // dst = the next operand, src = the partial result (AllreduceAlgos.cpp:72-74)
    if (r->algo == MCCLX_ALGO_RING) p.flags = MCCLX_PLAN_ACC_IS_SRC;
    return p;
}

// The launches of one or more fused allreduces that share a plan, gathered phase
// by phase: what every rank encodes for the wire, the folds, the casts on
// arrival, and the plain copies of the allgather leg.  Each phase is one launch.
struct FoldPass {
    mcclx_plan plan;
    std::vector<mcclx_seg> segs;
};

struct Phases {
    bool planned = false;
    mcclx_plan enc, dec;
    std::vector<mcclx_seg> enc_segs, dec_segs;
    std::vector<FoldPass> folds;  // one pass, or a chain of passes when the world is wider than one fold
    std::vector<mcclx_copy_desc> copies;
    int fan = 0;  // > 0: the fold itself stores every reduced chunk into the other ranks' tensors
                  // (in[k .. k+fan-1] of its segments); there is no allgather launch then
};

// A sum over so few ranks that operands and destinations fit one segment (k ranks +
// k-1 other tensors <= MCCLX_MAX_INPUTS, i.e. up to 4 ranks): the owner's fold writes
// the result to everybody -- what the allgather leg and the final cast would
// deliver (AllreduceAlgos.cpp:77-86,116-131,185-200, ProcessGroupMCCL.cpp:179-183: the
// other ranks' cast of the bf16 result gives the very fp32 values the owner holds).
// MCCLX_FANOUT=0 keeps the separate allgather launch.
int fan_of(const mcclx_replay* r) {
    static const bool enabled = [] {
        const char* e = getenv("MCCLX_FANOUT");
        return !(e && e[0] == '0');
    }();
    const bool sum = r->op == MCCLX_SUM || r->op == MCCLX_AVG;
    const bool wire = r->wire_bf16 && r->dtype == MCCLX_F32;
    const bool step = r->acc == MCCLX_ACC_STEP || (r->dtype == MCCLX_F32 && !wire);  // fp32 has no rounding to skip
    if (!enabled || !sum || !step || r->world < 2 || 2 * r->world - 1 > MCCLX_MAX_INPUTS) return 0;
    return r->world - 1;
}

// MIN / MAX / PRODUCT over the wire codec: the fold kernels mix fp32 and bf16
// operands for sums only, so for these ops every rank encodes its WHOLE tensor
// (the owner's chunk too), the fold runs on bf16 operands alone, in place over
// the owner's wire copy, and every rank -- the owner included -- casts the
// result back.  Same arithmetic as the reference (cast, reduce in bf16, cast
// back: ProcessGroupMCCL.cpp:131-132, 179-183), in three launches.
// The same holds for a world wider than one fold (see chain_lengths).
bool all_on_wire(const mcclx_replay* r) {
    return (r->op != MCCLX_SUM && r->op != MCCLX_AVG) || r->world > MCCLX_MAX_INPUTS;
}

// DIRECT: a sum over the wire codec whose operands fit one fold reads every
// rank's fp32 tensor itself and encodes it in registers -- the bits of
// `t.to(at::kBFloat16)` (ProcessGroupMCCL.cpp:131-132) without the bf16 copy.
bool direct_applies(const mcclx_replay* r) {
    return r->mode == MCCLX_REPLAY_DIRECT && r->wire_bf16 && r->dtype == MCCLX_F32 && !all_on_wire(r);
}

// A fold takes MCCLX_MAX_INPUTS operands.  A wider world is folded by a chain
// of passes over same-dtype buffers: the first takes 8 operands, every later
// one the partial result plus up to 7 more, in the schedule's own order -- a
// left fold cut into pieces, so rounding happens exactly where the one-pass
// fold (and the reference's step-by-step loop) has it.  The scale goes with
// the last pass.
std::vector<int> chain_lengths(int world) {
    std::vector<int> ks;
    int left = world;
    ks.push_back(left < MCCLX_MAX_INPUTS ? left : MCCLX_MAX_INPUTS);
    left -= ks.back();
    while (left > 0) {
        int more = left < MCCLX_MAX_INPUTS - 1 ? left : MCCLX_MAX_INPUTS - 1;
        ks.push_back(more + 1);  // + the partial result
        left -= more;
    }
    return ks;
}

void plan_phases(const mcclx_replay* r, const Layout& L, Phases& ph) {
    if (ph.planned) return;
    ph.planned = true;
    if (r->algo == MCCLX_ALGO_TREE && r->world > MCCLX_MAX_INPUTS) {
        // The binomial tree of up to 64 ranks is a binomial tree of binomial trees:
        // masks 1, 2, 4 combine each block of 8 consecutive ranks into its first
        // rank, masks 8, 16, 32 combine the blocks' first ranks the same way
        // (AllreduceAlgos.cpp:100-114).  Pass 0 folds the full blocks, pass 1 the
        // last, shorter block, pass 2 the block results into rank 0 (and scales).
        const int blocks = (r->world + MCCLX_MAX_INPUTS - 1) / MCCLX_MAX_INPUTS;
        const int last = r->world - (blocks - 1) * MCCLX_MAX_INPUTS;
        ph.folds.resize(3);
        const int ks3[3] = {MCCLX_MAX_INPUTS, last, blocks};
        for (int p = 0; p < 3; ++p) {
            ph.folds[(size_t)p].plan = base_plan(r, L, ks3[p]);
            ph.folds[(size_t)p].plan.topo = MCCLX_TOPO_BINOMIAL;
            if (p < 2) ph.folds[(size_t)p].plan.scale_mode = MCCLX_SCALE_NONE;
        }
        ph.enc = base_plan(r, L, 1);
        ph.enc.io = MCCLX_IO_OWN_FIRST_F32;
        ph.enc.op = MCCLX_SUM;
        ph.enc.scale_mode = MCCLX_SCALE_NONE;
        ph.dec = ph.enc;
        ph.dec.io = MCCLX_IO_OUT_F32;
        return;
    }
    const std::vector<int> ks = chain_lengths(r->world);
    ph.folds.resize(ks.size());
    for (size_t p = 0; p < ks.size(); ++p) {
        mcclx_plan& f = ph.folds[p].plan;
        f = base_plan(r, L, ks[p]);
        if (p + 1 < ks.size()) f.scale_mode = MCCLX_SCALE_NONE;  // only the last pass scales
    }
    mcclx_plan& fold = ph.folds[0].plan;
    if (r->algo == MCCLX_ALGO_TREE) fold.topo = MCCLX_TOPO_BINOMIAL;
    ph.fan = fan_of(r);
    if (ph.fan) fold.flags |= MCCLX_PLAN_FANOUT(ph.fan);
    if (direct_applies(r)) {          // every operand is read as fp32 and encoded in registers
        fold.io = MCCLX_IO_ALL_F32;
    } else if (L.wire && !all_on_wire(r)) {  // the owner's operand is read as fp32 and encoded in registers
        if (r->algo == MCCLX_ALGO_TREE)
            fold.io = MCCLX_IO_OWN_FIRST_F32;
        else
            fold.io = r->algo == MCCLX_ALGO_RING ? MCCLX_IO_OWN_LAST_F32 : MCCLX_IO_OWN_FIRST_F32;
    }
    ph.enc = base_plan(r, L, 1);  // fp32 -> bf16 of what travels
    ph.enc.io = MCCLX_IO_OWN_FIRST_F32;
    ph.enc.op = MCCLX_SUM;
    ph.enc.flags = 0;
    ph.enc.scale_mode = MCCLX_SCALE_NONE;
    ph.dec = ph.enc;              // bf16 -> fp32 on arrival
    ph.dec.io = MCCLX_IO_OUT_F32;
}

void collect_fused(const mcclx_replay* r, const Layout& L, Phases& ph) {
    plan_phases(r, L, ph);
    const int N = r->world;
    const uint64_t es = esize(L.wdtype);  // element size on the "wire"
    const uint64_t ts = esize(r->dtype);  // element size of the rank tensors
    auto wire_of = [&](int rank) -> void* { return at(r->workspace, (uint64_t)rank * L.wire_stride); };
    mcclx_seg z;
    memset(&z, 0, sizeof z);

    const bool bf16_only = L.wire && all_on_wire(r);
    const bool direct = direct_applies(r);  // peers' fp32 tensors are the operands: nothing is encoded
    if (r->algo == MCCLX_ALGO_TREE) {
        // allreduce_tree: rank 0 ends with the binomial combination of all
        // tensors (AllreduceAlgos.cpp:100-114), everyone else receives a copy.
        if (L.wire && !direct)
            for (int q = bf16_only ? 0 : 1; q < N; ++q) {  // ranks 1.. encode: their tensors travel
                mcclx_seg s = z;
                s.wire_out = wire_of(q);
                s.in[0] = r->tensors[q];
                s.count = r->numel;
                ph.enc_segs.push_back(s);
            }
        if (N > MCCLX_MAX_INPUTS) {  // blocks of 8 ranks, then the blocks' first ranks (see plan_phases)
            auto buf = [&](int q) -> void* { return bf16_only ? wire_of(q) : r->tensors[q]; };
            const int blocks = (N + MCCLX_MAX_INPUTS - 1) / MCCLX_MAX_INPUTS;
            mcclx_seg top = z;
            top.count = r->numel;
            top.out = buf(0);
            for (int b = 0; b < blocks; ++b) {
                const int first = b * MCCLX_MAX_INPUTS;
                const int kb = (N - first < MCCLX_MAX_INPUTS) ? N - first : MCCLX_MAX_INPUTS;
                top.in[b] = buf(first);
                if (kb < 2) continue;  // a block of one rank is its own result
                mcclx_seg g = z;
                g.count = r->numel;
                g.out = buf(first);    // intermediate ranks' buffers hold partial sums, as in the reference
                for (int j = 0; j < kb; ++j) g.in[j] = buf(first + j);
                ph.folds[kb == MCCLX_MAX_INPUTS ? 0 : 1].segs.push_back(g);
            }
            ph.folds[2].segs.push_back(top);
            for (int q = bf16_only ? 0 : 1; q < N; ++q) {
                if (L.wire) {
                    mcclx_seg g = z;
                    g.out = r->tensors[q];
                    g.in[0] = wire_of(0);
                    g.count = r->numel;
                    ph.dec_segs.push_back(g);
                } else {
                    ph.copies.push_back(mcclx_copy_desc{r->tensors[q], r->tensors[0], r->numel * ts});
                }
            }
            return;
        }
        mcclx_seg s = z;
        s.count = r->numel;
        if (bf16_only) {
            s.out = wire_of(0);
            for (int q = 0; q < N; ++q) s.in[q] = wire_of(q);
        } else {
            s.out = r->tensors[0];
            s.in[0] = r->tensors[0];
            for (int q = 1; q < N; ++q) s.in[q] = (L.wire && !direct) ? wire_of(q) : r->tensors[q];
            if (ph.fan) {  // rank 0's fold hands the result to ranks 1..N-1 itself
                for (int q = 1; q < N; ++q) s.in[N + q - 1] = r->tensors[q];
            } else if (L.wire) {
                s.wire_out = wire_of(0);
            }
        }
        ph.folds[0].segs.push_back(s);
        if (ph.fan) return;
        for (int q = bf16_only ? 0 : 1; q < N; ++q) {
            if (L.wire) {  // broadcast of the bf16 result + the final cast on every rank
                mcclx_seg g = z;
                g.out = r->tensors[q];
                g.in[0] = wire_of(0);
                g.count = r->numel;
                ph.dec_segs.push_back(g);
            } else {
                ph.copies.push_back(mcclx_copy_desc{r->tensors[q], r->tensors[0], r->numel * ts});
            }
        }
        return;
    }

    // ring and butterfly: chunk c has one final owner who folds all N operands.
    //   butterfly (AllreduceAlgos.cpp:151-180): owner c; order own, then peers ascending.
    //   ring      (AllreduceAlgos.cpp:62-75)  : owner (c-1) mod N; order c, c+1, ..., owner.
    const bool ring = r->algo == MCCLX_ALGO_RING;
    Chunks c((int64_t)r->numel, 1, N);  // element offsets; bytes derived per buffer
    auto owner_of = [&](int chunk) { return ring ? (chunk - 1 + N) % N : chunk; };
    auto order_of = [&](int chunk, int j) {  // rank of the j-th operand
        if (ring) return (chunk + j) % N;
        if (j == 0) return chunk;
        return (j - 1 < chunk) ? j - 1 : j;  // ascending peers, skipping the owner
    };

    if (L.wire && !direct)  // every rank encodes what it sends: all chunks except the one it owns
        for (int q = 0; q < N; ++q)
            for (int ch = 0; ch < N; ++ch) {
                if ((owner_of(ch) == q && !bf16_only) || c[ch].elem_count == 0) continue;
                mcclx_seg s = z;
                s.wire_out = at(wire_of(q), (uint64_t)c[ch].elem_start * 2);
                s.in[0] = at(r->tensors[q], (uint64_t)c[ch].elem_start * 4);
                s.count = (uint64_t)c[ch].elem_count;
                ph.enc_segs.push_back(s);
            }

    for (int ch = 0; ch < N; ++ch) {
        if (c[ch].elem_count == 0) continue;
        int o = owner_of(ch);
        // operands in schedule order, and where the result goes
        std::vector<const void*> ops((size_t)N);
        for (int j = 0; j < N; ++j) {
            int q = order_of(ch, j);
            if (L.wire && !direct && (q != o || bf16_only))
                ops[(size_t)j] = at(wire_of(q), (uint64_t)c[ch].elem_start * es);
            else
                ops[(size_t)j] = at(r->tensors[q], (uint64_t)c[ch].elem_start * ts);
        }
        void* dest = bf16_only ? (void*)at(wire_of(o), (uint64_t)c[ch].elem_start * 2)
                               : (void*)at(r->tensors[o], (uint64_t)c[ch].elem_start * ts);
        if (ph.folds.size() == 1) {
            mcclx_seg s = z;
            s.count = (uint64_t)c[ch].elem_count;
            s.out = dest;
            for (int j = 0; j < N; ++j) s.in[j] = ops[(size_t)j];
            if (ph.fan) {  // the owner's fold hands the reduced chunk to every other rank itself
                int f = 0;
                for (int q = 0; q < N; ++q)
                    if (q != o) s.in[N + f++] = at(r->tensors[q], (uint64_t)c[ch].elem_start * ts);
            } else if (L.wire && !bf16_only) {
                s.wire_out = at(wire_of(o), (uint64_t)c[ch].elem_start * 2);
            }
            ph.folds[0].segs.push_back(s);
            continue;
        }
        // A chain.  Butterfly's first operand is the owner's own chunk, so the partial
        // result can live in `dest` from the first pass on; ring's owner comes last, so
        // the partial result waits in the owner's recv scratch until the last pass.
        void* partial = ring ? (void*)at(r->workspace, L.scratch_off + (uint64_t)o * L.scratch_stride) : dest;
        int next = 0;
        for (size_t p = 0; p < ph.folds.size(); ++p) {
            const int k = ph.folds[p].plan.k;
            mcclx_seg s = z;
            s.count = (uint64_t)c[ch].elem_count;
            int j = 0;
            if (p > 0) s.in[j++] = partial;
            while (j < k) s.in[j++] = ops[(size_t)next++];
            s.out = (p + 1 == ph.folds.size()) ? dest : partial;
            ph.folds[p].segs.push_back(s);
        }
    }

    // allgather leg (AllreduceAlgos.cpp:77-86,185-200): every other rank gets
    // the owner's reduced chunk; with the wire codec it arrives as bf16 and is
    // cast on arrival (ProcessGroupMCCL.cpp:179-183).
    if (ph.fan) return;  // done by the folds
    for (int ch = 0; ch < N; ++ch) {
        if (c[ch].elem_count == 0) continue;
        int o = owner_of(ch);
        for (int q = 0; q < N; ++q) {
            if (q == o && !bf16_only) continue;
            if (L.wire) {
                mcclx_seg s = z;
                s.out = at(r->tensors[q], (uint64_t)c[ch].elem_start * 4);
                s.in[0] = at(wire_of(o), (uint64_t)c[ch].elem_start * 2);
                s.count = (uint64_t)c[ch].elem_count;
                ph.dec_segs.push_back(s);
            } else {
                ph.copies.push_back(mcclx_copy_desc{at(r->tensors[q], (uint64_t)c[ch].elem_start * ts),
                                                    at(r->tensors[o], (uint64_t)c[ch].elem_start * ts),
                                                    (uint64_t)c[ch].elem_count * ts});
            }
        }
    }
}

int issue_phases(mcclx_ctx* ctx, Phases& ph) {
    if (!ph.enc_segs.empty())
        TRY(mcclx_fold_batched(ctx, &ph.enc, ph.enc_segs.data(), (uint32_t)ph.enc_segs.size()));
    for (FoldPass& f : ph.folds)
        if (!f.segs.empty()) TRY(mcclx_fold_batched(ctx, &f.plan, f.segs.data(), (uint32_t)f.segs.size()));
    if (!ph.dec_segs.empty())
        TRY(mcclx_fold_batched(ctx, &ph.dec, ph.dec_segs.data(), (uint32_t)ph.dec_segs.size()));
    if (!ph.copies.empty()) TRY(mcclx_copy_batched(ctx, ph.copies.data(), (uint32_t)ph.copies.size()));
    return MCCLX_OK;
}

// Argument checks of one replay; *fused says whether the fused schedule can run it.
int check_replay(mcclx_ctx* ctx, const mcclx_replay* r, bool* fused, bool* nothing_to_do) {
    *fused = false;
    *nothing_to_do = false;
    if (!ctx || !r || !r->tensors) return bad("replay: null argument");
    if (r->world < 1 || r->reserved != 0) return bad("replay: bad world");
    if (r->algo < MCCLX_ALGO_RING || r->algo > MCCLX_ALGO_BUTTERFLY) return bad("replay: bad algo");
    if (r->mode < MCCLX_REPLAY_STEPWISE || r->mode > MCCLX_REPLAY_DIRECT) return bad("replay: bad mode");
    if (r->op < MCCLX_SUM || r->op > MCCLX_MAX) {
        // surfaces "Unsupported ReduceOp: n" through the kernel layer
        return mcclx_reduce(ctx, r->tensors[0], r->tensors[0], r->dtype, 0, r->op);
    }
    if (r->world == 1) {  // ProcessGroupMCCL.cpp:107
        *nothing_to_do = true;
        return MCCLX_OK;
    }
    if (r->numel == 0) return bad("replay: empty tensor");  // TensorChecks.hpp:31-34
    // AllreduceAlgos.cpp:55,137
    if (r->algo != MCCLX_ALGO_TREE && r->numel < (uint64_t)r->world) return bad("numel must be >= world");
    for (int i = 0; i < r->world; ++i)
        if (!r->tensors[i]) return bad("replay: null tensor");
    Layout L = layout_of(r);
    if (L.total > 0 && (!r->workspace || r->workspace_bytes < L.total)) return bad("workspace too small");
    // the tree is fused as a tree of 8-rank trees: up to 8 x 8 ranks
    *fused = r->mode != MCCLX_REPLAY_STEPWISE &&
             (r->algo != MCCLX_ALGO_TREE || r->world <= MCCLX_MAX_INPUTS * MCCLX_MAX_INPUTS);
    return MCCLX_OK;
}

int run_stepwise(mcclx_ctx* ctx, const mcclx_replay* r) {
    mcclx_replay s = *r;
    s.mode = MCCLX_REPLAY_STEPWISE;
    Layout Ls = layout_of(&s);
    if (Ls.total > 0 && (!r->workspace || r->workspace_bytes < Ls.total)) return bad("workspace too small");
    return replay_stepwise(ctx, &s, Ls);
}

// Byte ranges one replay reads or writes: its rank tensors and its workspace.
struct Range {
    uintptr_t lo, hi;
};
void ranges_of(const mcclx_replay* r, std::vector<Range>& out) {
    const uint64_t tb = r->numel * esize(r->dtype);
    for (int i = 0; i < r->world; ++i) {
        const uintptr_t p = reinterpret_cast<uintptr_t>(r->tensors[i]);
        out.push_back(Range{p, p + tb});
    }
    if (r->workspace && r->workspace_bytes) {
        const uintptr_t p = reinterpret_cast<uintptr_t>(r->workspace);
        out.push_back(Range{p, p + r->workspace_bytes});
    }
}
bool overlaps(const std::vector<Range>& a, const std::vector<Range>& b) {
    for (const Range& x : a)
        for (const Range& y : b)
            if (x.lo < y.hi && y.lo < x.hi) return true;
    return false;
}

// Same plan for every phase?
bool same_plan(const mcclx_replay* a, const mcclx_replay* b) {
    return a->world == b->world && a->algo == b->algo && a->op == b->op && a->dtype == b->dtype &&
           (a->wire_bf16 != 0) == (b->wire_bf16 != 0) && a->acc == b->acc && a->mode == b->mode;
}

}  // namespace

extern "C" {

int mcclx_chunkize(int64_t numel, uint64_t elem_size, int world, mcclx_chunk* out) {
    if (world < 1 || numel < 0 || !out) return bad("chunkize: bad argument");
    const int64_t per = (numel + world - 1) / world;  // AllreduceAlgos.cpp:23
    for (int i = 0; i < world; ++i) {
        int64_t lo = (int64_t)i * per, hi = lo + per;
        lo = lo < numel ? lo : numel;
        hi = hi < numel ? hi : numel;
        out[i] = mcclx_chunk{lo, hi - lo, (uint64_t)lo * elem_size, (uint64_t)(hi - lo) * elem_size};
    }
    return MCCLX_OK;
}

int mcclx_select_algo(const char* env_algo, int64_t tree_below, uint64_t wire_nbytes,
                      int64_t numel, int world) {
    std::string alg = env_algo ? env_algo : "auto";  // ProcessGroupMCCL.cpp:134-135
    int algo = MCCLX_ALGO_TREE;                     // any unknown name runs the tree (:173-176)
    if (alg == "auto") {
        uint64_t below = tree_below < 0 ? 256ull * 1024 : (uint64_t)tree_below;  // :137-139
        algo = wire_nbytes <= below ? MCCLX_ALGO_TREE : MCCLX_ALGO_RING;        // :140
    } else if (alg == "ring") {
        algo = MCCLX_ALGO_RING;
    } else if (alg == "butterfly") {
        algo = MCCLX_ALGO_BUTTERFLY;
    }
    if (algo == MCCLX_ALGO_RING && numel < world) algo = MCCLX_ALGO_TREE;  // :143
    if (algo == MCCLX_ALGO_BUTTERFLY && (world < 2 || numel < world)) algo = MCCLX_ALGO_TREE;  // :144-145
    return algo;
}

uint64_t mcclx_replay_workspace_bytes(const mcclx_replay* r) {
    if (!r || r->world < 1) return 0;
    uint64_t need = layout_of(r).total;
    if (r->mode != MCCLX_REPLAY_STEPWISE && r->algo == MCCLX_ALGO_TREE &&
        r->world > MCCLX_MAX_INPUTS * MCCLX_MAX_INPUTS) {  // runs the stepwise schedule (check_replay)
        mcclx_replay s = *r;
        s.mode = MCCLX_REPLAY_STEPWISE;
        const uint64_t step = layout_of(&s).total;
        need = step > need ? step : need;
    }
    return need;
}

int mcclx_allreduce_replay(mcclx_ctx* ctx, const mcclx_replay* r) {
    return mcclx_allreduce_replay_many(ctx, r, 1);
}

int mcclx_allreduce_replay_many(mcclx_ctx* ctx, const mcclx_replay* rs, uint32_t n) {
    if (n && !rs) return bad("replay: null argument");
    uint32_t i = 0;
    while (i < n) {
        bool fused, nothing;
        TRY(check_replay(ctx, &rs[i], &fused, &nothing));
        if (nothing) {
            ++i;
            continue;
        }
        if (!fused) {
            TRY(run_stepwise(ctx, &rs[i]));
            ++i;
            continue;
        }
        // Gather the run of fused replays that share this one's plan.  The entries of a
        // run are issued phase by phase, not one after another, so a run also ends at an
        // entry that touches memory an earlier entry of the run touches (a tensor named
        // twice, overlapping workspaces): that entry starts a run of its own and sees the
        // earlier result, as in the reference's one-by-one loop (ProcessGroupMCCL.cpp:173-177).
        Phases ph;
        const mcclx_replay* first = &rs[i];
        std::vector<Range> taken, mine;
        while (i < n) {
            if (&rs[i] != first) {
                if (!same_plan(first, &rs[i])) break;
                TRY(check_replay(ctx, &rs[i], &fused, &nothing));
                if (!fused || nothing) break;
            }
            mine.clear();
            ranges_of(&rs[i], mine);
            if (overlaps(taken, mine)) break;
            taken.insert(taken.end(), mine.begin(), mine.end());
            collect_fused(&rs[i], layout_of(&rs[i]), ph);
            ++i;
        }
        TRY(issue_phases(ctx, ph));
    }
    return MCCLX_OK;
}

int mcclx_reduce_scatter_shares(mcclx_ctx* ctx, int world, void* const* outs,
                                const void* const* shares, int dtype, uint64_t chunk_numel, int op,
                                int mode, int acc) {
    if (!ctx || !outs || !shares || world < 1) return bad("reduce_scatter: bad argument");
    auto share = [&](int r, int p) { return shares[(size_t)r * (size_t)world + (size_t)p]; };
    const uint64_t cb = chunk_numel * esize(dtype);
    if (world == 1) return mcclx_copy(ctx, outs[0], share(0, 0), cb);  // ProcessGroupMCCL.cpp:333-337
    // MIN / MAX / PRODUCT and fp16 round after every step by definition
    bool step_only = (op != MCCLX_SUM && op != MCCLX_AVG) || dtype == MCCLX_F16;
    if (mode == MCCLX_REPLAY_STEPWISE) {
        for (int r = 0; r < world; ++r) {  // :357, :378-386
            TRY(mcclx_copy(ctx, outs[r], share(r, r), cb));
            for (int p = 0; p < world; ++p)
                if (p != r) TRY(mcclx_reduce(ctx, outs[r], share(r, p), dtype, chunk_numel, op));
            if (op == MCCLX_AVG)
                TRY(mcclx_scale(ctx, outs[r], dtype, chunk_numel, 1.0 / (double)world, MCCLX_SCALE_TENSOR));
        }
        return MCCLX_OK;
    }
    // One fold per rank; a world wider than one fold is cut into a chain of passes
    // (chain_lengths), the partial result waiting in the rank's output between them.
    // fp32 accumulation (ACC_F32) has a meaning inside one fold only: a chain rounds
    // where it is cut, so it runs with per-step rounding.
    const std::vector<int> ks = chain_lengths(world);
    mcclx_plan p;
    memset(&p, 0, sizeof p);
    p.dtype = dtype;
    p.io = MCCLX_IO_PURE;
    p.topo = MCCLX_TOPO_FOLD;
    p.op = op;
    p.acc = (step_only || ks.size() > 1) ? MCCLX_ACC_STEP : acc;
    p.scale = 1.0 / (double)world;
    std::vector<int> next((size_t)world, 0);  // per rank: operands consumed so far
    auto operand = [&](int r, int j) {        // own share first (:357), then ascending peers (:379-383)
        if (j == 0) return share(r, r);
        return share(r, (j - 1 < r) ? j - 1 : j);
    };
    for (size_t pass = 0; pass < ks.size(); ++pass) {
        p.k = ks[pass];
        const bool last = pass + 1 == ks.size();
        p.scale_mode = (last && op == MCCLX_AVG) ? MCCLX_SCALE_TENSOR : MCCLX_SCALE_NONE;  // metal_scale_inplace
        std::vector<mcclx_seg> segs((size_t)world);
        for (int r = 0; r < world; ++r) {
            mcclx_seg& g = segs[(size_t)r];
            memset(&g, 0, sizeof g);
            g.out = outs[r];
            g.count = chunk_numel;
            int j = 0;
            if (pass > 0) g.in[j++] = outs[r];
            while (j < p.k) g.in[j++] = operand(r, next[(size_t)r]++);
        }
        TRY(mcclx_fold_batched(ctx, &p, segs.data(), (uint32_t)segs.size()));
    }
    return MCCLX_OK;
}

int mcclx_reduce_scatter_replay(mcclx_ctx* ctx, int world, void* const* outs,
                                const void* const* ins, int dtype, uint64_t chunk_numel, int op,
                                int mode, int acc) {
    if (!ctx || !outs || !ins || world < 1) return bad("reduce_scatter: bad argument");
    const uint64_t cb = chunk_numel * esize(dtype);
    std::vector<const void*> shares((size_t)world * (size_t)world);
    for (int r = 0; r < world; ++r)
        for (int p = 0; p < world; ++p) shares[(size_t)r * world + p] = at(ins[p], (uint64_t)r * cb);
    return mcclx_reduce_scatter_shares(ctx, world, outs, shares.data(), dtype, chunk_numel, op, mode, acc);
}

int mcclx_allgather_replay(mcclx_ctx* ctx, int world, void* const* outs, const void* const* ins,
                           uint64_t chunk_nbytes) {
    if (!ctx || !outs || !ins || world < 1) return bad("allgather: bad argument");
    std::vector<mcclx_copy_desc> copies;
    copies.reserve((size_t)world * (size_t)world);
    for (int r = 0; r < world; ++r)
        for (int p = 0; p < world; ++p)  // ProcessGroupMCCL.cpp:256-270
            copies.push_back(mcclx_copy_desc{at(outs[r], (uint64_t)p * chunk_nbytes), ins[p], chunk_nbytes});
    // small chunks go out in one launch, large ones stream one launch each
    return mcclx_copy_batched(ctx, copies.data(), (uint32_t)copies.size());
}

}  // extern "C"
