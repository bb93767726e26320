// LocalMesh.hpp -- the in-process stand-in for the reference's PeerMesh
// (csrc/backend/PeerMesh.hpp:12-31).
//
// The reference moves peer chunks over blocking TCP sockets between processes.
// This build runs every rank of a group inside ONE process on ONE GPU (there is
// no cross-GPU transport here), and offers the ranks two ways to meet:
//
//  * rendezvous: every rank publishes where its tensors live, waits until all
//    ranks of the group have reached the same collective, and the last rank to
//    arrive launches the device work for the whole group -- peers' chunks are
//    read in place (the default path of every collective);
//  * a byte transport with PeerMesh's own interface, send(peer, buf, len) /
//    recv(peer, buf, len) on host-addressable memory (LocalPeer below): one
//    FIFO per ordered pair of ranks, as a socket per peer gives the reference.
//    The allreduce's host-wire modes (MCCL_WIRE=host|staged) run over it.
//
// Collectives must be issued in the same order on every rank, exactly as with
// the reference's FIFO engine (Progress.hpp:12-18).
#pragma once

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace mccl {

// Event-based completion: how far one rank's stream has already been put behind each of
// the mesh's reduce queues (the id of the newest launch an event it waits for covers).
struct WaitMarks {
    std::mutex mu;
    void* stream[2] = {nullptr, nullptr};
    bool valid[2] = {false, false};
    uint64_t upto[2] = {0, 0};
};

// What one rank contributes to a collective: raw device addresses plus the
// parameters all ranks must agree on.
struct Contribution {
    int kind = 0;                  // collective id; must match across ranks
    std::vector<void*> dst;        // output buffers (per tensor)
    std::vector<const void*> src;  // input buffers (per tensor, or world entries per tensor for list forms)
    std::vector<uint64_t> numel;   // per tensor
    std::vector<int> dtype;        // per tensor (MCCLX_F32/F16/BF16, or -1 for byte copies)
    std::vector<int> algo;         // per tensor (allreduce)
    std::vector<uint64_t> nbytes;  // per tensor (copies)
    int op = 0;
    int wire_bf16 = 0;
    int root = 0;
    void* stream = nullptr;        // the rank's producer/consumer HIP stream
    void* work = nullptr;          // the rank's completion object, when the leader (or a later
                                   // launch) settles it instead of the rank itself
    std::shared_ptr<WaitMarks> marks;  // the rank's record of what its stream already waits for
    int async = 0;                 // allreduce: event-based completion asked for (ranks must agree)
    int direct = 1;                // allreduce: read peers' fp32 tensors in place (rank 0's setting is used)
    int transport = 0;             // allreduce: 0 = peers read in place, 1 = pinned host wire, 2 = staged host wire
    std::vector<uint64_t> in_off;  // all-to-all: byte offsets (or sizes) of what goes to each peer
    std::vector<uint64_t> out_off; // all-to-all: byte offsets (or sizes) of what comes from each peer
    std::string error;             // set when this rank failed its own argument checks: the
                                   // rank still arrives, and every rank then fails with this
                                   // message instead of waiting for a peer that never comes
};

// One point-to-point message (the reference's 8-byte {tag, nbytes} header followed
// by the payload, ProcessGroupMCCL.cpp:624-628).  `keep` owns the device buffer
// `data` points into until the receiver has consumed it.
struct Parcel {
    int32_t tag = 0;
    uint64_t nbytes = 0;
    const void* data = nullptr;
    std::shared_ptr<void> keep;
};

// One message on the byte transport: `len` bytes at `data`, which either live in
// `owned` (the sender's bytes were copied, as a socket buffer would hold them) or
// stay valid for as long as `keep` is held (a sender that hands over a buffer it
// will not touch again until the exchange is over).
struct WireMessage {
    std::vector<uint8_t> owned;
    const void* data = nullptr;
    size_t len = 0;
    std::shared_ptr<void> keep;
};

class LocalMesh {
public:
    using Leader = std::function<void(const std::vector<Contribution>&)>;

    explicit LocalMesh(int world);

    // Process-wide registry: ranks of one group find their mesh by the key the
    // group's store hands out.
    static std::shared_ptr<LocalMesh> create(const std::string& key, int world);
    static std::shared_ptr<LocalMesh> find(const std::string& key);
    static void forget(const std::string& key);
    static std::string fresh_key();

    int world() const { return world_; }

    // Blocks until all ranks have contributed to this collective.  The last
    // arrival runs `leader` with every rank's contribution (index = rank);
    // all ranks return when it is done.  If `leader` throws, every rank
    // rethrows that error.  If peers do not arrive within `timeout`, throws
    // TimeoutError and poisons the mesh (later calls fail at once).  The device work
    // of a gradient bucket takes tens of microseconds, less than it takes to put a
    // thread to sleep and wake it: a waiter first polls for MCCL_MEET_SPIN_US
    // microseconds (default 200, 0 = sleep at once).
    void rendezvous(int rank, Contribution c, std::chrono::milliseconds timeout, const Leader& leader);

    // Point-to-point: one FIFO per ordered pair of ranks, as a socket per peer
    // gives the reference.  post never blocks (the sender has already copied the
    // payload into a buffer the parcel owns); take blocks until a parcel from
    // `src` is there or `timeout` passes (TimeoutError; the mesh stays usable).
    void post(int src, int dst, Parcel p);
    Parcel take(int src, int dst, std::chrono::milliseconds timeout);

    // Byte transport (PeerMesh::send / recv, PeerMesh.hpp:19-20).  wire_send never
    // blocks: the bytes are copied into the message unless `keep` is given, in which
    // case `buf` is handed over as it is.  wire_recv blocks until the next message
    // from `src` is there (TimeoutError after `timeout`), requires its length to be
    // `len` -- the reference's receivers always know how much is coming -- and copies
    // it into `buf`.
    void wire_send(int src, int dst, const void* buf, size_t len, std::shared_ptr<void> keep = nullptr);
    void wire_recv(int src, int dst, void* buf, size_t len, std::chrono::milliseconds timeout);

private:
    const int world_;
    std::mutex mu_;
    std::condition_variable cv_;
    std::vector<Contribution> slots_;
    static constexpr int kCountBits = 16;
    static constexpr uint64_t kCountMask = (1ull << kCountBits) - 1;
    std::atomic<uint64_t> state_{0};       // generation << 16 | ranks that have arrived for it; the last arrival moves
                                           // the generation on when its work is done, the others poll it
    std::exception_ptr last_error_;        // of the collective that just ended: written before the generation moves on
    std::atomic<bool> broken_{false};
    const int spin_us_;                    // how long a waiter polls before it sleeps (MCCL_MEET_SPIN_US)

    std::mutex box_mu_;
    std::condition_variable box_cv_;
    std::vector<std::deque<Parcel>> boxes_;   // [src * world + dst]

    std::mutex wire_mu_;
    std::condition_variable wire_cv_;
    std::vector<std::deque<WireMessage>> wires_;  // [src * world + dst]
};

// One rank's end of the byte transport, with the reference's PeerMesh interface
// (csrc/backend/PeerMesh.hpp:12-31): what the reference's algorithms hold as `mesh`.
class LocalPeer {
public:
    LocalPeer(std::shared_ptr<LocalMesh> mesh, int rank, std::chrono::milliseconds timeout)
        : mesh_(std::move(mesh)), rank_(rank), timeout_(timeout) {}

    void send(int peer, const void* buf, size_t len) { mesh_->wire_send(rank_, peer, buf, len); }
    void recv(int peer, void* buf, size_t len) { mesh_->wire_recv(peer, rank_, buf, len, timeout_); }
    // send without the copy: `keep` holds `buf` until the receiver has taken the bytes
    void send_kept(int peer, const void* buf, size_t len, std::shared_ptr<void> keep) {
        mesh_->wire_send(rank_, peer, buf, len, std::move(keep));
    }

    int world() const { return mesh_->world(); }
    int rank() const { return rank_; }

private:
    std::shared_ptr<LocalMesh> mesh_;
    int rank_;
    std::chrono::milliseconds timeout_;
};

}  // namespace mccl
