// LocalMesh.hpp -- the in-process stand-in for the reference's PeerMesh
// (csrc/backend/PeerMesh.hpp:12-31).
//
// The reference moves peer chunks over blocking TCP sockets between processes.
// This build runs every rank of a group inside ONE process on ONE GPU (there is
// no cross-GPU transport here), so "send/recv" degenerates to: every rank
// publishes where its tensors live, waits until all ranks of the group have
// reached the same collective, and the last rank to arrive launches the device
// work for the whole group -- peers' chunks are read in place.  Collectives
// must be issued in the same order on every rank, exactly as with the
// reference's FIFO engine (Progress.hpp:12-18).
#pragma once

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
    int async = 0;                 // allreduce: event-based completion asked for (ranks must agree)
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

class LocalMesh {
public:
    using Leader = std::function<void(const std::vector<Contribution>&)>;

    explicit LocalMesh(int world)
        : world_(world), slots_(static_cast<size_t>(world)),
          boxes_(static_cast<size_t>(world) * static_cast<size_t>(world)) {}

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
    // TimeoutError and poisons the mesh (later calls fail at once).
    void rendezvous(int rank, Contribution c, std::chrono::milliseconds timeout, const Leader& leader);

    // Point-to-point: one FIFO per ordered pair of ranks, as a socket per peer
    // gives the reference.  post never blocks (the sender has already copied the
    // payload into a buffer the parcel owns); take blocks until a parcel from
    // `src` is there or `timeout` passes (TimeoutError; the mesh stays usable).
    void post(int src, int dst, Parcel p);
    Parcel take(int src, int dst, std::chrono::milliseconds timeout);

private:
    const int world_;
    std::mutex mu_;
    std::condition_variable cv_;
    std::vector<Contribution> slots_;
    int arrived_ = 0;
    uint64_t generation_ = 0;
    std::exception_ptr last_error_;
    bool broken_ = false;

    std::mutex box_mu_;
    std::condition_variable box_cv_;
    std::vector<std::deque<Parcel>> boxes_;   // [src * world + dst]
};

}  // namespace mccl
