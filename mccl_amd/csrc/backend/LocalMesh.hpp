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
};

class LocalMesh {
public:
    using Leader = std::function<void(const std::vector<Contribution>&)>;

    explicit LocalMesh(int world) : world_(world), slots_(static_cast<size_t>(world)) {}

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

private:
    const int world_;
    std::mutex mu_;
    std::condition_variable cv_;
    std::vector<Contribution> slots_;
    int arrived_ = 0;
    uint64_t generation_ = 0;
    std::exception_ptr last_error_;
    bool broken_ = false;
};

}  // namespace mccl
