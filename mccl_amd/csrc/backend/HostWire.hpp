// HostWire.hpp -- one rank's allreduce over a host-memory wire.
//
// The default path of this backend lets the last rank to arrive launch the
// device work of the whole group and read the peers' chunks where they lie in
// HBM.  The host-wire modes run the collective the way the reference does, rank
// by rank, with every chunk crossing a byte transport in host memory
// (PeerMesh::send / recv, csrc/backend/AllreduceAlgos.cpp:62-86,151-200):
//
//   MCCL_WIRE=host    zero-copy: a rank encodes what it sends straight into
//                     pinned, device-mapped host memory; the wire delivers into
//                     the receiver's pinned buffer; the receiver's fold reads the
//                     peers' chunks from there through the device alias (PCIe),
//                     its own operand from HBM, and writes the result to HBM and,
//                     in wire form, back to pinned memory for the allgather leg.
//   MCCL_WIRE=staged  for wires that deliver into memory the GPU cannot map: the
//                     wire form is built in HBM, mcclx_stage_for_send moves it to a
//                     pinned staging buffer for the send, received bytes land in
//                     pageable memory and mcclx_unstage_from_recv moves them to HBM
//                     (stage_for_send_nosync / unstage_from_recv of the reference,
//                     csrc/metal/MPSInterop.mm:365-435).
//
// The arithmetic is the fused schedule's: the final owner of a chunk folds all
// operands in the schedule's order in one pass, so the result is bit-identical
// to the default path and to the reference's step-by-step schedule.
#pragma once

#include <ATen/ATen.h>

#include <chrono>
#include <cstdint>
#include <memory>
#include <vector>

#include "backend/LocalMesh.hpp"
#include "mcclx.h"

namespace mccl {

class HostWire {
public:
    enum class Mode { Pinned, Staged };

    // What the last allreduce moved and how long its fold launch took (device time).
    struct Stats {
        uint64_t calls = 0;
        uint64_t fold_elems = 0;           // elements this rank folded in the last call
        uint64_t fold_peer_bytes = 0;      // bytes of peer operands the fold read (across PCIe in Pinned mode)
        uint64_t fold_hbm_bytes = 0;       // bytes the fold read from and wrote to HBM
        double fold_ms = 0.0;
        uint64_t wire_bytes_sent = 0;      // bytes this rank handed to the transport in the last call
        // host wall-clock milliseconds of the last call's legs: wire form of what is sent (encode,
        // drained), reduce-scatter leg of the wire, fold (drained), allgather leg, casts on arrival
        double leg_ms[5] = {0, 0, 0, 0, 0};
    };

    HostWire(std::shared_ptr<LocalMesh> mesh, int rank, int device, std::chrono::milliseconds timeout);
    ~HostWire();
    HostWire(const HostWire&) = delete;
    HostWire& operator=(const HostWire&) = delete;

    // In-place allreduce of this rank's tensor; every rank of the mesh calls it with
    // the same numel, dtype, op, algorithm and codec setting.  Blocks until this
    // rank's tensor holds the result (the reference's allreduce is synchronous,
    // ProcessGroupMCCL.cpp:170-185).  `torch_stream` is the stream the tensor was
    // produced on.  Supports up to MCCLX_MAX_INPUTS ranks.
    void allreduce(void* tensor, int dtype, uint64_t numel, int op, int algo, bool wire_bf16, Mode mode,
                   void* torch_stream);

    const Stats& stats() const { return stats_; }

private:
    struct Pinned;  // a device-mapped pinned allocation, freed with its context
    struct Ctx;     // this rank's own reduce queue

    std::shared_ptr<Pinned> pinned(std::shared_ptr<Pinned>& slot, uint64_t nbytes);
    void* device_scratch(at::Tensor& slot, uint64_t nbytes);

    LocalPeer peer_;
    int rank_, world_, device_;
    std::shared_ptr<Ctx> ctx_;
    // Two send buffers, used in turn: a peer may still be copying this rank's last
    // message of call n out of its send buffer while this rank already encodes call
    // n+1.  Nobody can finish call n+1 before every rank has finished call n (every
    // fold needs an operand from every rank), so call n+2 may take call n's buffer.
    std::shared_ptr<Pinned> send_pin_[2], recv_a_pin_, recv_b_pin_;
    at::Tensor send_dev_, recv_a_dev_, recv_b_dev_;  // Staged mode: the same buffers in HBM
    std::vector<uint8_t> pageable_;                  // Staged mode: where the wire delivers
    Stats stats_;
};

}  // namespace mccl
