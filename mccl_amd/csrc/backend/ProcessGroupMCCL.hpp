// ProcessGroupMCCL.hpp -- backend "mccl" for ROCm tensors: the c10d::Backend
// surface of the reference (csrc/backend/ProcessGroupMCCL.hpp:43-94) over the
// reduce + wire-codec path in libmcclx.
//
// The collectives keep the reference's observable behaviour (which run on the
// caller's thread, which on the FIFO engine, what fails how).  What differs is
// underneath: a group of N > 1 ranks lives inside one process on one GPU, its
// ranks meet in a LocalMesh instead of over TCP, and the last rank to arrive
// launches the device work of the whole group through the chunk scheduler.
// A group of size 1 completes every collective at once, like the reference.
#pragma once

#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>

#include <ATen/ATen.h>

#include <chrono>
#include <functional>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "mcclx.h"

namespace mccl {

class Progress;
class LocalMesh;
class HostWire;
struct Contribution;
struct WaitMarks;

class ProcessGroupMCCL : public c10d::Backend {
    using Tensors = std::vector<at::Tensor>;
    using TensorLists = std::vector<std::vector<at::Tensor>>;
    using WorkPtr = c10::intrusive_ptr<c10d::Work>;

public:
    struct Options {
        std::chrono::milliseconds timeout{30 * 60 * 1000};
    };

    ProcessGroupMCCL(c10::intrusive_ptr<c10d::Store> store, int rank, int size, Options opts);
    ~ProcessGroupMCCL() override;

    const std::string getBackendName() const override { return "mccl"; }

    // reductions: the hot path.  allreduce blocks and returns a finished Work
    // (ProcessGroupMCCL.cpp:105-186); the others run on the engine thread.
    WorkPtr allreduce(Tensors& tensors, const c10d::AllreduceOptions& opts = {}) override;
    WorkPtr _reduce_scatter_base(at::Tensor& output, at::Tensor& input,
                                 const c10d::ReduceScatterOptions& opts = {}) override;
    WorkPtr reduce_scatter(Tensors& outputs, TensorLists& inputs,
                           const c10d::ReduceScatterOptions& opts = {}) override;

    // data movement between the ranks of the group
    WorkPtr _allgather_base(at::Tensor& output, at::Tensor& input, const c10d::AllgatherOptions& opts = {}) override;
    WorkPtr allgather(TensorLists& outputs, Tensors& inputs, const c10d::AllgatherOptions& opts = {}) override;
    WorkPtr broadcast(Tensors& tensors, const c10d::BroadcastOptions& opts = {}) override;
    WorkPtr alltoall_base(at::Tensor& output, at::Tensor& input, std::vector<int64_t>& output_split_sizes,
                          std::vector<int64_t>& input_split_sizes, const c10d::AllToAllOptions& opts = {}) override;
    WorkPtr alltoall(Tensors& outputs, Tensors& inputs, const c10d::AllToAllOptions& opts = {}) override;
    WorkPtr send(Tensors& tensors, int dst_rank, int tag) override;
    WorkPtr recv(Tensors& tensors, int src_rank, int tag) override;
    WorkPtr barrier(const c10d::BarrierOptions& opts = {}) override;

    // Algorithm the last allreduce on this rank ran (MCCLX_ALGO_*), for tests.
    int lastAlgo() const { return last_algo_; }
    // Allreduces of this rank's group that were replayed from a recorded graph, for tests.
    uint64_t graphHits() const;
    // Event-based allreduces of this rank's group: (launches issued, buckets they carried), and the
    // kernel launches the group's reduce queue has issued so far; for tests and the benchmark.
    std::pair<uint64_t, uint64_t> asyncStats() const;
    uint64_t launchCount() const;
    // The last host-wire allreduce of this rank (MCCL_WIRE=host|staged): elements folded, bytes of
    // peer operands the fold read, device milliseconds of the fold launch, bytes handed to the wire,
    // then the host milliseconds of its five legs (wire form, reduce-scatter leg, fold, allgather leg, casts).
    std::vector<double> wireStats() const;

private:
    struct Shared;  // reduce queue, scratch and recorded graphs shared by the ranks of one mesh

    void meet(Contribution c, const std::function<void(const std::vector<Contribution>&)>& leader);
    void meet_built(int kind, void* stream, const std::function<void(Contribution&)>& build,
                    const std::function<void(const std::vector<Contribution>&)>& leader);
    void* my_stream() const;
    void flush_engine_();

    c10::intrusive_ptr<c10d::Store> store_;
    Options opts_;
    int device_ = 0;
    mcclx_ctx* ctx_ = nullptr;          // size == 1: own context; size > 1: the mesh's
    std::shared_ptr<Shared> shared_;
    std::shared_ptr<LocalMesh> mesh_;
    std::string mesh_key_;
    std::unique_ptr<Progress> engine_;
    std::shared_ptr<WaitMarks> wait_marks_;  // event-based allreduce: what this rank's stream already waits for
    std::unique_ptr<HostWire> host_wire_;  // MCCL_WIRE=host|staged: this rank's end of the byte transport
    int last_algo_ = -1;
};

}  // namespace mccl
