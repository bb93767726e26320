// ProcessGroupMCCL.hpp -- the c10d Backend surface of the reference
// (csrc/backend/ProcessGroupMCCL.hpp:43-94) for ROCm tensors.
//
// Same virtuals, same option structs, same error behaviour; the work behind
// them is the reduce + wire-codec path in libmcclx (C ABI), reached through
// the chunk scheduler.  A group of size 1 completes every collective at once,
// like the reference.  A group of size N > 1 lives inside one process on one
// GPU: its ranks meet in a LocalMesh instead of over TCP.
//
// In scope: allreduce, reduce_scatter (+ _base), allgather (+ _base), plus
// broadcast and barrier (pure copies / a rendezvous, needed by callers such as
// DistributedDataParallel).  alltoall, send and recv move bytes between
// processes without any arithmetic; they return a failed Work here.
#pragma once

#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>

#include <ATen/ATen.h>

#include <chrono>
#include <memory>
#include <string>
#include <vector>

#include "mcclx.h"

namespace mccl {

class Progress;
class LocalMesh;
struct Contribution;

class ProcessGroupMCCL : public c10d::Backend {
public:
    struct Options {
        std::chrono::milliseconds timeout{30 * 60 * 1000};
    };

    ProcessGroupMCCL(c10::intrusive_ptr<c10d::Store> store, int rank, int size, Options opts);
    ~ProcessGroupMCCL() override;

    const std::string getBackendName() const override { return "mccl"; }

    c10::intrusive_ptr<c10d::Work> allreduce(std::vector<at::Tensor>& tensors,
                                             const c10d::AllreduceOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> broadcast(std::vector<at::Tensor>& tensors,
                                             const c10d::BroadcastOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> allgather(std::vector<std::vector<at::Tensor>>& output_tensors,
                                             std::vector<at::Tensor>& input_tensors,
                                             const c10d::AllgatherOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> _allgather_base(at::Tensor& output_tensor, at::Tensor& input_tensor,
                                                   const c10d::AllgatherOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> reduce_scatter(std::vector<at::Tensor>& output_tensors,
                                                  std::vector<std::vector<at::Tensor>>& input_tensors,
                                                  const c10d::ReduceScatterOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> _reduce_scatter_base(at::Tensor& output_tensor, at::Tensor& input_tensor,
                                                        const c10d::ReduceScatterOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> alltoall_base(at::Tensor& output_tensor, at::Tensor& input_tensor,
                                                 std::vector<int64_t>& output_split_sizes,
                                                 std::vector<int64_t>& input_split_sizes,
                                                 const c10d::AllToAllOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> alltoall(std::vector<at::Tensor>& output_tensors,
                                            std::vector<at::Tensor>& input_tensors,
                                            const c10d::AllToAllOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> barrier(const c10d::BarrierOptions& opts = {}) override;
    c10::intrusive_ptr<c10d::Work> send(std::vector<at::Tensor>& tensors, int dst_rank, int tag) override;
    c10::intrusive_ptr<c10d::Work> recv(std::vector<at::Tensor>& tensors, int src_rank, int tag) override;

    // Algorithm the last allreduce on this rank ran (MCCLX_ALGO_*), for tests.
    int lastAlgo() const { return last_algo_; }
    // Allreduces of this rank's group that were replayed from a recorded graph, for tests.
    uint64_t graphHits() const;

private:
    struct Shared;  // reduce queue + scratch shared by the ranks of one mesh

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
    int last_algo_ = -1;
};

}  // namespace mccl
