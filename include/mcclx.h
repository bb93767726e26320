/*
 * mcclx.h -- C ABI of the MI355X reduce + wire-codec library (libmcclx.so).
 *
 * This is the boundary a maintainer of dormlab/mccl binds in place of the
 * calls csrc/backend makes into csrc/metal.  Plain pointers and sizes only:
 * no torch types, no C++ types, no exceptions.  Every function returns
 * MCCLX_OK (0) or a negative error code; mcclx_last_error() gives the message
 * of the last failure on the calling thread.
 *
 * Memory: the library never owns caller buffers.  Every `void*` data pointer
 * must be readable/writable by the GPU (HBM, or pinned host memory mapped into
 * the device address space -- see mcclx_host_alloc).  Pointers only need
 * element alignment; 16-byte aligned buffers run fastest.  An output may alias
 * one input exactly (same address, in-place reduce); any other overlap between
 * an output and an input of the same launch is undefined.
 *
 * Ordering: every launch is asynchronous on the context's reduce queue (one HIP
 * stream per context) and ordered after earlier launches on that queue.
 * mcclx_queue_drain blocks the host until the queue is empty.
 *
 * Reference citations are paths inside the dormlab/mccl checkout.
 */
#ifndef MCCLX_H
#define MCCLX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MCCLX_API __attribute__((visibility("default")))
/* 2: mcclx_plan.flags (was a reserved field that had to be 0), mcclx_fold_batched_noalloc,
 *    mcclx_probe_stream (gone again in 4).  Layouts of version 1 callers stay valid.
 * 3: MCCLX_IO_ALL_F32, MCCLX_REPLAY_DIRECT, mcclx_set_hold, mcclx_hold_launch_count.
 *    Layouts unchanged.
 * 4: mcclx_hold_model; the measurement aids mcclx_probe_stream and mcclx_timer_begin / _end
 *    left the library (the measurement build declares its own in mcclx_bench.h).
 *    Layouts unchanged. */
#define MCCLX_ABI_VERSION 4
#define MCCLX_MAX_INPUTS 8 /* inputs one launch folds; wider worlds chain launches */

/* ---- codes ---------------------------------------------------------------- */

enum {
    MCCLX_OK = 0,
    MCCLX_ERR_INVALID = -1,     /* bad argument (null pointer, k out of range, ...)      */
    MCCLX_ERR_UNSUPPORTED = -2, /* "Unsupported ReduceOp" / no kernel for dtype          */
    MCCLX_ERR_HIP = -3,         /* a HIP runtime call failed                             */
    MCCLX_ERR_STATE = -4,       /* wrong state: batch already active, context destroyed  */
    MCCLX_ERR_NOMEM = -5
};

/* element types the reference's kernels cover (shaders.metal: f32 / f16 / bf16) */
enum { MCCLX_F32 = 0, MCCLX_F16 = 1, MCCLX_BF16 = 2 };

/* numeric values of c10d::ReduceOp::RedOpType */
enum { MCCLX_SUM = 0, MCCLX_AVG = 1, MCCLX_PRODUCT = 2, MCCLX_MIN = 3, MCCLX_MAX = 4 };

/* how a 16-bit scale constant is derived from (float)scale */
enum {
    MCCLX_SCALE_NONE = 0,
    MCCLX_SCALE_VIEW = 1,  /* bf16: bits >> 16, truncation (MetalKernels.mm:659-662)   */
    MCCLX_SCALE_TENSOR = 2 /* bf16: round to nearest even (MetalKernels.mm:390-392)    */
};

/* where the operands of a fold live, relative to its arithmetic dtype W */
enum {
    MCCLX_IO_PURE = 0,          /* every input and the output are W                     */
    MCCLX_IO_OUT_F32 = 1,       /* W = bf16: inputs bf16, output fp32 (decode on store) */
    MCCLX_IO_OWN_FIRST_F32 = 2, /* W = bf16: in[0] fp32 (encoded in registers), out fp32 */
    MCCLX_IO_OWN_LAST_F32 = 3,  /* W = bf16: in[k-1] fp32, out fp32 (ring order)        */
    MCCLX_IO_ALL_F32 = 4        /* W = bf16: every input fp32 (each encoded in registers,
                                   the cast of ProcessGroupMCCL.cpp:131-132), out fp32: ranks
                                   that share one GPU read each other's tensors where they
                                   lie, and no wire copy is ever written                    */
};

enum {
    MCCLX_TOPO_FOLD = 0,    /* ((in0 op in1) op in2) ... : ring, butterfly, reduce_scatter */
    MCCLX_TOPO_BINOMIAL = 1 /* binomial tree of allreduce_tree (AllreduceAlgos.cpp:100-114) */
};

enum {
    MCCLX_ACC_STEP = 0, /* round to W after every operation: bit-exact to the reference   */
    MCCLX_ACC_F32 = 1   /* NOT the reference: fp32 accumulator, the scale applied as
                           (float)scale in fp32, one final rounding (inside one fold: a
                           world wider than MCCLX_MAX_INPUTS chains folds and rounds between) */
};

enum { MCCLX_ALGO_RING = 0, MCCLX_ALGO_TREE = 1, MCCLX_ALGO_BUTTERFLY = 2 };

typedef struct mcclx_ctx mcclx_ctx; /* opaque: device, reduce queue, events, staging */

MCCLX_API const char* mcclx_last_error(void);
MCCLX_API int mcclx_abi_version(void);

/* ---- context = kernel cache + reduce queue --------------------------------- */

/* Replaces metal_kernels_init (MetalKernels.mm:189-325) and the dedicated
 * command queue (MPSInterop.mm:32-36).  Creates a HIP stream at the default
 * priority on `device`. */
MCCLX_API int mcclx_init(int device, mcclx_ctx** out);
/* Same, but the reduce queue IS `hip_stream` (a hipStream_t owned by the
 * caller, e.g. PyTorch's current stream); nothing is created or destroyed. */
MCCLX_API int mcclx_init_on_stream(int device, void* hip_stream, mcclx_ctx** out);
MCCLX_API int mcclx_destroy(mcclx_ctx* ctx);
/* The queue's hipStream_t, for callers that enqueue their own work on it. */
MCCLX_API void* mcclx_queue_stream(mcclx_ctx* ctx);
/* Number of compute units of the context's device (sizing of persistent grids). */
MCCLX_API int mcclx_device_cus(mcclx_ctx* ctx);

/* Diagnostic: kernel launches this context has issued so far (recorded ones
 * count when they are recorded, not when a graph replays them). */
MCCLX_API uint64_t mcclx_launch_count(mcclx_ctx* ctx);

/* The hold form of a fold launch (no counterpart in the reference; results are
 * the same bits).  A launch that mixes reads and writes streams about 10 %
 * slower on this part than one that only reads or only writes.  A by-value
 * fold launch (up to 32 segments) of two to four operands that reads at least
 * 10 MiB (15 MiB with fan-out) and is small enough for one generation of blocks to cover it -- a
 * 25 MiB gradient bucket is -- therefore issues all its loads first, holds its
 * results in registers and stores them only when its reads are through: the
 * host passes, from the bytes the launch reads, the time before which no lane
 * stores.  That model assumes the launch has the memory system to itself: a
 * queue whose launches run next to other work on the GPU (a second reduce
 * queue) does better without it.  enabled = 0 switches the form off for this
 * context, 1 on again; MCCLX_HOLD=0 in the environment switches it off for
 * every context made afterwards. */
MCCLX_API int mcclx_set_hold(mcclx_ctx* ctx, int enabled);
/* Diagnostic: launches of this context that took the hold form. */
MCCLX_API uint64_t mcclx_hold_launch_count(mcclx_ctx* ctx);
/* Diagnostic: the model behind that time -- no store before `latency_ticks` +
 * bytes read / `bytes_per_tick` ticks of a 100 MHz clock after a block's start.
 * The rate is measured on the device when the first context of a process is made
 * on it (two read-only launches over scratch memory; MCCLX_HOLD_CALIBRATE=0 keeps
 * the built-in value).  Returns 1 if this context's rate was measured, 0 if it is
 * the built-in value or an MCCLX_HOLD_BYTES_PER_TICK override. */
MCCLX_API int mcclx_hold_model(mcclx_ctx* ctx, uint32_t* latency_ticks, uint32_t* bytes_per_tick);

/* ---- the reference's four kernel entry points, one to one ------------------- */

/* dst[i] = dst[i] (op) src[i].  Replaces metal_reduce_op_view
 * (MetalKernels.mm:628-640) and metal_reduce_op (:530-550); AVG runs the SUM
 * kernel as select_op_pipeline (:606-624) does.  `count` is 64-bit (the
 * reference narrows to uint32, MetalKernels.mm:156-163).  Does not drain. */
MCCLX_API int mcclx_reduce(mcclx_ctx* ctx, void* dst, const void* src, int dtype, uint64_t count, int op);

/* buf[i] *= s.  Replaces metal_scale_inplace_view (MetalKernels.mm:642-674,
 * scale_mode VIEW) and metal_scale_inplace (:365-405, scale_mode TENSOR). */
MCCLX_API int mcclx_scale(mcclx_ctx* ctx, void* buf, int dtype, uint64_t count, double scale,
                int scale_mode);

/* dst[i] = (dst[i] + src[i]) * s.  Replaces metal_accumulate_and_scale
 * (MetalKernels.mm:408-458; 16-bit types round after the add and after the
 * multiply, constant as scale_mode TENSOR). */
MCCLX_API int mcclx_accumulate_scale(mcclx_ctx* ctx, void* dst, const void* src, int dtype, uint64_t count,
                           double scale);

/* Reuse of one submission for many launches.  Replaces metal_begin_batch /
 * metal_end_batch (MetalKernels.mm:559-577).  HIP launches are already
 * asynchronous, so a batch only (a) rejects nesting like the reference
 * ("Metal batch already active") and (b) is a no-op to end when none is open. */
MCCLX_API int mcclx_batch_begin(mcclx_ctx* ctx, const char* label);
MCCLX_API int mcclx_batch_end(mcclx_ctx* ctx);

/* ---- wire codec (done by torch casts in the reference) ---------------------- */

/* dst_bf16[i] = RNE(src_f32[i]); NaN -> 0x7FC0.  Replaces `t.to(at::kBFloat16)`
 * (ProcessGroupMCCL.cpp:131-132). */
MCCLX_API int mcclx_encode_bf16(mcclx_ctx* ctx, void* dst_bf16, const void* src_f32, uint64_t count);
/* dst_f32[i] = bits(src_bf16[i]) << 16.  Replaces `tensors[i].copy_(work.to(fp32))`
 * (ProcessGroupMCCL.cpp:179-183). */
MCCLX_API int mcclx_decode_bf16(mcclx_ctx* ctx, void* dst_f32, const void* src_bf16, uint64_t count);

/* ---- fused multi-input fold (new; replaces N-1 binary launches + casts) ------ */

typedef struct {
    void* out;       /* primary output (W, or fp32 for the *_F32 io modes); may be NULL if wire_out is set */
    void* wire_out;  /* optional second output of the same values in W (bf16 only); NULL if unused */
    const void* in[MCCLX_MAX_INPUTS]; /* in[0..k-1], in fold order */
    uint64_t count;  /* elements */
} mcclx_seg;

/* plan.flags.  By default every step of a fold computes op(dst = partial
 * result, src = in[j]): the roles the butterfly, the tree and reduce_scatter
 * give their operands (AllreduceAlgos.cpp:108-111,172-180,
 * ProcessGroupMCCL.cpp:378-386).  The ring reduces the travelling partial
 * result INTO the receiver's own chunk, op(dst = in[j], src = partial)
 * (AllreduceAlgos.cpp:72-74); MIN and MAX keep dst on a tie or a NaN
 * (shaders.metal:65-72), so they can tell the two apart. */
#define MCCLX_PLAN_ACC_IS_SRC 1
/* Fan-out: the result is also written to n further destinations, in[k] ..
 * in[k+n-1], in the form `out` has (the allgather leg of an allreduce done by
 * the reduce itself: the owner stores its reduced chunk into every other
 * rank's tensor instead of a second pass reading it back; with the bf16 wire
 * the other ranks' cast of the wire copy, ProcessGroupMCCL.cpp:179-183, yields
 * the very fp32 values the owner holds).  A destination may be one of the
 * operands.  Sums with per-step rounding only, k + n <= MCCLX_MAX_INPUTS, `out`
 * required, io PURE or OWN_*_F32. */
#define MCCLX_PLAN_FANOUT_SHIFT 8
#define MCCLX_PLAN_FANOUT_MASK 0x700
#define MCCLX_PLAN_FANOUT(n) ((n) << MCCLX_PLAN_FANOUT_SHIFT)

typedef struct {
    int32_t dtype;      /* W: MCCLX_F32 / F16 / BF16                                  */
    int32_t io;         /* MCCLX_IO_*  (non-PURE needs W = bf16)                      */
    int32_t k;          /* 1..MCCLX_MAX_INPUTS                                        */
    int32_t topo;       /* MCCLX_TOPO_*                                               */
    int32_t op;         /* MCCLX_SUM/AVG(=SUM)/PRODUCT/MIN/MAX                        */
    int32_t acc;        /* MCCLX_ACC_*                                                */
    int32_t scale_mode; /* MCCLX_SCALE_*; NONE ignores `scale`                        */
    int32_t flags;      /* MCCLX_PLAN_* bits, 0 otherwise                             */
    double scale;       /* e.g. 1.0 / world (AllreduceAlgos.cpp:88-91)                */
} mcclx_plan;

/* One launch: out = [scale *] fold(in[0..k-1]) over one segment.
 * With acc = STEP the result is bit-identical to running the reference's
 * binary kernels one peer at a time in the same order (plus its scale pass
 * and, for the *_F32 io modes, its encode/decode casts). */
MCCLX_API int mcclx_fold(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* seg);

/* One launch over `nseg` independent segments sharing a plan:
 * the tree path's many sub-256 KB messages, or all virtual ranks' chunks of
 * one schedule phase.  Segment descriptors are copied before the call returns. */
MCCLX_API int mcclx_fold_batched(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* segs,
                       uint32_t nseg);

/* The batched fold for callers that cannot allocate.  It has no counterpart
 * in the reference: it exists for code under HIP graph capture, tight serving
 * loops and harnesses that forbid hipMalloc.  Same arguments, checks and
 * results as mcclx_fold_batched, but the call allocates nothing on the device
 * or the host: up to 32 segments travel in the kernel
 * arguments, more go through a descriptor table in a static device array
 * (128 KiB per GPU, held until the process ends) that small writer kernels
 * fill from their own arguments -- the whole call is kernel launches only.
 * More than MCCLX_NOALLOC_MAX_SEGS segments are refused with MCCLX_ERR_INVALID.
 * Every call on a GPU shares that GPU's array: calls on one context are
 * ordered by its queue; a call that enters while another thread's call on the
 * same GPU is still filling the array is refused with MCCLX_ERR_STATE; launches
 * of different contexts that are both queued and overlap on the device race.
 * Nothing in the array needs to start at zero; each call overwrites the part it
 * reads.  Launches of up to 32 segments of similar length carry their
 * descriptors in the kernel arguments and do not touch the array. */
#define MCCLX_NOALLOC_MAX_SEGS 1024
MCCLX_API int mcclx_fold_batched_noalloc(mcclx_ctx* ctx, const mcclx_plan* plan, const mcclx_seg* segs,
                               uint32_t nseg);

/* dst <- src, nbytes, on the reduce queue.  Replaces unstage_from_recv
 * (MPSInterop.mm:408-435) and the allgather legs (AllreduceAlgos.cpp:77-86,
 * ProcessGroupMCCL.cpp:232-273). */
MCCLX_API int mcclx_copy(mcclx_ctx* ctx, void* dst, const void* src, uint64_t nbytes);

/* Many copies with one launch: the allgather leg of a schedule hands every
 * reduced chunk to every other rank (AllreduceAlgos.cpp:77-86, 185-200; the
 * tree's broadcast :119-126), N-1 sends per chunk in the reference.  Ranges of
 * different descriptors must not overlap each other's destinations; a
 * descriptor with nbytes == 0 or dst == src is skipped.  A few large copies are
 * issued one launch each (that streams best); many small ones go out together. */
typedef struct mcclx_copy_desc {
    void* dst;
    const void* src;
    uint64_t nbytes;
} mcclx_copy_desc;
MCCLX_API int mcclx_copy_batched(mcclx_ctx* ctx, const mcclx_copy_desc* descs, uint32_t n);

/* ---- reduce queue: completion and cross-stream ordering --------------------- */

/* Block until every launch on the queue has finished.  Replaces
 * mccl_queue_drain (MPSInterop.mm:312-318) and metal_sync (MetalKernels.mm:552). */
MCCLX_API int mcclx_queue_drain(mcclx_ctx* ctx);
/* The queue waits (on the device, host not blocked) for everything enqueued so
 * far on `producer_stream`.  Replaces mps_stream_sync (MPSInterop.mm:308-310)
 * and mps_event_sync_nonblocking + wait_for_mps (:336-356, EventSync.mm:112-132). */
MCCLX_API int mcclx_queue_wait_stream(mcclx_ctx* ctx, void* producer_stream);
/* `consumer_stream` waits for everything enqueued so far on the queue: the
 * non-blocking form of "queue drained before the Work completes"
 * (ProcessGroupMCCL.cpp:178, WorkMCCL.cpp:71-90). */
MCCLX_API int mcclx_stream_wait_queue(mcclx_ctx* ctx, void* consumer_stream);
/* Record a completion ticket / test it / wait for it (EventSync.mm:112-132). */
MCCLX_API int mcclx_event_record(mcclx_ctx* ctx, uint64_t* ticket);
MCCLX_API int mcclx_event_query(mcclx_ctx* ctx, uint64_t ticket, int* done);
MCCLX_API int mcclx_event_wait(mcclx_ctx* ctx, uint64_t ticket);

/* ---- launch graphs ---------------------------------------------------------- */

/* Gradient buckets have fixed shapes and addresses, so the launches of one
 * bucket's reduction can be recorded once and replayed every iteration with a
 * single submission -- the HIP form of the reference's "many launches, one
 * command buffer" batch (MetalKernels.mm:559-577).  Between graph_begin and
 * graph_end every launch on this context is recorded instead of executed
 * (queue_drain and event_* are refused while recording).  Buffers
 * named by recorded launches must stay valid for the graph's lifetime. */
typedef struct mcclx_graph mcclx_graph;
MCCLX_API int mcclx_graph_begin(mcclx_ctx* ctx);
MCCLX_API int mcclx_graph_end(mcclx_ctx* ctx, mcclx_graph** out);
MCCLX_API int mcclx_graph_launch(mcclx_ctx* ctx, mcclx_graph* graph);
MCCLX_API int mcclx_graph_destroy(mcclx_ctx* ctx, mcclx_graph* graph);

/* ---- host-buffer interop ---------------------------------------------------- */

/* Pinned host memory mapped into the device address space: what the wire
 * receives into and the kernels read directly (zero-copy).  Replaces the
 * shared-storage MTLBuffer view (MPSBufferView, MPSInterop.hpp:10-16) and the
 * staging pool (MPSInterop.mm:47-204).  *device_ptr is what kernels take. */
MCCLX_API int mcclx_host_alloc(mcclx_ctx* ctx, uint64_t nbytes, void** host_ptr, void** device_ptr);
MCCLX_API int mcclx_host_free(mcclx_ctx* ctx, void* host_ptr);

/* Staging for memory the host cannot address (HBM), the other way the
 * reference moves tensors to and from the wire (MPSInterop.mm:365-435):
 *   stage_for_send   device -> a pinned staging buffer owned by the context;
 *                    blocks until the bytes are there; *host_ptr stays valid
 *                    until the next stage_for_send on this context
 *                    (StagingBuffer, MPSInterop.hpp:45-51).  Source memory that
 *                    is already host-addressable (mcclx_host_alloc) is returned
 *                    as is, without a copy ("direct CPU path", :373-376).
 *   unstage_from_recv host bytes (any host memory) -> device, asynchronously on
 *                    the reduce queue; pageable sources go through the pinned
 *                    staging buffer in pipelined chunks (chunked blits, :47-204). */
MCCLX_API int mcclx_stage_for_send(mcclx_ctx* ctx, const void* device_src, uint64_t nbytes, void** host_ptr);
MCCLX_API int mcclx_unstage_from_recv(mcclx_ctx* ctx, void* device_dst, const void* host_src, uint64_t nbytes);

/* ---- chunk scheduler -------------------------------------------------------- */

typedef struct {
    int64_t elem_start;
    int64_t elem_count;
    uint64_t byte_off;
    uint64_t byte_len;
} mcclx_chunk;

/* chunkize (AllreduceAlgos.cpp:22-34). */
MCCLX_API int mcclx_chunkize(int64_t numel, uint64_t elem_size, int world, mcclx_chunk* out);

/* Algorithm choice of ProcessGroupMCCL::allreduce (ProcessGroupMCCL.cpp:134-145).
 * env_algo NULL = MCCL_ALLREDUCE_ALGO unset; tree_below < 0 = MCCL_TREE_BELOW unset. */
MCCLX_API int mcclx_select_algo(const char* env_algo, int64_t tree_below, uint64_t wire_nbytes,
                      int64_t numel, int world);

enum {
    MCCLX_REPLAY_STEPWISE = 0, /* the reference's launches one by one (binary reduce per received chunk) */
    MCCLX_REPLAY_FUSED = 1,    /* one multi-input fold per owned chunk, peers read in place */
    MCCLX_REPLAY_DIRECT = 2    /* FUSED, and with the wire codec on a sum of up to MCCLX_MAX_INPUTS
                                  ranks the fold reads every rank's fp32 tensor where it lies and
                                  encodes it in registers (MCCLX_IO_ALL_F32): no rank writes a bf16
                                  copy, there is no encode launch.  For ranks that share one GPU,
                                  where the wire is HBM and an fp32 read costs less than writing
                                  and re-reading a bf16 copy; across GPUs FUSED keeps the link
                                  traffic at 2 bytes per element.  Elsewhere the same as FUSED.  */
};

typedef struct {
    int32_t world;      /* virtual ranks, >= 1                                         */
    int32_t algo;       /* MCCLX_ALGO_*                                                */
    int32_t op;         /* MCCLX_SUM / AVG / PRODUCT / MIN / MAX                       */
    int32_t dtype;      /* dtype of the rank tensors                                   */
    int32_t wire_bf16;  /* MCCL_WIRE_DTYPE=bf16 (only acts on fp32 tensors)            */
    int32_t mode;       /* MCCLX_REPLAY_*                                              */
    int32_t acc;        /* MCCLX_ACC_* (FUSED and DIRECT only)                         */
    int32_t reserved;
    uint64_t numel;
    void* const* tensors;  /* world device pointers; reduced in place                  */
    void* workspace;       /* device-accessible scratch (HBM or mapped pinned host)    */
    uint64_t workspace_bytes;
} mcclx_replay;

/* Scratch a replay needs: the recv scratch of ProcessGroupMCCL.cpp:152-162 per
 * virtual rank plus, with the wire codec, one bf16 copy per rank.  0 for a
 * DIRECT replay whose fold also hands the result to every rank (a sum of up to
 * four ranks): `workspace` may then be NULL. */
MCCLX_API uint64_t mcclx_replay_workspace_bytes(const mcclx_replay* r);

/* Single-process replay of allreduce_ring / _tree / _butterfly
 * (AllreduceAlgos.cpp:52-206) for `world` virtual ranks whose tensors all live
 * on this GPU: every send/recv becomes a device copy (STEPWISE) or a direct
 * read of the peer's chunk (FUSED, DIRECT).  All modes produce bit-identical tensors. */
MCCLX_API int mcclx_allreduce_replay(mcclx_ctx* ctx, const mcclx_replay* r);

/* The same for a list of tensors, as ProcessGroupMCCL::allreduce takes one
 * (ProcessGroupMCCL.cpp:122-168 runs the list one tensor after another).  Here
 * consecutive entries that share world, algorithm, op, dtype and wire setting
 * are issued together: one launch per phase (encode, fold, cast, copies) for
 * the whole run instead of one per tensor -- thousands of small tree messages
 * become a handful of launches.  Results are those of n single replays. */
MCCLX_API int mcclx_allreduce_replay_many(mcclx_ctx* ctx, const mcclx_replay* replays, uint32_t n);

/* _reduce_scatter_base (ProcessGroupMCCL.cpp:331-390): ins[r] holds
 * world*chunk_numel elements, outs[r] receives chunk_numel.  FUSED: one
 * k=world fold per rank in one batched launch. */
MCCLX_API int mcclx_reduce_scatter_replay(mcclx_ctx* ctx, int world, void* const* outs,
                                const void* const* ins, int dtype, uint64_t chunk_numel, int op,
                                int mode, int acc);

/* The list form, reduce_scatter (ProcessGroupMCCL.cpp:392-464): shares[r*world + p]
 * is rank p's contribution to rank r's output (chunk_numel elements each). */
MCCLX_API int mcclx_reduce_scatter_shares(mcclx_ctx* ctx, int world, void* const* outs,
                                const void* const* shares, int dtype, uint64_t chunk_numel,
                                int op, int mode, int acc);

/* _allgather_base (ProcessGroupMCCL.cpp:232-273): outs[r] = concat_p ins[p]. */
MCCLX_API int mcclx_allgather_replay(mcclx_ctx* ctx, int world, void* const* outs, const void* const* ins,
                           uint64_t chunk_nbytes);

#ifdef __cplusplus
}
#endif
#endif /* MCCLX_H */
