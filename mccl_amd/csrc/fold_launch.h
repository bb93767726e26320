// fold_launch.h -- host/device shared argument blocks of the fold kernels and
// the internal launch entry used by the C ABI (mcclx_api.cpp).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mcclx.h"

namespace mcclx {

// Segments that travel by value in the kernel arguments (32 x 88 B = 2.8 KB).
// A block that finds its descriptor there starts loading data at once; one that
// must first fetch it from a device table loses 5-10 % on large segments.
constexpr int kFewSegs = 32;

// Device-side view of mcclx_seg (same layout: the table is uploaded verbatim).
struct SegArgs {
    void* out;
    void* wire_out;
    const void* in[MCCLX_MAX_INPUTS];
    uint64_t count;
};
static_assert(sizeof(SegArgs) == sizeof(mcclx_seg), "SegArgs must mirror mcclx_seg");

// Launch-timeline instrumentation (a tuning build only, -DMCCLX_TUNE_TIMELINE=1):
// every block of a by-value fold launch records when it started, when its
// arguments had arrived and when it had issued its last store.
#ifndef MCCLX_TUNE_TIMELINE
#define MCCLX_TUNE_TIMELINE 0
#endif
struct TimelineRecord {
    uint64_t t_start, t_args, t_end;  // 100 MHz wall clock (10 ns ticks)
    uint32_t hw_id, xcc_id;           // where the block ran: HW_ID register, XCC_ID register
};

struct FewArgs {
    SegArgs seg[kFewSegs];
    float scale;        // the constant as the fp32 value the kernel multiplies by
    int32_t has_scale;
    int32_t nseg;
    int32_t fan;        // further destinations of the result, in[k .. k+fan-1] (fan-out kernels only)
#if MCCLX_TUNE_TIMELINE
    TimelineRecord* timeline;  // this launch's records, one per block (x fastest, then y), or null
#endif
};

struct TableArgs {
    const SegArgs* __restrict__ segs;         // device memory, nseg entries
    const uint64_t* __restrict__ first_item;  // device memory, nseg+1 prefix sums (unused when uniform)
    const uint2* __restrict__ item_map;       // device memory, (segment, tile) of every work item, or null
    uint64_t total_items;
    uint64_t uniform_items;      // >0: every segment has this many work items
    uint32_t nseg;
    float scale;
    int32_t has_scale;
    int32_t fan;                 // further destinations of the result, in[k .. k+fan-1] (fan-out kernels only)
};

// Kernel-side operator codes beyond the public MCCLX_* ones: MIN / MAX with the
// accumulator in the reference's `src` role (plan flag MCCLX_PLAN_ACC_IS_SRC).
enum { MCCLX_MIN_ACC_SRC = 5, MCCLX_MAX_ACC_SRC = 6 };

struct PlanKey {
    int dtype, io, k, topo, op, acc;
};

struct LaunchParams {
    const FewArgs* few = nullptr;      // exactly one of few / table is set
    const TableArgs* table = nullptr;
    uint32_t max_blocks = 0;           // cap on the grid (persistent sizing)
    int fan = 0;                       // > 0: the fan-out form of the kernel (plans in fan_plan_ok only)
    // Reads-then-writes form of a by-value launch that one generation of blocks covers:
    // taken when the launch reads at least hold_min_read_bytes (0 = never); no lane stores
    // before hold_latency_ticks + read bytes / hold_bytes_per_tick ticks of the 100 MHz
    // wall clock have passed since its block started.
    int cus = 0;
    bool* held = nullptr;              // set when the launch took that form (diagnostic)
    uint64_t hold_min_read_bytes = 0;
    uint32_t hold_latency_ticks = 40;
    uint32_t hold_bytes_per_tick = 72000;
};
// Plans that have a fan-out form: sums with per-step rounding, 2..7 operands.
bool fan_plan_ok(const PlanKey& key);

// Packets-per-lane unroll and threads per block the kernel template uses for this plan.
int plan_unroll(const PlanKey& key);
int plan_block(const PlanKey& key);
// Work items (tiles) a segment of `count` elements splits into under this plan.
uint32_t items_for(const PlanKey& key, uint64_t count);
// hipErrorInvalidValue = no kernel for this plan.
hipError_t launch_fold(hipStream_t st, const PlanKey& key, const LaunchParams& lp);

// Many copies in one launch: descriptors and nseg+1 work-item prefix sums in
// device memory (mirrors mcclx_copy_desc).
struct CopyDesc {
    void* dst;
    const void* src;
    uint64_t nbytes;
};
struct CopyTable {
    const CopyDesc* __restrict__ descs;
    const uint64_t* __restrict__ first_item;
    const uint2* __restrict__ item_map;  // (copy, tile) of every work item, or null
    uint32_t total_items;
    uint32_t uniform_items;  // >0: every copy has this many work items
    uint32_t n;
};
// A few copies by value in the kernel arguments (one grid: y = copy, x = tile).
constexpr int kFewCopies = 32;
struct CopyFew {
    CopyDesc d[kFewCopies];
    uint32_t n;
};
hipError_t launch_copy_few(hipStream_t st, const CopyFew& copies, int align);
// Work items (tiles) one copy of nbytes splits into.
uint64_t copy_items(uint64_t nbytes);
// `align`: the widest of 4 / 2 / 1 bytes that every pointer in the table is aligned to.
hipError_t launch_copy_many(hipStream_t st, const CopyTable& t, int align, uint32_t max_blocks);

// Plain device copy with the same packet shape (also the calibration kernel for
// the memory counters): dst <- src, nbytes.
hipError_t launch_copy(hipStream_t st, void* dst, const void* src, uint64_t nbytes,
                       uint32_t max_blocks);

// Reads (write == false) or writes nbytes of `buf` once, one 16-byte packet per
// lane like the copy kernel: the one-directional ceilings of a launch of that size.
hipError_t launch_stream_probe(hipStream_t st, void* buf, uint64_t nbytes, bool write);

// The allocation-free batched fold keeps its descriptor table in a static
// device array of kStaticTableBytes (one per GPU): room for
// MCCLX_NOALLOC_MAX_SEGS descriptors of 88 bytes plus their work-item prefix
// sums.  `static_table_resolve` returns that array's address on `device`, which
// must be the current device; `launch_table_write` stores up to kUploadWords
// 8-byte words there, carried in the kernel arguments of a one-block launch.
constexpr size_t kStaticTableBytes = 128 * 1024;
constexpr uint32_t kUploadWords = 448;  // 3584 bytes of payload per writer launch
static_assert((size_t)MCCLX_NOALLOC_MAX_SEGS * sizeof(SegArgs) +
                  ((size_t)MCCLX_NOALLOC_MAX_SEGS + 1) * sizeof(uint64_t) <= kStaticTableBytes,
              "the static table must hold the largest allocation-free launch");
hipError_t static_table_resolve(int device, void** out);
hipError_t launch_table_write(hipStream_t st, void* dst_words, const uint64_t* words, uint32_t n);

}  // namespace mcclx
