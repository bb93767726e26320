// ref_bridge.cpp -- TEST INFRASTRUCTURE ONLY.
//
// Compiles the two torch-free pieces of the reference straight from the
// reference checkout (nothing is copied into this repository) and exposes
// them over a C ABI so tests can compare this repository's restatements with
// the reference's own code:
//   * chunkize, as held by tests/internal/test_ring_chunks.cpp:10-22 (the
//     reference's unit-test copy of AllreduceAlgos.cpp:22-34);
//   * mccl::Progress, csrc/backend/Progress.cpp (the FIFO task engine).
// MCCL_REF_ROOT is passed by the Makefile (-DMCCL_REF_ROOT=...).
#define MCCL_STR2(x) #x
#define MCCL_STR(x) MCCL_STR2(x)
#define MCCL_REF_FILE(rel) MCCL_STR(MCCL_REF_ROOT/rel)

// The reference's test file ends in MCCL_RUN_ALL(), which defines main();
// rename it so the file can live inside a shared library.
#define main mccl_ref_ring_chunks_main
#include MCCL_REF_FILE(tests/internal/test_ring_chunks.cpp)
#undef main

#include MCCL_REF_FILE(csrc/backend/Progress.hpp)

#include <cstdint>
#include <mutex>
#include <stdexcept>

extern "C" {

// out[4*i..4*i+3] = {elem_start, elem_end, byte_off, byte_len} of chunk i.
void ref_chunkize(int64_t numel, int world, uint64_t esize, int64_t* out) {
    auto c = chunkize(numel, world, static_cast<size_t>(esize));
    for (int i = 0; i < world; ++i) {
        out[4 * i + 0] = c[i].s;
        out[4 * i + 1] = c[i].e;
        out[4 * i + 2] = static_cast<int64_t>(c[i].off);
        out[4 * i + 3] = static_cast<int64_t>(c[i].len);
    }
}

// Runs the reference's own chunkize test cases; returns its failure count.
int ref_ring_chunks_selftest(void) { return mccl_ref_ring_chunks_main(); }

// Submits n tasks (task i throws if throw_mask bit (i % 64) is set and i < 64),
// shuts the engine down, writes the order in which non-throwing tasks ran.
int ref_progress_order(int n, uint64_t throw_mask, int* order_out) {
    std::mutex mu;
    int ran = 0;
    {
        mccl::Progress p;
        for (int i = 0; i < n; ++i) {
            bool thr = i < 64 && ((throw_mask >> i) & 1u);
            p.submit([i, thr, &mu, &ran, order_out] {
                if (thr) throw std::runtime_error("boom");
                std::lock_guard<std::mutex> lk(mu);
                order_out[ran++] = i;
            });
        }
        p.shutdown();
        p.shutdown();
    }
    return ran;
}

}  // extern "C"
