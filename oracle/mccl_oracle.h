/*
 * mccl_oracle.h -- CPU restatement of the reference's per-rank reduction path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it exists so that tests, the smoke check and the CPU leg of
 * the benchmark have an independent statement of what the reference computes.
 *
 * The reference (dormlab/mccl) has no CPU implementation of this path: the
 * arithmetic lives in Metal kernels (csrc/metal/shaders.metal) and, for the
 * bf16 wire codec, in PyTorch's tensor casts.  Every function below restates
 * one of those pieces in plain C and cites the file:line it follows.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_chunkize          reference's own chunkize compiled from
 *                         tests/internal/test_ring_chunks.cpp (oracle/_ref) and
 *                         that file's coverage/contiguity/degenerate cases.
 *   orc_f32_to_bf16 etc.  torch CPU `Tensor.to(torch.bfloat16)` -- the very
 *                         call the reference makes -- on every special value,
 *                         tie pair and a strided sweep of all 2^32 inputs.
 *   orc_reduce (bf16)     torch CPU bf16 add/mul/min/max, brute force pairs.
 *   orc_reduce (f32)      IEEE-754 fixes the result; numpy float32 check and
 *                         the reference's known-answer vectors.
 *   orc_reduce (f16)      numpy float16 arithmetic (exhaustive decode).
 *   orc_scale             closed forms: 1/2,1/4,1/8 exact; 1/3 constants
 *                         0x3EAAAAAB (f32), 0x3EAA (bf16 truncated, view
 *                         variant), 0x3EAB (bf16 RNE, tensor variant).
 *   orc_allreduce_*       hand-derived fold orders per algorithm, all ranks
 *                         bit-identical, exact integer sums, the reference
 *                         tests' rank+1 vectors.
 * Parity unpinned: MIN/MAX with a NaN operand or a +0/-0 tie, and fp16 NaN
 * payloads (Apple GPU behaviour under Metal fast-math is not specified); the
 * bit pattern of an encoded NaN (0x7FC0 here, as torch's scalar conversion;
 * torch's AVX path gives 0xFFFF, Metal's cast is unknown).
 */
#ifndef MCCL_ORACLE_H
#define MCCL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes (shared with the HIP library's C ABI) */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };

/* reduce ops: numeric values of c10d::ReduceOp::RedOpType */
enum { ORC_SUM = 0, ORC_AVG = 1, ORC_PRODUCT = 2, ORC_MIN = 3, ORC_MAX = 4 };

/* algorithms (csrc/backend/ProcessGroupMCCL.cpp:134-176) */
enum { ORC_ALGO_RING = 0, ORC_ALGO_TREE = 1, ORC_ALGO_BUTTERFLY = 2 };

/* how the bf16 scale constant is derived from (float)(1.0/world) */
enum {
    ORC_SCALE_VIEW = 0,  /* MetalKernels.mm:659-662 -- bits >> 16 (truncate)   */
    ORC_SCALE_TENSOR = 1 /* MetalKernels.mm:390-392 -- c10::BFloat16(float) RNE */
};

typedef struct {
    int64_t elem_start;
    int64_t elem_count;
    uint64_t byte_off;
    uint64_t byte_len;
} orc_chunk;

size_t orc_elem_size(int dtype);

/* AllreduceAlgos.cpp:22-34 */
void orc_chunkize(int64_t numel, size_t elem_size, int world, orc_chunk* out);

/* scalar codec */
uint16_t orc_f32_to_bf16(float x);    /* torch/headeronly/util/BFloat16.h:100-114 */
float orc_bf16_to_f32(uint16_t h);    /* bits << 16 */
uint16_t orc_f64_to_f16(double x);    /* (__fp16)scale, MetalKernels.mm:387,656 */
uint16_t orc_f32_to_f16(float x);
float orc_f16_to_f32(uint16_t h);

/* whole-buffer codec: ProcessGroupMCCL.cpp:131-132 (encode), :179-183 (decode) */
void orc_encode_bf16(uint16_t* dst, const float* src, size_t n, int threads);
void orc_decode_bf16(float* dst, const uint16_t* src, size_t n, int threads);

/* dst[i] = dst[i] (op) src[i] -- shaders.metal:196-229, 336-443 via
 * metal_reduce_op_view (MetalKernels.mm:628-640).  Returns 0, or -1 for an
 * unsupported op / dtype (the reference throws "Unsupported ReduceOp"). */
int orc_reduce(void* dst, const void* src, int dtype, size_t count, int op, int threads);

/* buf[i] *= s -- shaders.metal:233-332; constant per MetalKernels.mm:642-674
 * (scale_mode VIEW) or :365-405 (TENSOR). */
int orc_scale(void* buf, int dtype, size_t count, double scale, int scale_mode, int threads);

/* dst[i] = (dst[i] + src[i]) * s -- shaders.metal:447-551, MetalKernels.mm:408-458
 * (tensor-variant constant).  For bf16/f16 the sum is rounded before the multiply
 * (Metal evaluates bfloat4 + bfloat4 in bfloat). */
int orc_accumulate_scale(void* dst, const void* src, int dtype, size_t count, double scale,
                         int threads);

/* The scale constant, as the bit pattern the kernel receives. */
uint32_t orc_scale_constant_bits(int dtype, double scale, int scale_mode);

/* ProcessGroupMCCL.cpp:134-145: resolve the algorithm.  env_algo may be NULL
 * ("auto").  tree_below < 0 means "MCCL_TREE_BELOW unset" (262144). */
int orc_select_algo(const char* env_algo, int64_t tree_below, uint64_t wire_nbytes, int64_t numel,
                    int world);

/* Replay one allreduce for `world` virtual ranks over in-memory buffers,
 * following AllreduceAlgos.cpp message by message (each send is a snapshot
 * copy, each recv lands in that rank's recv scratch, each reduce is the binary
 * in-place kernel).  bufs[r] is rank r's tensor of `numel` elements of `dtype`;
 * on return it holds rank r's result.  Returns 0, -1 on a failed precondition
 * (numel < world for ring/butterfly: AllreduceAlgos.cpp:55,137). */
int orc_allreduce(int algo, int world, void* const* bufs, int dtype, int64_t numel, int op,
                  int threads);

/* ProcessGroupMCCL::allreduce (ProcessGroupMCCL.cpp:105-186) for `world`
 * virtual ranks holding fp32/f16/bf16 tensors: optional bf16 wire cast of fp32
 * inputs, algorithm selection, the schedule, cast back.  algo_out (nullable)
 * receives the algorithm actually used. */
int orc_pg_allreduce(int world, void* const* bufs, int dtype, int64_t numel, int op,
                     int wire_bf16, const char* env_algo, int64_t tree_below, int* algo_out,
                     int threads);

/* _reduce_scatter_base (ProcessGroupMCCL.cpp:331-390): ins[r] has world*chunk
 * elements, outs[r] receives chunk elements. */
int orc_reduce_scatter(int world, void* const* outs, const void* const* ins, int dtype,
                       int64_t chunk_numel, int op, int threads);

/* NOT the reference: fp32 accumulation with one final rounding ("fp32
 * accumulation and bf16 output"), kept as a labelled alternative. */
int orc_reduce_scatter_f32acc(int world, void* const* outs, const void* const* ins,
                              int64_t chunk_numel, int op, int threads);

/* _allgather_base (ProcessGroupMCCL.cpp:232-273): outs[r] = concat_p ins[p]. */
void orc_allgather(int world, void* const* outs, const void* const* ins, size_t chunk_nbytes);

/* The job the fused device kernel replaces, in reference-shaped passes, for
 * one owner's chunk: encode own fp32 chunk (PG.cpp:131), one binary bf16
 * reduce per peer in the given order (AllreduceAlgos.cpp:172-180), optional
 * view-variant scale (AllreduceAlgos.cpp:202), decode (PG.cpp:181).
 * own_last != 0 puts the own chunk last in the fold (ring order).
 * tmp must hold n bf16 values. */
void orc_wire_fold_chunk(float* out, const float* own, const uint16_t* const* peers, int npeers,
                         size_t n, int own_last, int do_scale, double scale, uint16_t* tmp,
                         uint16_t* wire_out, int threads);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
