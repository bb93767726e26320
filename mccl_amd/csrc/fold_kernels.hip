// fold_kernels.hip -- CDNA4 (gfx950) kernels of the reduce + wire-codec path.
//
// One kernel template, `fold`, covers every arithmetic launch of the path:
//   reference kernel (csrc/metal/shaders.metal)        fold configuration
//   accumulate_chunk_{f32,f16,bf16}      :196-229       k=2, PURE, SUM, out = in[0]
//   elementwise_{min,max,product}_*      :336-443       k=2, PURE, MIN/MAX/PRODUCT
//   scale_inplace_*                      :233-332       k=1, PURE, scale
//   accumulate_scale_*                   :447-551       k=2, PURE, SUM, scale
//   torch fp32->bf16 cast (ProcessGroupMCCL.cpp:131)    k=1, OWN_FIRST_F32, wire_out only
//   torch bf16->fp32 cast (ProcessGroupMCCL.cpp:181)    k=1, OUT_F32
//   N-1 binary launches + casts + scale of one schedule k=N, any io, one pass
//
// The work is HBM-bound streaming (0.1-0.25 flop/byte), so there is no MFMA
// and no LDS: every lane moves 16-byte packets (global_load/store_dwordx4),
// a wavefront covers 1 KiB of each stream per packet, all loads of an
// iteration are issued before the first dependent ALU op, and the arithmetic
// (bf16 round-to-nearest-even in integer ops) hides under the memory time.
// Pointers only need element alignment: gfx950 global accesses are
// alignment-agnostic and the compiler is told so through under-aligned types.
//
// Numerics: IEEE fp32 add/mul (no contraction, denormals kept), rounded to the
// arithmetic dtype after EVERY operation in MCCLX_ACC_STEP mode -- the
// accumulator is a float register that always holds a W-representable value,
// which is what makes one k-input pass bit-identical to k-1 binary kernels.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fold_launch.h"

namespace mcclx {
namespace {

constexpr int kBlock = 256;   // 4 wavefronts of 64
constexpr int kPack = 8;      // elements per packet: 16 B of bf16/f16, 32 B of fp32

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Under-aligned views: element alignment is all the kernels may assume.
struct __attribute__((packed, aligned(2))) Raw16 { u32x4 q; };
struct __attribute__((packed, aligned(4))) Raw32 { u32x4 lo; u32x4 hi; };

// Every operand lives in global memory (HBM or host memory mapped into the
// device).  Pointers that reach a kernel through a descriptor table are
// generic to the compiler; these casts let it emit global_load/global_store
// instead of flat accesses.
#define MCCLX_GLOBAL __attribute__((address_space(1)))
template <class T> __device__ __forceinline__ const MCCLX_GLOBAL T* gptr(const void* p) {
    return (const MCCLX_GLOBAL T*)p;
}
template <class T> __device__ __forceinline__ MCCLX_GLOBAL T* gptr(void* p) {
    return (MCCLX_GLOBAL T*)p;
}

// ---------------------------------------------------------------- rounding

// fp32 -> bf16 round-to-nearest-even, NaN -> 0x7FC0, result kept as the fp32
// whose low half is zero (torch/headeronly/util/BFloat16.h:100-114).
__device__ __forceinline__ uint32_t bf16_round_bits(float x) {
    uint32_t u = __float_as_uint(x);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    return ((u & 0x7FFFFFFFu) > 0x7F800000u) ? 0x7FC00000u : r;
}

template <int W> struct Num;  // arithmetic dtype traits

template <> struct Num<MCCLX_F32> {
    __device__ static __forceinline__ float rnd(float x) { return x; }
};
template <> struct Num<MCCLX_BF16> {
    __device__ static __forceinline__ float rnd(float x) {
        return __uint_as_float(bf16_round_bits(x));
    }
    __device__ static __forceinline__ uint32_t enc(float x) { return bf16_round_bits(x) >> 16; }
    __device__ static __forceinline__ float dec(uint32_t h) { return __uint_as_float(h << 16); }
};
template <> struct Num<MCCLX_F16> {
    // v_cvt_f16_f32 rounds to nearest even and keeps half denormals.
    __device__ static __forceinline__ float rnd(float x) { return (float)(_Float16)x; }
    __device__ static __forceinline__ uint32_t enc(float x) {
        _Float16 h = (_Float16)x;
        return (uint32_t) __builtin_bit_cast(uint16_t, h);
    }
    __device__ static __forceinline__ float dec(uint32_t h) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
    }
};

// The reference's element operators.  min/max follow the Metal definition
// "y if y < x else x" / "y if x < y else x" with x = accumulator (dst).
template <int OP> __device__ __forceinline__ float apply(float a, float b) {
    if constexpr (OP == MCCLX_SUM) return a + b;
    else if constexpr (OP == MCCLX_PRODUCT) return a * b;
    else if constexpr (OP == MCCLX_MIN) return (b < a) ? b : a;
    else return (a < b) ? b : a;
}

// ------------------------------------------------------------ configuration

template <int W_, int IO_, int K_, int TOPO_, int OP_, int ACC_>
struct Cfg {
    static constexpr int W = W_, IO = IO_, K = K_, TOPO = TOPO_, OP = OP_, ACC = ACC_;
    static constexpr bool kOutF32 = (IO != MCCLX_IO_PURE);
    __host__ __device__ static constexpr bool in_is_f32(int k) {
        return W == MCCLX_F32 || (IO == MCCLX_IO_OWN_FIRST_F32 && k == 0) ||
               (IO == MCCLX_IO_OWN_LAST_F32 && k == K - 1);
    }
    __host__ __device__ static constexpr int regs_per_pack() {
        int r = 0;
        for (int k = 0; k < K; ++k) r += in_is_f32(k) ? 8 : 4;
        return r;
    }
    // packets in flight per lane per iteration: keep raw loads near 64 registers
    static constexpr int U = (TOPO == MCCLX_TOPO_BINOMIAL) ? 1
                             : (64 / regs_per_pack() >= 4 ? 4 : 64 / regs_per_pack() >= 2 ? 2 : 1);
};

struct RawPack { u32x4 a; u32x4 b; };  // b only used by fp32 packets

template <class C, int k>
__device__ __forceinline__ RawPack load_raw(const void* p, uint64_t pack) {
    RawPack r;
    if constexpr (C::in_is_f32(k)) {
        const MCCLX_GLOBAL Raw32* q = gptr<Raw32>(static_cast<const float*>(p) + pack * kPack);
        r.a = q->lo; r.b = q->hi;
    } else {
        const MCCLX_GLOBAL Raw16* q = gptr<Raw16>(static_cast<const uint16_t*>(p) + pack * kPack);
        r.a = q->q; r.b = r.a;
    }
    return r;
}

// Operand k of one packet as 8 floats holding W-representable values.
template <class C, int k>
__device__ __forceinline__ void decode(const RawPack& r, float (&v)[kPack]) {
    if constexpr (C::in_is_f32(k)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[j] = Num<C::W>::rnd(__uint_as_float(r.a[j]));      // own fp32 -> wire value
            v[4 + j] = Num<C::W>::rnd(__uint_as_float(r.b[j]));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = Num<C::W>::dec(r.a[j] & 0xFFFFu);
            v[2 * j + 1] = Num<C::W>::dec(r.a[j] >> 16);
        }
    }
}

template <class C>
__device__ __forceinline__ float step(float a, float b) {
    float r = apply<C::OP>(a, b);
    if constexpr (C::ACC == MCCLX_ACC_STEP) r = Num<C::W>::rnd(r);
    return r;
}

template <class C>
__device__ __forceinline__ float finish(float acc, float scale, bool has_scale) {
    if (has_scale) {
        acc = acc * scale;
        if constexpr (C::ACC == MCCLX_ACC_STEP) acc = Num<C::W>::rnd(acc);
    }
    if constexpr (C::ACC != MCCLX_ACC_STEP) acc = Num<C::W>::rnd(acc);
    return acc;
}

template <class C, int k, int U>
__device__ __forceinline__ void load_all(const SegArgs& s, const uint64_t (&pk)[U],
                                         RawPack (&raw)[C::K][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) raw[k][u] = load_raw<C, k>(s.in[k], pk[u]);
    if constexpr (k + 1 < C::K) load_all<C, k + 1, U>(s, pk, raw);
}

template <class C, int k>
__device__ __forceinline__ void fold_from(const RawPack (&raw)[C::K], float (&acc)[kPack]) {
    float v[kPack];
    decode<C, k>(raw[k], v);
#pragma unroll
    for (int j = 0; j < kPack; ++j) acc[j] = step<C>(acc[j], v[j]);
    if constexpr (k + 1 < C::K) fold_from<C, k + 1>(raw, acc);
}

template <class C, int k>
__device__ __forceinline__ void decode_all(const RawPack (&raw)[C::K], float (&v)[C::K][kPack]) {
    decode<C, k>(raw[k], v[k]);
    if constexpr (k + 1 < C::K) decode_all<C, k + 1>(raw, v);
}

// Reduce one packet's K operands to acc[8].
template <class C>
__device__ __forceinline__ void combine(const RawPack (&raw)[C::K], float (&acc)[kPack]) {
    if constexpr (C::TOPO == MCCLX_TOPO_FOLD) {
        decode<C, 0>(raw[0], acc);
        if constexpr (C::K > 1) fold_from<C, 1>(raw, acc);
    } else {
        // allreduce_tree's reduce phase (AllreduceAlgos.cpp:100-114): at level
        // `mask` every surviving rank r (r % 2mask == 0) absorbs rank r+mask.
        float v[C::K][kPack];
        decode_all<C, 0>(raw, v);
#pragma unroll
        for (int mask = 1; mask < C::K; mask <<= 1)
#pragma unroll
            for (int r = 0; r + mask < C::K; r += 2 * mask)
#pragma unroll
                for (int j = 0; j < kPack; ++j) v[r][j] = step<C>(v[r][j], v[r + mask][j]);
#pragma unroll
        for (int j = 0; j < kPack; ++j) acc[j] = v[0][j];
    }
}

template <class C>
__device__ __forceinline__ void store_pack(const SegArgs& s, uint64_t pack, const float (&y)[kPack]) {
    if constexpr (C::W == MCCLX_F32 || C::kOutF32) {
        if (s.out) {
            u32x4 lo, hi;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lo[j] = __float_as_uint(y[j]);
                hi[j] = __float_as_uint(y[4 + j]);
            }
            MCCLX_GLOBAL Raw32* o = gptr<Raw32>(static_cast<float*>(s.out) + pack * kPack);
            o->lo = lo;
            o->hi = hi;
        }
    }
    if constexpr (C::W != MCCLX_F32) {
        void* w = C::kOutF32 ? s.wire_out : (s.out ? s.out : s.wire_out);
        if (w) {
            u32x4 t;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                t[j] = Num<C::W>::enc(y[2 * j]) | (Num<C::W>::enc(y[2 * j + 1]) << 16);
            gptr<Raw16>(static_cast<uint16_t*>(w) + pack * kPack)->q = t;
            if constexpr (!C::kOutF32)
                if (s.out && s.wire_out)  // PURE with both outputs set
                    gptr<Raw16>(static_cast<uint16_t*>(s.wire_out) + pack * kPack)->q = t;
        }
    }
}

// One element through the same arithmetic (segment tails).
template <class C, int k>
__device__ __forceinline__ float load_elem(const SegArgs& s, uint64_t i) {
    if constexpr (C::in_is_f32(k))
        return Num<C::W>::rnd(gptr<float>(s.in[k])[i]);
    else
        return Num<C::W>::dec(gptr<uint16_t>(s.in[k])[i]);
}
template <class C, int k>
__device__ __forceinline__ void load_elems(const SegArgs& s, uint64_t i, float (&v)[C::K]) {
    v[k] = load_elem<C, k>(s, i);
    if constexpr (k + 1 < C::K) load_elems<C, k + 1>(s, i, v);
}
template <class C>
__device__ __forceinline__ void fold_elem(const SegArgs& s, uint64_t i, float scale, bool has_scale) {
    float v[C::K];
    load_elems<C, 0>(s, i, v);
    if constexpr (C::TOPO == MCCLX_TOPO_FOLD) {
#pragma unroll
        for (int k = 1; k < C::K; ++k) v[0] = step<C>(v[0], v[k]);
    } else {
#pragma unroll
        for (int mask = 1; mask < C::K; mask <<= 1)
#pragma unroll
            for (int r = 0; r + mask < C::K; r += 2 * mask) v[r] = step<C>(v[r], v[r + mask]);
    }
    float y = finish<C>(v[0], scale, has_scale);
    if constexpr (C::W == MCCLX_F32 || C::kOutF32) {
        if (s.out) gptr<float>(s.out)[i] = y;
    }
    if constexpr (C::W != MCCLX_F32) {
        uint16_t h = (uint16_t)Num<C::W>::enc(y);
        if constexpr (C::kOutF32) {
            if (s.wire_out) gptr<uint16_t>(s.wire_out)[i] = h;
        } else {
            if (s.out) gptr<uint16_t>(s.out)[i] = h;
            if (s.wire_out) gptr<uint16_t>(s.wire_out)[i] = h;
        }
    }
}

// U packets per lane: all loads first, then arithmetic, then stores.
template <class C, int U>
__device__ __forceinline__ void fold_packs(const SegArgs& s, const uint64_t (&pk)[U], float scale,
                                           bool has_scale) {
    RawPack raw[C::K][U];
    load_all<C, 0, U>(s, pk, raw);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        RawPack col[C::K];
#pragma unroll
        for (int k = 0; k < C::K; ++k) col[k] = raw[k][u];
        float acc[kPack];
        combine<C>(col, acc);
#pragma unroll
        for (int j = 0; j < kPack; ++j) acc[j] = finish<C>(acc[j], scale, has_scale);
        store_pack<C>(s, pk[u], acc);
    }
}

// The block's share of one segment: packets [first, P) in strides of `stride`
// packets, plus the sub-packet tail when `do_tail`.
template <class C>
__device__ __forceinline__ void fold_segment(const SegArgs& s, float scale, bool has_scale,
                                             uint64_t first, uint64_t stride, bool do_tail) {
    constexpr int U = C::U;
    const uint64_t P = s.count / kPack;
    const uint32_t tid = threadIdx.x;
    for (uint64_t base = first; base < P; base += stride) {
        if (base + (uint64_t)U * kBlock <= P) {
            uint64_t pk[U];
#pragma unroll
            for (int u = 0; u < U; ++u) pk[u] = base + (uint64_t)u * kBlock + tid;
            fold_packs<C, U>(s, pk, scale, has_scale);
        } else {
            for (uint64_t p = base + tid; p < P && p < base + (uint64_t)U * kBlock; p += kBlock) {
                uint64_t one[1] = {p};
                fold_packs<C, 1>(s, one, scale, has_scale);
            }
        }
    }
    if (do_tail) {
        uint64_t i = P * kPack + tid;
        if (i < s.count) fold_elem<C>(s, i, scale, has_scale);
    }
}

}  // namespace

// ------------------------------------------------------------------ kernels

// Up to kFewSegs segments passed by value in the kernel arguments: blockIdx.y
// picks the segment, blockIdx.x strides over its packets.
template <class C>
__global__ void __launch_bounds__(kBlock) fold_few_kernel(FewArgs a) {
    const SegArgs& s = a.seg[blockIdx.y];
    const uint64_t span = (uint64_t)C::U * kBlock;
    fold_segment<C>(s, a.scale, a.has_scale != 0, (uint64_t)blockIdx.x * span,
                    (uint64_t)gridDim.x * span, blockIdx.x == 0);
}

// Persistent blocks over a descriptor table in device memory: work item w is
// tile (w - first_item[seg]) of segment seg; a block takes items
// blockIdx.x, blockIdx.x + gridDim.x, ...  The loop bound is fixed at launch,
// so every wave exits.
template <class C>
__global__ void __launch_bounds__(kBlock) fold_table_kernel(TableArgs a) {
    const uint64_t span = (uint64_t)C::U * kBlock;
    for (uint64_t w = blockIdx.x; w < a.total_items; w += gridDim.x) {
        uint32_t seg;
        uint64_t tile;
        if (a.uniform_items) {
            seg = (uint32_t)(w / a.uniform_items);
            tile = w - (uint64_t)seg * a.uniform_items;
        } else {
            uint32_t lo = 0, hi = a.nseg;  // first_item[lo] <= w < first_item[hi]
            while (hi - lo > 1) {
                uint32_t mid = (lo + hi) >> 1;
                if (a.first_item[mid] <= w) lo = mid; else hi = mid;
            }
            seg = lo;
            tile = w - a.first_item[seg];
        }
        // w depends on blockIdx only, so the segment is the same for every lane:
        // say so, and its descriptor is fetched with scalar loads
        seg = __builtin_amdgcn_readfirstlane(seg);
        SegArgs s = a.segs[seg];
        // one tile: packets [tile*span, tile*span + span); tile 0 also owns the tail
        fold_segment<C>(s, a.scale, a.has_scale != 0, tile * span, ~0ull >> 1, tile == 0);
    }
}

// ----------------------------------------------------------------- dispatch

template <class C>
static hipError_t launch_cfg(hipStream_t st, const LaunchParams& lp) {
    const uint64_t span = (uint64_t)C::U * kBlock * kPack;  // elements per block iteration
    if (lp.table) {
        TableArgs a = *lp.table;
        uint32_t grid = (uint32_t)(a.total_items < lp.max_blocks ? a.total_items : lp.max_blocks);
        if (grid == 0) return hipSuccess;
        fold_table_kernel<C><<<dim3(grid), dim3(kBlock), 0, st>>>(a);
    } else {
        FewArgs a = *lp.few;
        uint64_t maxc = 0;
        for (int i = 0; i < a.nseg; ++i) maxc = a.seg[i].count > maxc ? a.seg[i].count : maxc;
        if (maxc == 0) return hipSuccess;
        uint64_t gx = (maxc + span - 1) / span;
        uint64_t cap = lp.max_blocks / (uint32_t)a.nseg;
        if (cap < 1) cap = 1;
        if (gx > cap) gx = cap;
        fold_few_kernel<C><<<dim3((uint32_t)gx, (uint32_t)a.nseg), dim3(kBlock), 0, st>>>(a);
    }
    return hipGetLastError();
}

uint32_t items_for(const PlanKey& k, uint64_t count) {
    // must mirror Cfg::U for the plan; computed on the host for table building
    uint64_t span = (uint64_t)plan_unroll(k) * kBlock * kPack;
    uint64_t n = (count + span - 1) / span;
    return (uint32_t)(n ? n : (count ? 1 : 0));
}

int plan_unroll(const PlanKey& key) {
    if (key.topo == MCCLX_TOPO_BINOMIAL) return 1;
    int regs = 0;
    for (int k = 0; k < key.k; ++k) {
        bool f32 = key.dtype == MCCLX_F32 || (key.io == MCCLX_IO_OWN_FIRST_F32 && k == 0) ||
                   (key.io == MCCLX_IO_OWN_LAST_F32 && k == key.k - 1);
        regs += f32 ? 8 : 4;
    }
    int q = 64 / regs;
    return q >= 4 ? 4 : q >= 2 ? 2 : 1;
}

#define MCCLX_K_CASES(W, IO, TOPO, OP, ACC)                                             \
    switch (key.k) {                                                                    \
        case 1: return launch_cfg<Cfg<W, IO, 1, MCCLX_TOPO_FOLD, OP, ACC>>(st, lp);     \
        case 2: return launch_cfg<Cfg<W, IO, 2, MCCLX_TOPO_FOLD, OP, ACC>>(st, lp);     \
        case 3: return launch_cfg<Cfg<W, IO, 3, MCCLX_TOPO_FOLD, OP, ACC>>(st, lp);     \
        case 4: return launch_cfg<Cfg<W, IO, 4, TOPO, OP, ACC>>(st, lp);                \
        case 5: return launch_cfg<Cfg<W, IO, 5, TOPO, OP, ACC>>(st, lp);                \
        case 6: return launch_cfg<Cfg<W, IO, 6, TOPO, OP, ACC>>(st, lp);                \
        case 7: return launch_cfg<Cfg<W, IO, 7, TOPO, OP, ACC>>(st, lp);                \
        case 8: return launch_cfg<Cfg<W, IO, 8, TOPO, OP, ACC>>(st, lp);                \
        default: return hipErrorInvalidValue;                                           \
    }

#define MCCLX_TOPO_CASES(W, IO, OP, ACC)                                                \
    if (key.topo == MCCLX_TOPO_BINOMIAL && key.k >= 4) {                                \
        MCCLX_K_CASES(W, IO, MCCLX_TOPO_BINOMIAL, OP, ACC)                              \
    } else {                                                                            \
        MCCLX_K_CASES(W, IO, MCCLX_TOPO_FOLD, OP, ACC)                                  \
    }

// k <= 2 only (the reference's binary kernels): MIN / MAX / PRODUCT and fp16.
#define MCCLX_BINARY_CASES(W, OP)                                                                  \
    switch (key.k) {                                                                               \
        case 1: return launch_cfg<Cfg<W, MCCLX_IO_PURE, 1, MCCLX_TOPO_FOLD, OP, MCCLX_ACC_STEP>>(st, lp); \
        case 2: return launch_cfg<Cfg<W, MCCLX_IO_PURE, 2, MCCLX_TOPO_FOLD, OP, MCCLX_ACC_STEP>>(st, lp); \
        default: return hipErrorInvalidValue;                                                      \
    }

#define MCCLX_OP_BINARY(W)                                              \
    switch (key.op) {                                                   \
        case MCCLX_PRODUCT: MCCLX_BINARY_CASES(W, MCCLX_PRODUCT)        \
        case MCCLX_MIN: MCCLX_BINARY_CASES(W, MCCLX_MIN)                \
        case MCCLX_MAX: MCCLX_BINARY_CASES(W, MCCLX_MAX)                \
        default: return hipErrorInvalidValue;                           \
    }

hipError_t launch_fold(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    if (key.op != MCCLX_SUM) {
        if (key.io != MCCLX_IO_PURE || key.acc != MCCLX_ACC_STEP) return hipErrorInvalidValue;
        switch (key.dtype) {
            case MCCLX_F32: MCCLX_OP_BINARY(MCCLX_F32)
            case MCCLX_F16: MCCLX_OP_BINARY(MCCLX_F16)
            case MCCLX_BF16: MCCLX_OP_BINARY(MCCLX_BF16)
            default: return hipErrorInvalidValue;
        }
    }
    if (key.dtype == MCCLX_F32) {
        if (key.io != MCCLX_IO_PURE) return hipErrorInvalidValue;
        MCCLX_TOPO_CASES(MCCLX_F32, MCCLX_IO_PURE, MCCLX_SUM, MCCLX_ACC_STEP)
    }
    if (key.dtype == MCCLX_F16) {
        if (key.io != MCCLX_IO_PURE || key.acc != MCCLX_ACC_STEP) return hipErrorInvalidValue;
        MCCLX_BINARY_CASES(MCCLX_F16, MCCLX_SUM)
    }
    if (key.dtype != MCCLX_BF16) return hipErrorInvalidValue;
#define MCCLX_IO_CASES(ACC)                                                                        \
    switch (key.io) {                                                                              \
        case MCCLX_IO_PURE: MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_PURE, MCCLX_SUM, ACC)            \
        case MCCLX_IO_OUT_F32: MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_OUT_F32, MCCLX_SUM, ACC)      \
        case MCCLX_IO_OWN_FIRST_F32:                                                               \
            MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_OWN_FIRST_F32, MCCLX_SUM, ACC)                   \
        case MCCLX_IO_OWN_LAST_F32:                                                                \
            MCCLX_K_CASES(MCCLX_BF16, MCCLX_IO_OWN_LAST_F32, MCCLX_TOPO_FOLD, MCCLX_SUM, ACC)      \
        default: return hipErrorInvalidValue;                                                      \
    }
    if (key.acc == MCCLX_ACC_STEP) {
        MCCLX_IO_CASES(MCCLX_ACC_STEP)
    } else {
        MCCLX_IO_CASES(MCCLX_ACC_F32)
    }
    return hipErrorInvalidValue;
}

}  // namespace mcclx
