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
// and no LDS.  Consecutive lanes take consecutive packets of E elements, so one
// wavefront instruction covers one contiguous span of every stream: E = 4 when
// any stream is fp32 (fp32: global_load/store_dwordx4 = 1 KiB per wavefront,
// 16-bit peers: dwordx2 = 512 B), E = 8 when every stream is 16-bit (dwordx4).
// All loads of an iteration are issued before the first dependent ALU op and
// the arithmetic (bf16 round-to-nearest-even) hides under the memory time.
// Accesses carry the non-temporal hint: every byte is touched exactly once.
// Pointers only need element alignment (gfx950 global accesses are
// alignment-agnostic and the compiler is told so through under-aligned
// types); a scalar head peel moves the packet grid onto a 128-byte boundary of
// the output, which also aligns the inputs whenever all buffers share the
// chunk's element offset.
//
// Numerics: IEEE fp32 add/mul (no contraction, denormals kept), rounded to the
// arithmetic dtype after EVERY operation in MCCLX_ACC_STEP mode -- the
// accumulator is a float register that always holds a W-representable value,
// which is what makes one k-input pass bit-identical to k-1 binary kernels.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "fold_launch.h"

namespace mcclx {
namespace {

// Launch shapes, each measured on MI355X.
constexpr int kBlock = 512;  // threads per block of folds that mix fp32 and 16-bit streams, and of one-operand passes
// Folds whose streams all have one element size -- all 16-bit (16 bytes per lane
// and operand) or all fp32 -- run one-wavefront blocks with one packet per lane:
// a 512-lane block keeps its wave slots until the last of its loads is back,
// 64-lane blocks turn them over eight times as often (two to eight 16-bit
// operands of 512 MiB: +5...9 %, fp32 operands: +3...4 %; launches of a few MB
// are level; fp32 operands encoded in registers, MCCLX_IO_ALL_F32: +7 % on
// 256 MiB tensors, +1.5 % on 25 MiB ones).
constexpr int kWideBlock = 64;
constexpr int kWideU = 1;
constexpr int kWideMinK = 2;   // all-16-bit folds of this many operands or more take the one-wavefront shape
constexpr int kF32Block = 64;
constexpr int kAllF32Block = 64;

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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// Under-aligned views: element alignment is all the kernels may assume.
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
// Loads and stores of one packet through the under-aligned pointer types
// (macros, so the typedef's alignment stays attached to the access).
// (the hold form with ordinary stores: 14.85 us for a launch the non-temporal ones run in 13.1 us)
#define MCCLX_LDG(p) __builtin_nontemporal_load(p)
#define MCCLX_STG(p, v) __builtin_nontemporal_store((v), (p))

// ---------------------------------------------------------------- rounding

// fp32 -> bf16 round-to-nearest-even, NaN -> 0x7FC0, result kept as the fp32
// whose low half is zero (torch/headeronly/util/BFloat16.h:100-114).
__device__ __forceinline__ uint32_t bf16_round_bits(float x) {
    uint32_t r = (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x) << 16;  // v_cvt_pk_bf16_f32
    return (x != x) ? 0x7FC00000u : r;
}

template <int W> struct Num;  // arithmetic dtype traits

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Besides the scalar rnd (round to W, NaN made canonical where W defines one),
// every dtype has the array form the packet path uses between the operands of
// a fold: round_mid rounds E values to W and only guarantees that a NaN stays
// a NaN -- which NaN is decided once, by canon, after the last operation.  That
// is the same result as canonicalising after every step (a NaN operand makes a
// sum or a product NaN whatever its payload; min and max either keep it to the
// end or drop it), for two instructions per element and step less.
template <> struct Num<MCCLX_F32> {
    __device__ static __forceinline__ float rnd(float x) { return x; }
    __device__ static __forceinline__ float scaled(float x, float s) { return x * s; }
    template <int E> __device__ static __forceinline__ void round_mid(float (&)[E]) {}
    template <int E> __device__ static __forceinline__ void canon(float (&)[E]) {}
};
template <> struct Num<MCCLX_BF16> {
    __device__ static __forceinline__ float rnd(float x) {
        return __uint_as_float(bf16_round_bits(x));
    }
    __device__ static __forceinline__ uint32_t enc(float x) { return bf16_round_bits(x) >> 16; }
    __device__ static __forceinline__ float dec(uint32_t h) { return __uint_as_float(h << 16); }
    __device__ static __forceinline__ float scaled(float x, float s) { return x * s; }
    // two values per v_cvt_pk_bf16_f32; a NaN whose quiet bit is set (every NaN an
    // add, a multiply or a decoded bf16 operand can hand over) converts to a NaN
    template <int E> __device__ static __forceinline__ void round_mid(float (&x)[E]) {
#pragma unroll
        for (int j = 0; j < E; j += 2) {
            const uint32_t u = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{x[j], x[j + 1]}, bf16x2));
            x[j] = __uint_as_float(u << 16);
            x[j + 1] = __uint_as_float(u & 0xFFFF0000u);
        }
    }
    template <int E> __device__ static __forceinline__ void canon(float (&x)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) x[j] = (x[j] != x[j]) ? __uint_as_float(0x7FC00000u) : x[j];
    }
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
    // x and the scale constant are both half values, so the half product IS the rounded
    // fp32 product (two 11-bit significands multiply exactly in fp32).  Written as a half
    // multiply on purpose: "round(x * s)" in fp32 is selected as a mixed-precision
    // fma(s, x, +0), which turns a product of -0 into +0.
    __device__ static __forceinline__ float scaled(float x, float s) {
        return (float)((_Float16)x * (_Float16)s);
    }
    template <int E> __device__ static __forceinline__ void round_mid(float (&x)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) x[j] = rnd(x[j]);
    }
    template <int E> __device__ static __forceinline__ void canon(float (&)[E]) {}
};

// The reference's element operators.  min/max follow the Metal definition
// "y if y < x else x" / "y if x < y else x" with x = dst, y = src: dst is kept on
// a tie (+0 against -0) and when either operand is NaN.  `a` is the accumulator,
// `b` the next operand; by default the accumulator is dst, the *_ACC_SRC forms
// (the ring's roles, AllreduceAlgos.cpp:72-74) make the next operand dst.
template <int OP> __device__ __forceinline__ float apply(float a, float b) {
    if constexpr (OP == MCCLX_SUM) return a + b;
    else if constexpr (OP == MCCLX_PRODUCT) return a * b;
    else if constexpr (OP == MCCLX_MIN) return (b < a) ? b : a;
    else if constexpr (OP == MCCLX_MAX) return (a < b) ? b : a;
    else if constexpr (OP == MCCLX_MIN_ACC_SRC) return (a < b) ? a : b;
    else return (b < a) ? a : b;  // MCCLX_MAX_ACC_SRC
}

// ------------------------------------------------------------ configuration

template <int W_, int IO_, int K_, int TOPO_, int OP_, int ACC_>
struct Cfg {
    static constexpr int W = W_, IO = IO_, K = K_, TOPO = TOPO_, OP = OP_, ACC = ACC_;
    static constexpr bool kOutF32 = (IO != MCCLX_IO_PURE);
    // elements per packet: 4 as soon as one stream (operand or output) is fp32
    static constexpr int E = (W == MCCLX_F32 || IO != MCCLX_IO_PURE) ? 4 : 8;
    __host__ __device__ static constexpr bool in_is_f32(int k) {
        return W == MCCLX_F32 || IO == MCCLX_IO_ALL_F32 || (IO == MCCLX_IO_OWN_FIRST_F32 && k == 0) ||
               (IO == MCCLX_IO_OWN_LAST_F32 && k == K - 1);
    }
    // Packets per lane per iteration.  Measured on MI355X (one block per tile,
    // no grid-stride looping): one packet per lane streams fastest for folds with
    // an fp32 stream; all-16-bit plans and the one-input codec passes (encode,
    // decode), whose lanes move few bytes, gain 4-12 % from two.
    static constexpr bool kWide = (E == 8 && K >= kWideMinK);
    static constexpr int U = kWide ? kWideU
                             : (TOPO == MCCLX_TOPO_BINOMIAL) ? 1
                             : ((E == 8 || (K == 1 && IO != MCCLX_IO_PURE)) ? 2 : 1);
    static constexpr bool kDecode = (K == 1 && IO == MCCLX_IO_OUT_F32);  // bf16 -> fp32 cast: +3 % at 64
    static constexpr int BLOCK = kWide ? kWideBlock
                                 : ((W == MCCLX_F32 && K >= 2) || kDecode) ? kF32Block
                                 : (IO == MCCLX_IO_ALL_F32 && K >= 2) ? kAllF32Block : kBlock;  // threads per block
};

typedef u32x4 RawPack;  // one packet of one operand: 16 B, or 8 B in .xy (16-bit operand, E = 4)

template <class C, int k>
__device__ __forceinline__ RawPack load_raw(const void* p, uint32_t pack) {
    if constexpr (C::in_is_f32(k)) {
        return MCCLX_LDG(gptr<u32x4_a4>(static_cast<const float*>(p) + pack * C::E));
    } else if constexpr (C::E == 8) {
        return MCCLX_LDG(gptr<u32x4_a2>(static_cast<const uint16_t*>(p) + pack * C::E));
    } else {
        u32x2 h = MCCLX_LDG(gptr<u32x2_a2>(static_cast<const uint16_t*>(p) + pack * C::E));
        return u32x4{h.x, h.y, 0u, 0u};
    }
}

// Operand k of one packet as E floats holding W-representable values.
template <class C, int k>
__device__ __forceinline__ void decode(const RawPack& r, float (&v)[C::E]) {
    if constexpr (C::in_is_f32(k)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = Num<C::W>::rnd(__uint_as_float(r[j]));  // own fp32 -> wire value
    } else {
#pragma unroll
        for (int j = 0; j < C::E / 2; ++j) {
            v[2 * j] = Num<C::W>::dec(r[j] & 0xFFFFu);
            v[2 * j + 1] = Num<C::W>::dec(r[j] >> 16);
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
        acc = Num<C::W>::scaled(acc, scale);
        if constexpr (C::ACC == MCCLX_ACC_STEP) acc = Num<C::W>::rnd(acc);
    }
    if constexpr (C::ACC != MCCLX_ACC_STEP) acc = Num<C::W>::rnd(acc);
    return acc;
}

template <class C, int k, int U>
__device__ __forceinline__ void load_all(const SegArgs& s, const uint32_t (&pk)[U],
                                         RawPack (&raw)[C::K][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) raw[k][u] = load_raw<C, k>(s.in[k], pk[u]);
    if constexpr (k + 1 < C::K) load_all<C, k + 1, U>(s, pk, raw);
}

// acc = acc (op) v for one packet, rounded to W in STEP mode (NaNs not yet canonical).
template <class C>
__device__ __forceinline__ void step_pack(float (&acc)[C::E], const float (&v)[C::E]) {
#pragma unroll
    for (int j = 0; j < C::E; ++j) acc[j] = apply<C::OP>(acc[j], v[j]);
    if constexpr (C::ACC == MCCLX_ACC_STEP) Num<C::W>::template round_mid<C::E>(acc);
}

// What follows the last operand: the scale, the final rounding of the fp32
// accumulator mode, and -- if the packet went through any rounding -- the one
// canonicalisation of NaNs (a fold of one operand without scale moves bits).
template <class C>
__device__ __forceinline__ void finish_pack(float (&acc)[C::E], float scale, bool has_scale) {
    if (has_scale) {
#pragma unroll
        for (int j = 0; j < C::E; ++j) acc[j] = Num<C::W>::scaled(acc[j], scale);
        if constexpr (C::ACC == MCCLX_ACC_STEP) Num<C::W>::template round_mid<C::E>(acc);
    }
    if constexpr (C::ACC != MCCLX_ACC_STEP) Num<C::W>::template round_mid<C::E>(acc);
    if constexpr (C::K > 1 || C::ACC != MCCLX_ACC_STEP) {
        Num<C::W>::template canon<C::E>(acc);
    } else {
        if (has_scale) Num<C::W>::template canon<C::E>(acc);
    }
}

template <class C, int k>
__device__ __forceinline__ void fold_from(const RawPack (&raw)[C::K], float (&acc)[C::E]) {
    float v[C::E];
    decode<C, k>(raw[k], v);
    step_pack<C>(acc, v);
    if constexpr (k + 1 < C::K) fold_from<C, k + 1>(raw, acc);
}

template <class C, int k>
__device__ __forceinline__ void decode_all(const RawPack (&raw)[C::K], float (&v)[C::K][C::E]) {
    decode<C, k>(raw[k], v[k]);
    if constexpr (k + 1 < C::K) decode_all<C, k + 1>(raw, v);
}

// Reduce one packet's K operands to acc[E].
template <class C>
__device__ __forceinline__ void combine(const RawPack (&raw)[C::K], float (&acc)[C::E]) {
    if constexpr (C::TOPO == MCCLX_TOPO_FOLD) {
        decode<C, 0>(raw[0], acc);
        if constexpr (C::K > 1) fold_from<C, 1>(raw, acc);
    } else {
        // allreduce_tree's reduce phase (AllreduceAlgos.cpp:100-114): at level
        // `mask` every surviving rank r (r % 2mask == 0) absorbs rank r+mask.
        float v[C::K][C::E];
        decode_all<C, 0>(raw, v);
#pragma unroll
        for (int mask = 1; mask < C::K; mask <<= 1)
#pragma unroll
            for (int r = 0; r + mask < C::K; r += 2 * mask) step_pack<C>(v[r], v[r + mask]);
#pragma unroll
        for (int j = 0; j < C::E; ++j) acc[j] = v[0][j];
    }
}

template <class C>
__device__ __forceinline__ void store16(void* base, uint32_t pack, const float (&y)[C::E]) {
    using V = Num<C::W>;
    if constexpr (C::E == 8) {
        u32x4 t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = V::enc(y[2 * j]) | (V::enc(y[2 * j + 1]) << 16);
        MCCLX_STG(gptr<u32x4_a2>(static_cast<uint16_t*>(base) + pack * C::E), t);
    } else {
        u32x2 t;
#pragma unroll
        for (int j = 0; j < 2; ++j) t[j] = V::enc(y[2 * j]) | (V::enc(y[2 * j + 1]) << 16);
        MCCLX_STG(gptr<u32x2_a2>(static_cast<uint16_t*>(base) + pack * C::E), t);
    }
}

// `has_out` / `has_wire`: which outputs the segment names (the pointers in `s` have
// been advanced to the tile, so they no longer tell).  `fan` (fan-out kernels): the
// result also goes to in[K .. K+fan-1], in the form `out` has.
template <class C, bool FAN = false>
__device__ __forceinline__ void store_pack(const SegArgs& s, bool has_out, bool has_wire, uint32_t pack,
                                           const float (&y)[C::E], int fan = 0) {
    if constexpr (C::W == MCCLX_F32 || C::kOutF32) {
        u32x4 t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = __float_as_uint(y[j]);
        if (has_out) MCCLX_STG(gptr<u32x4_a4>(static_cast<float*>(s.out) + pack * C::E), t);
        if constexpr (FAN) {
#pragma unroll
            for (int f = 0; f < MCCLX_MAX_INPUTS - C::K; ++f)
                if (f < fan)
                    MCCLX_STG(gptr<u32x4_a4>(static_cast<float*>(const_cast<void*>(s.in[C::K + f])) + pack * C::E), t);
        }
    }
    if constexpr (C::W != MCCLX_F32) {
        if constexpr (C::kOutF32) {
            if (has_wire) store16<C>(s.wire_out, pack, y);
        } else {
            if (has_out) store16<C>(s.out, pack, y);
            if (has_wire) store16<C>(s.wire_out, pack, y);
            if constexpr (FAN) {
#pragma unroll
                for (int f = 0; f < MCCLX_MAX_INPUTS - C::K; ++f)
                    if (f < fan) store16<C>(const_cast<void*>(s.in[C::K + f]), pack, y);
            }
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
template <class C, bool FAN = false>
__device__ __forceinline__ void fold_elem(const SegArgs& s, uint64_t i, float scale, bool has_scale, int fan = 0) {
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
        if constexpr (FAN) {
#pragma unroll
            for (int f = 0; f < MCCLX_MAX_INPUTS - C::K; ++f)
                if (f < fan) gptr<float>(const_cast<void*>(s.in[C::K + f]))[i] = y;
        }
    }
    if constexpr (C::W != MCCLX_F32) {
        uint16_t h = (uint16_t)Num<C::W>::enc(y);
        if constexpr (C::kOutF32) {
            if (s.wire_out) gptr<uint16_t>(s.wire_out)[i] = h;
        } else {
            if (s.out) gptr<uint16_t>(s.out)[i] = h;
            if (s.wire_out) gptr<uint16_t>(s.wire_out)[i] = h;
            if constexpr (FAN) {
#pragma unroll
                for (int f = 0; f < MCCLX_MAX_INPUTS - C::K; ++f)
                    if (f < fan) gptr<uint16_t>(const_cast<void*>(s.in[C::K + f]))[i] = h;
            }
        }
    }
}

// U packets per lane: all loads first, then arithmetic, then stores.  `s` points
// at the tile's first packet; pk[] are packet indices inside the tile, so every
// address is a uniform 64-bit base plus a 32-bit lane offset.
template <class C, int U, bool FAN = false>
__device__ __forceinline__ void fold_packs(const SegArgs& s, bool has_out, bool has_wire, const uint32_t (&pk)[U],
                                           float scale, bool has_scale, int fan = 0) {
    RawPack raw[C::K][U];
    load_all<C, 0, U>(s, pk, raw);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        RawPack col[C::K];
#pragma unroll
        for (int k = 0; k < C::K; ++k) col[k] = raw[k][u];
        float acc[C::E];
        combine<C>(col, acc);
        finish_pack<C>(acc, scale, has_scale);
        store_pack<C, FAN>(s, has_out, has_wire, pk[u], acc, fan);
    }
}

// Elements in front of the packet grid: up to the 128-byte boundary of the
// buffer the widest stores go to.
template <class C>
__device__ __forceinline__ uint32_t head_elems(const SegArgs& s) {
    const bool wide_out = (C::W == MCCLX_F32 || C::kOutF32) && s.out;
    const uint32_t a = (uint32_t)reinterpret_cast<uintptr_t>(s.out ? s.out : s.wire_out);
    const uint32_t mis = a & 127u;
    const uint32_t h = mis ? (128u - mis) >> (wide_out ? 2 : 1) : 0u;
    return s.count < h ? (uint32_t)s.count : h;
}

// Every pointer of the segment moved `elems` elements on (null outputs become
// garbage: the caller keeps their presence in flags).
template <class C, bool FAN = false>
__device__ __forceinline__ SegArgs advanced(const SegArgs& s, uint64_t elems) {
    SegArgs t;
    const uint64_t b2 = elems * 2, b4 = elems * 4;
    const bool out_f32 = (C::W == MCCLX_F32 || C::kOutF32);
    t.out = static_cast<char*>(s.out) + (out_f32 ? b4 : b2);
    t.wire_out = static_cast<char*>(s.wire_out) + b2;
#pragma unroll
    for (int k = 0; k < MCCLX_MAX_INPUTS; ++k) {
        if (k < C::K)
            t.in[k] = static_cast<const char*>(s.in[k]) + (C::in_is_f32(k) ? b4 : b2);
        else if constexpr (FAN)
            t.in[k] = static_cast<const char*>(s.in[k]) + (out_f32 ? b4 : b2);  // a further destination
        else
            t.in[k] = nullptr;
    }
    t.count = 0;
    return t;
}

// One tile of a segment: after the head peel, the U * BLOCK packets from packet
// `first` on (fewer at the segment's end); the block with `do_edges` also runs
// the head and the sub-packet tail, one element per lane.  The path to the first
// load is kept short -- a block lives for about 2 us and eight waves per SIMD
// share one scalar unit, so every scalar instruction in front of the loads is
// paid eight times over.
template <class C, bool FAN = false>
__device__ __forceinline__ void fold_tile(const SegArgs& s, float scale, bool has_scale, uint64_t first,
                                          bool do_edges, int fan = 0) {
    constexpr int U = C::U;
    const uint32_t tid = threadIdx.x;
    constexpr int kB = C::BLOCK;
    const uint32_t head = head_elems<C>(s);  // < 64 <= kB
    const uint64_t P = (s.count - head) / C::E;
    const bool has_out = s.out != nullptr, has_wire = s.wire_out != nullptr;
    if (first < P) {
        const SegArgs t = advanced<C, FAN>(s, head + first * C::E);
        const uint64_t left = P - first;
        if (left >= (uint64_t)U * kB) {
            uint32_t pk[U];
#pragma unroll
            for (int u = 0; u < U; ++u) pk[u] = (uint32_t)u * kB + tid;
            fold_packs<C, U, FAN>(t, has_out, has_wire, pk, scale, has_scale, fan);
        } else {
            for (uint32_t p = tid; p < (uint32_t)left; p += kB) {
                uint32_t one[1] = {p};
                fold_packs<C, 1, FAN>(t, has_out, has_wire, one, scale, has_scale, fan);
            }
        }
    }
    if (do_edges) {
        if (tid < head) fold_elem<C, FAN>(s, tid, scale, has_scale, fan);
        const uint64_t i = head + P * C::E + tid;  // fewer than E <= 8 elements remain
        if (i < s.count) fold_elem<C, FAN>(s, i, scale, has_scale, fan);
    }
}

}  // namespace

// ------------------------------------------------------------------ kernels

// Everything a block needs from the kernel arguments, fetched with ONE batch of
// scalar loads and one wait.  Left to itself the compiler fetches the fields
// where they are first used -- three dependent fetch-and-wait rounds before the
// block can issue its first data load, 0.2-0.3 us per block on a kernel whose
// blocks live for 2 us.  The empty asm makes every field live at one point.
// Only the K operand pointers the plan reads are fetched: scalar registers are
// what decides how many blocks a CU holds (see fold_few_kernel).
template <int K>
__device__ __forceinline__ void fetch_together(SegArgs& s, float& scale, int32_t& has_scale, uint32_t& grid) {
    asm volatile("" : "+s"(s.out), "+s"(s.wire_out), "+s"(s.count), "+s"(scale), "+s"(has_scale), "+s"(grid));
#pragma unroll
    for (int k = 0; k < K; ++k) asm volatile("" : "+s"(s.in[k]));
}

// Up to kFewSegs segments passed by value in the kernel arguments: blockIdx.y
// picks the segment, blockIdx.x strides over its packets.
//
// Occupancy: a CU holds four 512-thread blocks (8 waves per SIMD) only while a
// wave's scalar registers fit an allocation of 80 -- measured on MI355X: a
// kernel with more starts 768 blocks at launch instead of 1024 and streams
// 2-4 % slower.  Six registers are set aside on top of what the code uses (VCC,
// flat scratch, XNACK mask), so the code itself has 74.
template <class C, bool FAN = false>
__device__ __forceinline__ void fold_few_body(const FewArgs& a) {
#if MCCLX_TUNE_TIMELINE
    const uint64_t t_start = wall_clock64();
#endif
    SegArgs s = a.seg[blockIdx.y];
    float scale = a.scale;
    int32_t has_scale = a.has_scale;
    uint32_t grid = gridDim.x;
    fetch_together<FAN ? MCCLX_MAX_INPUTS : C::K>(s, scale, has_scale, grid);
    int32_t fan = 0;
    if constexpr (FAN) fan = a.fan;
#if MCCLX_TUNE_TIMELINE
    const uint64_t t_args = wall_clock64();
#endif
    const uint64_t span = (uint64_t)C::U * C::BLOCK;
    // one tile per block, no loop: the launch sizes the grid to the longest segment.  Blocks are
    // dispatched in address order (giving each XCD one contiguous part of a segment instead was
    // level on a 25 MiB bucket and 3.5-9 % slower on large operands).
    (void)grid;
    fold_tile<C, FAN>(s, scale, has_scale != 0, (uint64_t)blockIdx.x * span, blockIdx.x == 0, fan);
#if MCCLX_TUNE_TIMELINE
    if (a.timeline && threadIdx.x == 0) {
        TimelineRecord r;
        r.t_start = t_start;
        r.t_args = t_args;
        r.t_end = wall_clock64();
        r.hw_id = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_ID: wave, SIMD, CU, SH, SE
        r.xcc_id = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
        a.timeline[(uint64_t)blockIdx.y * gridDim.x + blockIdx.x] = r;
    }
#endif
}

// Plans whose vector registers allow 8 waves per SIMD are held to 74 scalar
// registers (a handful of spills into vector-register lanes); wide folds, which
// the vector registers already limit to fewer waves, keep what they need.
#define MCCLX_SGPR_CAP __attribute__((amdgpu_num_sgpr(80)))
template <class C> constexpr bool kLightPlan = C::K <= 4;

template <class C>
__global__ void __launch_bounds__(C::BLOCK) MCCLX_SGPR_CAP fold_few_kernel(FewArgs a) { fold_few_body<C>(a); }
template <class C>
__global__ void __launch_bounds__(C::BLOCK) fold_few_wide_kernel(FewArgs a) { fold_few_body<C>(a); }
// Fan-out form: the result also goes to in[K .. K+fan-1] (the other ranks' tensors: the
// allgather leg of an allreduce done by the reduce itself, stores instead of a second pass).
template <class C>
__global__ void __launch_bounds__(C::BLOCK) fold_few_fan_kernel(FewArgs a) { fold_few_body<C, true>(a); }

#if MCCLX_TUNE_TIMELINE
// Where the next by-value launches put their records (measurement build): a caller-provided
// device buffer cut into `slots` regions of `per_slot` records, used round robin.  This file
// is compiled once per part; part 0 holds the state.
TimelineRecord* timeline_next(uint64_t blocks);
#endif

// ------------------------------------------------------ reads, then writes
//
// A launch that mixes its reads and writes streams about 10 % slower on this
// part than one that only reads or only writes (the memory bus pays for every
// change of direction).  A launch small enough for ONE generation of blocks to
// cover it can keep the two apart: every lane issues the loads of all its T
// packets at once, folds them as they arrive, keeps the T results in registers
// and stores them only when the launch's reads are through.  "Through" is a
// matter of time, not of a barrier: the host knows how many bytes the launch
// reads and passes the moment (in ticks of the device's wall clock, 100 MHz on
// gfx950, counted from the block's own start) before which no lane stores.  A gate that is too late
// costs its excess, one that is too early lets writes into the reads again --
// results do not depend on it.  C2 (78.6 MB per launch): 14.1 -> 12.9 us.
//
// What one generation holds is set by the vector registers (every packet in
// flight occupies them until it is stored; a packet's result takes the place of
// its first operand): the launch takes T = 4 or 5 packets per lane, in 512-lane
// blocks, whichever covers the longest segment in one generation -- C2-shaped
// folds of up to 40 MiB per rank, the all-fp32 fold of a 25 MiB bucket.  More
// packets per lane would cover more, but from about 80 MB read on the plain
// form has caught up (a 40 MiB bucket at T = 7: 21.0 us against 20.7 us); and
// 256-lane blocks run the C2 fold in 14.3 us where 512-lane blocks take 13.1 us.
template <class C, int T, int kHoldBlock, bool FAN>
__global__ void __launch_bounds__(kHoldBlock) fold_few_hold_kernel(FewArgs a, uint32_t gate) {
    const uint64_t t_start = wall_clock64();
    SegArgs s = a.seg[blockIdx.y];
    float scale = a.scale;
    int32_t has_scale = a.has_scale;
    uint32_t grid = gridDim.x;
    fetch_together<FAN ? MCCLX_MAX_INPUTS : C::K>(s, scale, has_scale, grid);
    int32_t fan = 0;
    if constexpr (FAN) fan = a.fan;
    const uint32_t head = head_elems<C>(s);
    const uint64_t P = (s.count - head) / C::E;
    const bool has_out = s.out != nullptr, has_wire = s.wire_out != nullptr;
    const SegArgs t = advanced<C, FAN>(s, head);
    // packet u of lane l is packet u * L + l of the segment: consecutive lanes, consecutive packets
    const uint32_t L = grid * kHoldBlock;
    const uint32_t lane = blockIdx.x * kHoldBlock + threadIdx.x;
    // Packet indices are worked out again for the arithmetic and for the stores (behind a
    // barrier the compiler cannot see through) instead of being kept in registers across
    // the wait: registers decide how many packets one generation holds.
    RawPack raw[C::K][T];
    {
#pragma unroll
        for (int u = 0; u < T; ++u) {
            const uint32_t p = (uint32_t)u * L + lane;
            if (p < P) {
                uint32_t one[1] = {p};
                RawPack col[C::K][1];
                load_all<C, 0, 1>(t, one, col);
#pragma unroll
                for (int k = 0; k < C::K; ++k) raw[k][u] = col[k][0];
            }
        }
    }
    // a packet's result takes the place of its first operand: four fp32 values, or eight
    // 16-bit ones in the form they are stored in
    uint32_t lane2 = lane;
    asm volatile("" : "+v"(lane2));
#pragma unroll
    for (int u = 0; u < T; ++u)
        if ((uint32_t)u * L + lane2 < P) {
            RawPack col[C::K];
#pragma unroll
            for (int k = 0; k < C::K; ++k) col[k] = raw[k][u];
            float acc[C::E];
            combine<C>(col, acc);
            finish_pack<C>(acc, scale, has_scale != 0);
            if constexpr (C::E == 4) {
                raw[0][u] = u32x4{__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]), __float_as_uint(acc[3])};
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) raw[0][u][j] = Num<C::W>::enc(acc[2 * j]) | (Num<C::W>::enc(acc[2 * j + 1]) << 16);
            }
        }
#if MCCLX_TUNE_TIMELINE
    const uint64_t t_args = wall_clock64();  // here: this block has its data
#endif
    // the clock only moves forward, so every wave leaves this loop
    while (wall_clock64() - t_start < gate) __builtin_amdgcn_s_sleep(8);
    uint32_t lane3 = lane2;
    asm volatile("" : "+v"(lane3));
#pragma unroll
    for (int u = 0; u < T; ++u) {
        const uint32_t p = (uint32_t)u * L + lane3;
        if (p < P) {
            if constexpr (C::E == 4) {
                const float y[C::E] = {__uint_as_float(raw[0][u].x), __uint_as_float(raw[0][u].y), __uint_as_float(raw[0][u].z),
                                       __uint_as_float(raw[0][u].w)};
                store_pack<C, FAN>(t, has_out, has_wire, p, y, fan);
            } else {  // all streams 16-bit: the packed result goes out as it is
                const u32x4 bits = raw[0][u];
                if (has_out) MCCLX_STG(gptr<u32x4_a2>(static_cast<uint16_t*>(t.out) + p * C::E), bits);
                if (has_wire) MCCLX_STG(gptr<u32x4_a2>(static_cast<uint16_t*>(t.wire_out) + p * C::E), bits);
                if constexpr (FAN) {
#pragma unroll
                    for (int f = 0; f < MCCLX_MAX_INPUTS - C::K; ++f)
                        if (f < fan)
                            MCCLX_STG(gptr<u32x4_a2>(static_cast<uint16_t*>(const_cast<void*>(t.in[C::K + f])) + p * C::E), bits);
                }
            }
        }
    }
    if (blockIdx.x == 0) {  // the elements in front of and behind the packet grid
        if (threadIdx.x < head) fold_elem<C, FAN>(s, threadIdx.x, scale, has_scale != 0, fan);
        const uint64_t i = head + P * C::E + threadIdx.x;
        if (i < s.count) fold_elem<C, FAN>(s, i, scale, has_scale != 0, fan);
    }
#if MCCLX_TUNE_TIMELINE
    if (a.timeline && threadIdx.x == 0) {
        TimelineRecord r;
        r.t_start = t_start;
        r.t_args = t_args;
        r.t_end = wall_clock64();
        r.hw_id = __builtin_amdgcn_s_getreg((31 << 11) | 4);
        r.xcc_id = __builtin_amdgcn_s_getreg((31 << 11) | 20);
        a.timeline[(uint64_t)blockIdx.y * gridDim.x + blockIdx.x] = r;
    }
#endif
}

// Plans with a reads-then-writes form: sums of two to four operands, rounding after every step,
// and the wire encode (one fp32 operand in, its bf16 form out: the first launch of every
// schedule that sends bf16 copies; ten 16-byte packets per lane cover three 25 MiB tensors).
template <class C>
constexpr bool kHoldEncode = C::K == 1 && C::IO == MCCLX_IO_OWN_FIRST_F32 && C::ACC == MCCLX_ACC_STEP;
constexpr uint64_t kHoldEncodeEarlyPct = 105;  // the encode's gate: the model's rate taken 5 % higher
constexpr uint64_t kHoldFanLatePct = 97;       // a fan-out fold at five packets per lane: the model's rate taken 3 % lower
template <class C>
constexpr bool kHoldPlan = ((C::K >= 2 && C::K <= 4) || kHoldEncode<C>) && C::OP == MCCLX_SUM &&
                           C::ACC == MCCLX_ACC_STEP && C::TOPO == MCCLX_TOPO_FOLD;

// Blocks of one generation: what the device holds at once of this kernel.
template <class C, int T, int HB, bool FAN>
static uint32_t hold_capacity(int cus) {
    static const int per_cu = [] {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fold_few_hold_kernel<C, T, HB, FAN>, HB, 0) != hipSuccess) {
            (void)hipGetLastError();
            n = 0;
        }
        return n;
    }();
    return (uint32_t)(per_cu * cus);
}

template <class C, int T, int HB, bool FAN>
static bool hold_launch(hipStream_t st, FewArgs& a, uint64_t packets, uint32_t gate, const LaunchParams& lp) {
    const uint32_t cap = hold_capacity<C, T, HB, FAN>(lp.cus);
    if (cap < (uint32_t)a.nseg) return false;
    uint32_t hx = cap / (uint32_t)a.nseg;
    if (packets > (uint64_t)hx * HB * T) return false;
    // As many blocks as the device holds -- the more waves share the launch's loads, the sooner
    // they are through (C2 with 267 instead of 341 blocks per segment: 16 us instead of 13) --
    // but a whole number of fours per segment: measured on a 25 MiB bucket of three segments,
    // 340 and 336 blocks per segment run the launch in 13.07 us, 341 in 13.22, 338 in 13.3 and
    // 339 in 13.9 (which blocks of the three segments share an XCD, and the distance between a
    // lane's packets, change with it).
    if (hx >= 8 && packets <= (uint64_t)(hx & ~3u) * HB * T) hx &= ~3u;
#if MCCLX_TUNE_TIMELINE
    a.timeline = timeline_next((uint64_t)hx * (uint64_t)a.nseg);
#endif
    fold_few_hold_kernel<C, T, HB, FAN><<<dim3(hx, (uint32_t)a.nseg), dim3(HB), 0, st>>>(a, gate);
    return true;
}

// Takes the launch if it reads enough for the separation to pay and one generation covers it.
template <class C, bool FAN>
static bool try_hold(hipStream_t st, FewArgs& a, uint64_t maxc, const LaunchParams& lp) {
    if (!lp.hold_min_read_bytes || lp.cus <= 0) return false;
    uint64_t read_bytes = 0;
    for (int i = 0; i < a.nseg; ++i)
        for (int k = 0; k < C::K; ++k) read_bytes += a.seg[i].count * (C::in_is_f32(k) ? 4 : 2);
    // measured break-even: 10 MiB read for a fold with one output, half as much again for one that
    // writes as much as it reads (fan-out)
    if (read_bytes < (FAN ? lp.hold_min_read_bytes * 3 / 2 : lp.hold_min_read_bytes)) return false;
    // The encode: measured on 1-8 tensors of 1-40 MiB, the form wins 4-10 % from three tensors and
    // 18 MiB read on (three of 25 MiB: 20.6 -> 19.0 us); on one or two tensors it ties or loses.
    if constexpr (kHoldEncode<C>)
        if (a.nseg < 3 || read_bytes < lp.hold_min_read_bytes * 9 / 5) return false;
    uint64_t ticks = lp.hold_latency_ticks + read_bytes / lp.hold_bytes_per_tick;
    // the encode writes half of what it reads and does best with its stores a little early
    if constexpr (kHoldEncode<C>) ticks = lp.hold_latency_ticks + read_bytes * 100 / (lp.hold_bytes_per_tick * kHoldEncodeEarlyPct);
    uint32_t gate5 = 0;  // a fan-out fold at five packets per lane (fewer waves, more loads each): its reads take 3 % longer
    if constexpr (FAN) {
        const uint64_t t5 = lp.hold_latency_ticks + read_bytes * 100 / (lp.hold_bytes_per_tick * kHoldFanLatePct);
        gate5 = t5 > 100000 ? 100000u : (uint32_t)t5;
    }
    const uint32_t gate = ticks > 100000 ? 100000u : (uint32_t)ticks;  // a millisecond at most
    const uint64_t packets = (maxc + C::E - 1) / C::E;
    // Four packets per lane if that covers the launch, five otherwise.  (The one-launch allreduce of a
    // 25 MiB bucket, which writes as much as it reads: 26.2 us at four, each form at its best gate,
    // 26.7 us at five.)
    bool took;
    if constexpr (kHoldEncode<C>)
        took = hold_launch<C, 10, 512, false>(st, a, packets, gate, lp);
    else
        took = hold_launch<C, 4, 512, FAN>(st, a, packets, gate, lp) || hold_launch<C, 5, 512, FAN>(st, a, packets, FAN ? gate5 : gate, lp);
    if (took && lp.held) *lp.held = true;
    return took;
}

// A value that is the same in every lane, moved to scalar registers.  The
// compiler cannot always prove it (a quotient comes out of the vector ALU), and
// a descriptor kept in vector registers costs the kernel a quarter of its
// resident blocks.
__device__ __forceinline__ uint32_t uni32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t uni64(uint64_t v) {
    return ((uint64_t)uni32((uint32_t)(v >> 32)) << 32) | uni32((uint32_t)v);
}
template <class P>
__device__ __forceinline__ P* uniptr(P* p) {
    return reinterpret_cast<P*>(uni64(reinterpret_cast<uint64_t>(p)));
}

// Blocks over a descriptor table in device memory: work item w is tile
// (w - first_item[seg]) of segment seg; a block takes items blockIdx.x,
// blockIdx.x + gridDim.x, ...  (one item per block unless the grid is capped).
// The loop bound is fixed at launch, so every wave exits.  total_items < 2^31
// (checked by the host).
template <class C, bool FAN = false>
__device__ __forceinline__ void fold_table_body(const TableArgs& a) {
    const uint64_t span = (uint64_t)C::U * C::BLOCK;
    const uint32_t total = (uint32_t)a.total_items;
    const uint32_t uniform = (uint32_t)a.uniform_items;
    for (uint32_t w = blockIdx.x; w < total; w += gridDim.x) {
        uint32_t seg, tile;
        if (uniform) {
            seg = w / uniform;
            tile = w - seg * uniform;
        } else if (a.item_map) {  // ragged segments: the host has written out who owns item w
            const uint2 m = a.item_map[w];
            seg = m.x;
            tile = m.y;
        } else {
            uint32_t lo = 0, hi = a.nseg;  // first_item[lo] <= w < first_item[hi]
            while (hi - lo > 1) {
                uint32_t mid = (lo + hi) >> 1;
                if ((uint32_t)a.first_item[mid] <= w) lo = mid; else hi = mid;
            }
            seg = lo;
            tile = w - (uint32_t)a.first_item[seg];
        }
        // w depends on blockIdx only, so segment and tile are the same for every lane
        seg = uni32(seg);
        tile = uni32(tile);
        const SegArgs* __restrict__ d = a.segs + seg;
        SegArgs s;
        s.out = uniptr(d->out);
        s.wire_out = uniptr(d->wire_out);
#pragma unroll
        for (int k = 0; k < MCCLX_MAX_INPUTS; ++k) s.in[k] = (k < C::K || FAN) ? uniptr(d->in[k]) : nullptr;
        s.count = uni64(d->count);
        // one tile: packets [tile*span, tile*span + span); tile 0 also owns the tail
        fold_tile<C, FAN>(s, a.scale, a.has_scale != 0, (uint64_t)tile * span, tile == 0, FAN ? a.fan : 0);
    }
}

template <class C>
__global__ void __launch_bounds__(C::BLOCK) MCCLX_SGPR_CAP fold_table_kernel(TableArgs a) { fold_table_body<C>(a); }
template <class C>
__global__ void __launch_bounds__(C::BLOCK) fold_table_wide_kernel(TableArgs a) { fold_table_body<C>(a); }
template <class C>
__global__ void __launch_bounds__(C::BLOCK) fold_table_fan_kernel(TableArgs a) { fold_table_body<C, true>(a); }

// Plans with a fan-out form (host mirror: fan_plan_ok).
template <class C>
constexpr bool kFanPlan = C::OP == MCCLX_SUM && C::ACC == MCCLX_ACC_STEP && C::K >= 2 && C::K < MCCLX_MAX_INPUTS &&
                          C::IO != MCCLX_IO_OUT_F32;

// ----------------------------------------------------------------- dispatch


template <class C>
static hipError_t launch_cfg(hipStream_t st, const LaunchParams& lp) {
    const uint64_t span = (uint64_t)C::U * C::BLOCK * C::E;  // elements per block iteration
    if (lp.fan > 0) {
        if constexpr (!kFanPlan<C>) {
            return hipErrorInvalidValue;
        } else {
            if (lp.fan > MCCLX_MAX_INPUTS - C::K) return hipErrorInvalidValue;
            if (lp.table) {
                TableArgs a = *lp.table;
                a.fan = lp.fan;
                uint32_t grid = (uint32_t)(a.total_items < lp.max_blocks ? a.total_items : lp.max_blocks);
                if (grid == 0) return hipSuccess;
                fold_table_fan_kernel<C><<<dim3(grid), dim3(C::BLOCK), 0, st>>>(a);
            } else {
                FewArgs a = *lp.few;
                a.fan = lp.fan;
                uint64_t maxc = 0;
                for (int i = 0; i < a.nseg; ++i) maxc = a.seg[i].count > maxc ? a.seg[i].count : maxc;
                if (maxc == 0) return hipSuccess;
                uint64_t gx = (maxc + span - 1) / span;
                if (gx >> 31) return hipErrorInvalidValue;
#if MCCLX_TUNE_TIMELINE
                a.timeline = nullptr;
#endif
                if constexpr (kHoldPlan<C>)
                    if (try_hold<C, true>(st, a, maxc, lp)) return hipGetLastError();
                fold_few_fan_kernel<C><<<dim3((uint32_t)gx, (uint32_t)a.nseg), dim3(C::BLOCK), 0, st>>>(a);
            }
            return hipGetLastError();
        }
    }
    if (lp.table) {
        TableArgs a = *lp.table;
        uint32_t grid = (uint32_t)(a.total_items < lp.max_blocks ? a.total_items : lp.max_blocks);
        if (grid == 0) return hipSuccess;
        if constexpr (kLightPlan<C>)
            fold_table_kernel<C><<<dim3(grid), dim3(C::BLOCK), 0, st>>>(a);
        else
            fold_table_wide_kernel<C><<<dim3(grid), dim3(C::BLOCK), 0, st>>>(a);
    } else {
        FewArgs a = *lp.few;
        uint64_t maxc = 0;
        for (int i = 0; i < a.nseg; ++i) maxc = a.seg[i].count > maxc ? a.seg[i].count : maxc;
        if (maxc == 0) return hipSuccess;
        // one block per tile of the longest segment (the by-value kernel does not loop)
        uint64_t gx = (maxc + span - 1) / span;
        if (gx >> 31) return hipErrorInvalidValue;
        if constexpr (kHoldPlan<C>)
            if (try_hold<C, false>(st, a, maxc, lp)) return hipGetLastError();
#if MCCLX_TUNE_TIMELINE
        a.timeline = timeline_next(gx * (uint64_t)a.nseg);
#endif
        if constexpr (kLightPlan<C>)
            fold_few_kernel<C><<<dim3((uint32_t)gx, (uint32_t)a.nseg), dim3(C::BLOCK), 0, st>>>(a);
        else
            fold_few_wide_kernel<C><<<dim3((uint32_t)gx, (uint32_t)a.nseg), dim3(C::BLOCK), 0, st>>>(a);
    }
    return hipGetLastError();
}

// The kernel template is instantiated for every supported plan.  To keep build
// times short the instantiations are spread over several translation units:
// this file is compiled once per part with -DMCCLX_PART=n (or once, with every
// part, when MCCLX_PART is not given).
#ifndef MCCLX_PART
#define MCCLX_PART -1
#endif
#define MCCLX_HAS_PART(n) (MCCLX_PART == -1 || MCCLX_PART == (n))

#if MCCLX_TUNE_TIMELINE && MCCLX_HAS_PART(0)
static TimelineRecord* g_tl_buf = nullptr;
static uint64_t g_tl_slots = 0, g_tl_per_slot = 0, g_tl_next = 0;
TimelineRecord* timeline_next(uint64_t blocks) {
    if (!g_tl_buf || blocks > g_tl_per_slot) return nullptr;
    return g_tl_buf + (g_tl_next++ % g_tl_slots) * g_tl_per_slot;
}
extern "C" MCCLX_API void mcclx_tune_timeline(void* device_buf, uint64_t slots, uint64_t records_per_slot) {
    g_tl_buf = static_cast<TimelineRecord*>(device_buf);
    g_tl_slots = slots;
    g_tl_per_slot = records_per_slot;
    g_tl_next = 0;
}
#endif

#if MCCLX_HAS_PART(0)
int plan_block(const PlanKey& key);
static int key_pack_elems(const PlanKey& key) {
    return (key.dtype == MCCLX_F32 || key.io != MCCLX_IO_PURE) ? 4 : 8;
}

uint32_t items_for(const PlanKey& k, uint64_t count) {
    // Mirrors Cfg::U / Cfg::E on the host, for table building.  The head peel
    // only ever removes elements from the packet grid, so this is an upper
    // bound; a tile past the end finds no packets and does nothing.
    uint64_t span = (uint64_t)plan_unroll(k) * plan_block(k) * key_pack_elems(k);
    uint64_t n = (count + span - 1) / span;
    return (uint32_t)(n ? n : (count ? 1 : 0));
}

static bool key_is_wide(const PlanKey& key) { return key_pack_elems(key) == 8 && key.k >= kWideMinK; }

int plan_block(const PlanKey& key) {
    const bool decode = key.k == 1 && key.io == MCCLX_IO_OUT_F32;
    if (key_is_wide(key)) return kWideBlock;
    if ((key.dtype == MCCLX_F32 && key.k >= 2) || decode) return kF32Block;
    return (key.io == MCCLX_IO_ALL_F32 && key.k >= 2) ? kAllF32Block : kBlock;
}

bool fan_plan_ok(const PlanKey& key) {
    return key.op == MCCLX_SUM && key.acc == MCCLX_ACC_STEP && key.k >= 2 && key.k < MCCLX_MAX_INPUTS &&
           key.io != MCCLX_IO_OUT_F32;
}

int plan_unroll(const PlanKey& key) {
    if (key_is_wide(key)) return kWideU;
    if (key.topo == MCCLX_TOPO_BINOMIAL) return 1;
    return (key_pack_elems(key) == 8 || (key.k == 1 && key.io != MCCLX_IO_PURE)) ? 2 : 1;
}
#endif  // part 0: host-side mirrors of the kernel configuration

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

// k < 4 has one shape only (the binomial tree of 2 or 3 ranks is the left fold)
#define MCCLX_TOPO_CASES(W, IO, OP, ACC)                                                \
    if (key.topo == MCCLX_TOPO_BINOMIAL && key.k >= 4) {                                \
        MCCLX_K_CASES(W, IO, MCCLX_TOPO_BINOMIAL, OP, ACC)                              \
    } else {                                                                            \
        MCCLX_K_CASES(W, IO, MCCLX_TOPO_FOLD, OP, ACC)                                  \
    }

// MIN / MAX / PRODUCT: same-dtype operands, rounding after every step
#define MCCLX_OTHER_OPS(W)                                                              \
    switch (key.op) {                                                                   \
        case MCCLX_PRODUCT: MCCLX_TOPO_CASES(W, MCCLX_IO_PURE, MCCLX_PRODUCT, MCCLX_ACC_STEP) \
        case MCCLX_MIN: MCCLX_TOPO_CASES(W, MCCLX_IO_PURE, MCCLX_MIN, MCCLX_ACC_STEP)   \
        case MCCLX_MAX: MCCLX_TOPO_CASES(W, MCCLX_IO_PURE, MCCLX_MAX, MCCLX_ACC_STEP)   \
        case MCCLX_MIN_ACC_SRC: MCCLX_K_CASES(W, MCCLX_IO_PURE, MCCLX_TOPO_FOLD, MCCLX_MIN_ACC_SRC, MCCLX_ACC_STEP) \
        case MCCLX_MAX_ACC_SRC: MCCLX_K_CASES(W, MCCLX_IO_PURE, MCCLX_TOPO_FOLD, MCCLX_MAX_ACC_SRC, MCCLX_ACC_STEP) \
        default: return hipErrorInvalidValue;                                           \
    }

#define MCCLX_BF16_IO_CASES(ACC)                                                                   \
    switch (key.io) {                                                                              \
        case MCCLX_IO_PURE: MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_PURE, MCCLX_SUM, ACC)            \
        case MCCLX_IO_OUT_F32: MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_OUT_F32, MCCLX_SUM, ACC)      \
        case MCCLX_IO_OWN_FIRST_F32:                                                               \
            MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_OWN_FIRST_F32, MCCLX_SUM, ACC)                   \
        case MCCLX_IO_OWN_LAST_F32:                                                                \
            MCCLX_K_CASES(MCCLX_BF16, MCCLX_IO_OWN_LAST_F32, MCCLX_TOPO_FOLD, MCCLX_SUM, ACC)      \
        case MCCLX_IO_ALL_F32: return launch_part_sum_bf16_all_f32(st, key, lp);                   \
        default: return hipErrorInvalidValue;                                                      \
    }

hipError_t launch_part_sum_f32_f16(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_sum_bf16_step(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_sum_bf16_f32acc(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_sum_bf16_all_f32(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_ops_f32(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_ops_f16(hipStream_t st, const PlanKey& key, const LaunchParams& lp);
hipError_t launch_part_ops_bf16(hipStream_t st, const PlanKey& key, const LaunchParams& lp);

#if MCCLX_HAS_PART(0)
hipError_t launch_fold(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    if (key.op != MCCLX_SUM) {
        if (key.io != MCCLX_IO_PURE || key.acc != MCCLX_ACC_STEP) return hipErrorInvalidValue;
        switch (key.dtype) {
            case MCCLX_F32: return launch_part_ops_f32(st, key, lp);
            case MCCLX_F16: return launch_part_ops_f16(st, key, lp);
            case MCCLX_BF16: return launch_part_ops_bf16(st, key, lp);
            default: return hipErrorInvalidValue;
        }
    }
    if (key.dtype == MCCLX_F32 || key.dtype == MCCLX_F16) {
        if (key.io != MCCLX_IO_PURE || key.acc != MCCLX_ACC_STEP) return hipErrorInvalidValue;
        return launch_part_sum_f32_f16(st, key, lp);
    }
    if (key.dtype != MCCLX_BF16) return hipErrorInvalidValue;
    return key.acc == MCCLX_ACC_STEP ? launch_part_sum_bf16_step(st, key, lp)
                                     : launch_part_sum_bf16_f32acc(st, key, lp);
}

hipError_t launch_part_sum_f32_f16(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    if (key.dtype == MCCLX_F32) {
        MCCLX_TOPO_CASES(MCCLX_F32, MCCLX_IO_PURE, MCCLX_SUM, MCCLX_ACC_STEP)
    }
    MCCLX_TOPO_CASES(MCCLX_F16, MCCLX_IO_PURE, MCCLX_SUM, MCCLX_ACC_STEP)
}
#endif

#if MCCLX_HAS_PART(1)
hipError_t launch_part_sum_bf16_step(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    MCCLX_BF16_IO_CASES(MCCLX_ACC_STEP)
}
#endif

#if MCCLX_HAS_PART(2)
hipError_t launch_part_sum_bf16_f32acc(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    MCCLX_BF16_IO_CASES(MCCLX_ACC_F32)
}
#endif

#if MCCLX_HAS_PART(3)
hipError_t launch_part_ops_f32(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    MCCLX_OTHER_OPS(MCCLX_F32)
}
#endif

#if MCCLX_HAS_PART(4)
hipError_t launch_part_ops_f16(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    MCCLX_OTHER_OPS(MCCLX_F16)
}
#endif

#if MCCLX_HAS_PART(5)
hipError_t launch_part_ops_bf16(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    MCCLX_OTHER_OPS(MCCLX_BF16)
}
#endif

#if MCCLX_HAS_PART(6)
// every operand fp32, encoded in registers (MCCLX_IO_ALL_F32)
hipError_t launch_part_sum_bf16_all_f32(hipStream_t st, const PlanKey& key, const LaunchParams& lp) {
    if (key.acc == MCCLX_ACC_STEP) {
        MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_ALL_F32, MCCLX_SUM, MCCLX_ACC_STEP)
    }
    MCCLX_TOPO_CASES(MCCLX_BF16, MCCLX_IO_ALL_F32, MCCLX_SUM, MCCLX_ACC_F32)
}
#endif

}  // namespace mcclx
