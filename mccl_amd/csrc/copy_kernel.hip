// copy_kernel.hip -- streaming device copies on the reduce queue: the allgather
// legs (AllreduceAlgos.cpp:77-86, ProcessGroupMCCL.cpp:232-273) and the
// unstage copy (MPSInterop.mm:408-435); a few copies travel by value in the
// kernel arguments and run as one grid, thousands go through a table.  Also the
// known-traffic kernel the memory counters are calibrated against, and the
// read-only / write-only probes a launch's footprint is measured against.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fold_launch.h"

namespace mcclx {
namespace {
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define MCCLX_GLOBAL __attribute__((address_space(1)))
// every byte is touched once: non-temporal loads and stores
#define COPY_LD(p) __builtin_nontemporal_load(p)
#define COPY_ST(p, v) __builtin_nontemporal_store((v), (p))
// the widest alignment both pointers share decides the packet type
template <int A> struct Packet;
template <> struct Packet<4> { typedef u32x4 type __attribute__((aligned(4))); };
template <> struct Packet<2> { typedef u32x4 type __attribute__((aligned(2))); };
template <> struct Packet<1> { typedef u32x4 type __attribute__((aligned(1))); };
constexpr int kBlock = 256;
constexpr int kU = 1;  // packets per lane

// Up to kFewCopies copies with their descriptors in the kernel arguments:
// blockIdx.y picks the copy, blockIdx.x one tile of kU * kBlock packets of 16
// bytes; block 0 of a copy also moves the bytes behind its last whole packet.
// One tile per block and no loop, like the fold kernels: a uniform 64-bit base
// plus a 32-bit lane offset per access, and a short path to the first load.
template <int A>
__global__ void __launch_bounds__(kBlock) copy_few_kernel(CopyFew a) {
    typedef typename Packet<A>::type V;
    const CopyDesc d = a.d[blockIdx.y];
    const uint64_t P = d.nbytes / 16;
    const uint64_t first = (uint64_t)blockIdx.x * (kU * kBlock);
    if (first < P) {
        const MCCLX_GLOBAL uint8_t* gs = (const MCCLX_GLOBAL uint8_t*)d.src + first * 16;
        MCCLX_GLOBAL uint8_t* gd = (MCCLX_GLOBAL uint8_t*)d.dst + first * 16;
        const uint64_t left = P - first;
        if (left >= (uint64_t)kU * kBlock) {
            u32x4 v[kU];
#pragma unroll
            for (int u = 0; u < kU; ++u) v[u] = COPY_LD((const MCCLX_GLOBAL V*)(gs + ((uint32_t)u * kBlock + threadIdx.x) * 16u));
#pragma unroll
            for (int u = 0; u < kU; ++u) COPY_ST((MCCLX_GLOBAL V*)(gd + ((uint32_t)u * kBlock + threadIdx.x) * 16u), v[u]);
        } else {
            for (uint32_t p = threadIdx.x; p < (uint32_t)left; p += kBlock) {
                u32x4 v = COPY_LD((const MCCLX_GLOBAL V*)(gs + p * 16u));
                COPY_ST((MCCLX_GLOBAL V*)(gd + p * 16u), v);
            }
        }
    }
    if (blockIdx.x == 0) {
        const uint64_t i = P * 16 + threadIdx.x;
        if (i < d.nbytes) ((MCCLX_GLOBAL uint8_t*)d.dst)[i] = ((const MCCLX_GLOBAL uint8_t*)d.src)[i];
    }
}

// One-directional streams with the copy kernel's access shape: what a launch
// that only reads, or only writes, nbytes costs.  The read keeps its loads alive
// through a store no input takes (packet XOR == magic, into the buffer's first
// word).
template <bool WRITE>
__global__ void __launch_bounds__(kBlock) stream_probe_kernel(uint8_t* buf, uint64_t nbytes, uint32_t magic) {
    typedef typename Packet<4>::type V;
    MCCLX_GLOBAL uint8_t* g = (MCCLX_GLOBAL uint8_t*)buf;
    const uint64_t P = nbytes / 16;
    const uint64_t p = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (p >= P) return;
    if (WRITE) {
        const uint32_t w = (uint32_t)p * 2654435761u;
        COPY_ST((MCCLX_GLOBAL V*)(g + p * 16), (u32x4{w, w ^ magic, ~w, w + magic}));
    } else {
        u32x4 v = COPY_LD((const MCCLX_GLOBAL V*)(g + p * 16));
        const uint32_t x = v[0] ^ v[1] ^ v[2] ^ v[3];
        if (x == magic) *(MCCLX_GLOBAL uint32_t*)g = x;
    }
}

__device__ __forceinline__ uint32_t uni32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t uni64(uint64_t v) {
    return ((uint64_t)uni32((uint32_t)(v >> 32)) << 32) | uni32((uint32_t)v);
}

// Many copies, one launch: work item w is tile (w - first_item[c]) of copy c.
// A tile is kManyU * kBlock packets of 16 bytes (16 KiB); tile 0 also moves the
// bytes behind the last whole packet.  The loop bound is fixed at launch.
constexpr int kManyU = 4;

template <int A>
__global__ void __launch_bounds__(kBlock) copy_many_kernel(CopyTable t) {
    typedef typename Packet<A>::type V;
    const uint64_t span = (uint64_t)kManyU * kBlock;
    for (uint32_t w = blockIdx.x; w < t.total_items; w += gridDim.x) {
        uint32_t c, tile;
        if (t.uniform_items) {  // every copy has the same number of tiles: no search
            c = w / t.uniform_items;
            tile = w - c * t.uniform_items;
        } else if (t.item_map) {
            const uint2 m = t.item_map[w];
            c = m.x;
            tile = m.y;
        } else {
            uint32_t lo = 0, hi = t.n;  // first_item[lo] <= w < first_item[hi]
            while (hi - lo > 1) {
                uint32_t mid = (lo + hi) >> 1;
                if ((uint32_t)t.first_item[mid] <= w) lo = mid; else hi = mid;
            }
            c = lo;
            tile = w - (uint32_t)t.first_item[c];
        }
        c = uni32(c);
        tile = uni32(tile);
        const CopyDesc* __restrict__ d = t.descs + c;
        const MCCLX_GLOBAL uint8_t* gs = (const MCCLX_GLOBAL uint8_t*)uni64(reinterpret_cast<uint64_t>(d->src));
        MCCLX_GLOBAL uint8_t* gd = (MCCLX_GLOBAL uint8_t*)uni64(reinterpret_cast<uint64_t>(d->dst));
        const uint64_t nbytes = uni64(d->nbytes);
        const uint64_t P = nbytes / 16;
        const uint64_t base = (uint64_t)tile * span;
        if (base + span <= P) {
            u32x4 v[kManyU];
#pragma unroll
            for (int u = 0; u < kManyU; ++u)
                v[u] = COPY_LD((const MCCLX_GLOBAL V*)(gs + (base + (uint64_t)u * kBlock + threadIdx.x) * 16));
#pragma unroll
            for (int u = 0; u < kManyU; ++u)
                COPY_ST((MCCLX_GLOBAL V*)(gd + (base + (uint64_t)u * kBlock + threadIdx.x) * 16), v[u]);
        } else {
            for (uint64_t p = base + threadIdx.x; p < P; p += kBlock) {
                u32x4 v = COPY_LD((const MCCLX_GLOBAL V*)(gs + p * 16));
                COPY_ST((MCCLX_GLOBAL V*)(gd + p * 16), v);
            }
        }
        if (tile == 0) {
            uint64_t i = P * 16 + threadIdx.x;
            if (i < nbytes) gd[i] = gs[i];
        }
    }
}
}  // namespace

uint64_t copy_items(uint64_t nbytes) {
    const uint64_t span = (uint64_t)kManyU * kBlock * 16;
    uint64_t n = (nbytes + span - 1) / span;
    return n ? n : (nbytes ? 1 : 0);
}

hipError_t launch_copy_many(hipStream_t st, const CopyTable& t, int align, uint32_t max_blocks) {
    if (t.total_items == 0) return hipSuccess;
    uint32_t g = t.total_items < max_blocks ? t.total_items : max_blocks;
    if (align == 4)
        copy_many_kernel<4><<<dim3(g), dim3(kBlock), 0, st>>>(t);
    else if (align == 2)
        copy_many_kernel<2><<<dim3(g), dim3(kBlock), 0, st>>>(t);
    else
        copy_many_kernel<1><<<dim3(g), dim3(kBlock), 0, st>>>(t);
    return hipGetLastError();
}

hipError_t launch_stream_probe(hipStream_t st, void* buf, uint64_t nbytes, bool write) {
    const uint64_t g = (nbytes / 16 + kBlock - 1) / kBlock;
    if (g == 0) return hipSuccess;
    if (g >> 31) return hipErrorInvalidValue;
    uint8_t* b = static_cast<uint8_t*>(buf);
    if (write)
        stream_probe_kernel<true><<<dim3((uint32_t)g), dim3(kBlock), 0, st>>>(b, nbytes, 0x9E3779B9u);
    else
        stream_probe_kernel<false><<<dim3((uint32_t)g), dim3(kBlock), 0, st>>>(b, nbytes, 0x9E3779B9u);
    return hipGetLastError();
}

hipError_t launch_copy_few(hipStream_t st, const CopyFew& a, int align) {
    uint64_t longest = 0;
    for (uint32_t i = 0; i < a.n; ++i) longest = a.d[i].nbytes > longest ? a.d[i].nbytes : longest;
    if (a.n == 0 || longest == 0) return hipSuccess;
    const uint64_t span = (uint64_t)kU * kBlock * 16;
    uint64_t g = (longest + span - 1) / span;
    if (g >> 31) return hipErrorInvalidValue;
    const dim3 grid((uint32_t)g, a.n);
    if (align == 4)
        copy_few_kernel<4><<<grid, dim3(kBlock), 0, st>>>(a);
    else if (align == 2)
        copy_few_kernel<2><<<grid, dim3(kBlock), 0, st>>>(a);
    else
        copy_few_kernel<1><<<grid, dim3(kBlock), 0, st>>>(a);
    return hipGetLastError();
}

hipError_t launch_copy(hipStream_t st, void* dst, const void* src, uint64_t nbytes, uint32_t) {
    if (nbytes == 0) return hipSuccess;
    CopyFew a;
    a.d[0] = CopyDesc{dst, src, nbytes};
    a.n = 1;
    const uintptr_t both = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
    return launch_copy_few(st, a, both % 4 == 0 ? 4 : both % 2 == 0 ? 2 : 1);
}

}  // namespace mcclx
