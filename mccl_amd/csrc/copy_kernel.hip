// copy_kernel.hip -- streaming device copy on the reduce queue: the allgather
// legs (AllreduceAlgos.cpp:77-86, ProcessGroupMCCL.cpp:232-273) and the
// unstage copy (MPSInterop.mm:408-435).  Also the known-traffic kernel the
// memory counters are calibrated against.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fold_launch.h"

#ifndef MCCLX_TUNE_COPY_U
#define MCCLX_TUNE_COPY_U 1
#endif
#ifndef MCCLX_TUNE_COPY_NT
#define MCCLX_TUNE_COPY_NT 1  // every byte is touched once: non-temporal loads and stores
#endif

namespace mcclx {
namespace {
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define MCCLX_GLOBAL __attribute__((address_space(1)))
#if MCCLX_TUNE_COPY_NT
#define COPY_LD(p) __builtin_nontemporal_load(p)
#define COPY_ST(p, v) __builtin_nontemporal_store((v), (p))
#else
#define COPY_LD(p) (*(p))
#define COPY_ST(p, v) (*(p) = (v))
#endif
// the widest alignment both pointers share decides the packet type
template <int A> struct Packet;
template <> struct Packet<4> { typedef u32x4 type __attribute__((aligned(4))); };
template <> struct Packet<2> { typedef u32x4 type __attribute__((aligned(2))); };
template <> struct Packet<1> { typedef u32x4 type __attribute__((aligned(1))); };
constexpr int kBlock = 256;
constexpr int kU = MCCLX_TUNE_COPY_U;

template <int A>
__global__ void __launch_bounds__(kBlock) copy_kernel(uint8_t* dst, const uint8_t* src, uint64_t nbytes) {
    typedef typename Packet<A>::type V;
    const MCCLX_GLOBAL uint8_t* gs = (const MCCLX_GLOBAL uint8_t*)src;
    MCCLX_GLOBAL uint8_t* gd = (MCCLX_GLOBAL uint8_t*)dst;
    const uint64_t P = nbytes / 16;
    const uint64_t span = (uint64_t)kU * kBlock;
    for (uint64_t base = (uint64_t)blockIdx.x * span; base < P; base += (uint64_t)gridDim.x * span) {
        if (base + span <= P) {
            u32x4 v[kU];
#pragma unroll
            for (int u = 0; u < kU; ++u)
                v[u] = COPY_LD((const MCCLX_GLOBAL V*)(gs + (base + (uint64_t)u * kBlock + threadIdx.x) * 16));
#pragma unroll
            for (int u = 0; u < kU; ++u)
                COPY_ST((MCCLX_GLOBAL V*)(gd + (base + (uint64_t)u * kBlock + threadIdx.x) * 16), v[u]);
        } else {
            for (uint64_t p = base + threadIdx.x; p < P; p += kBlock) {
                u32x4 v = COPY_LD((const MCCLX_GLOBAL V*)(gs + p * 16));
                COPY_ST((MCCLX_GLOBAL V*)(gd + p * 16), v);
            }
        }
    }
    if (blockIdx.x == 0) {
        uint64_t i = P * 16 + threadIdx.x;
        if (i < nbytes) gd[i] = gs[i];
    }
}
}  // namespace

hipError_t launch_copy(hipStream_t st, void* dst, const void* src, uint64_t nbytes,
                       uint32_t max_blocks) {
    if (nbytes == 0) return hipSuccess;
    const uint64_t span = (uint64_t)kU * kBlock * 16;
    uint64_t g = (nbytes + span - 1) / span;
    if (g > max_blocks) g = max_blocks;
    if (g < 1) g = 1;
    uint8_t* d = static_cast<uint8_t*>(dst);
    const uint8_t* s = static_cast<const uint8_t*>(src);
    const uintptr_t both = reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(s);
    if (both % 4 == 0)
        copy_kernel<4><<<dim3((uint32_t)g), dim3(kBlock), 0, st>>>(d, s, nbytes);
    else if (both % 2 == 0)
        copy_kernel<2><<<dim3((uint32_t)g), dim3(kBlock), 0, st>>>(d, s, nbytes);
    else
        copy_kernel<1><<<dim3((uint32_t)g), dim3(kBlock), 0, st>>>(d, s, nbytes);
    return hipGetLastError();
}

}  // namespace mcclx
