// copy_kernel.hip -- streaming device copy on the reduce queue: the allgather
// legs (AllreduceAlgos.cpp:77-86, ProcessGroupMCCL.cpp:232-273) and the
// unstage copy (MPSInterop.mm:408-435).  Also the known-traffic kernel the
// memory counters are calibrated against.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fold_launch.h"

namespace mcclx {
namespace {
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// the widest alignment both pointers share decides the packet type
template <int A> struct __attribute__((packed, aligned(A))) Packet { u32x4 q; };
constexpr int kBlock = 256;
constexpr int kU = 4;

template <int A>
__global__ void __launch_bounds__(kBlock) copy_kernel(uint8_t* dst, const uint8_t* src, uint64_t nbytes) {
    using Raw16B = Packet<A>;
    const uint64_t P = nbytes / 16;
    const uint64_t span = (uint64_t)kU * kBlock;
    for (uint64_t base = (uint64_t)blockIdx.x * span; base < P; base += (uint64_t)gridDim.x * span) {
        if (base + span <= P) {
            u32x4 v[kU];
#pragma unroll
            for (int u = 0; u < kU; ++u)
                v[u] = reinterpret_cast<const Raw16B*>(src + (base + (uint64_t)u * kBlock + threadIdx.x) * 16)->q;
#pragma unroll
            for (int u = 0; u < kU; ++u)
                reinterpret_cast<Raw16B*>(dst + (base + (uint64_t)u * kBlock + threadIdx.x) * 16)->q = v[u];
        } else {
            for (uint64_t p = base + threadIdx.x; p < P; p += kBlock) {
                u32x4 v = reinterpret_cast<const Raw16B*>(src + p * 16)->q;
                reinterpret_cast<Raw16B*>(dst + p * 16)->q = v;
            }
        }
    }
    if (blockIdx.x == 0) {
        uint64_t i = P * 16 + threadIdx.x;
        if (i < nbytes) dst[i] = src[i];
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
