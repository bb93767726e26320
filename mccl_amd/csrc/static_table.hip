// static_table.hip -- a descriptor table in static device memory, for the one
// entry point that must not allocate (mcclx_fold_batched_noalloc).
//
// The table of a batched fold normally lives in a device buffer the context
// allocates on demand.  Callers that cannot allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc) get the same launch
// with the table in `scratch` below: a file-scope device array, one copy per
// GPU, held until the process ends.  Descriptors reach it through the kernel
// arguments of a small writer kernel, so the whole call is kernel launches
// only -- no memcpy, no memset, nothing a graph would replay wrongly.
//
// In host code the array's name is a stand-in, not a device address: every use
// goes through the per-device pointer hipGetSymbolAddress returns.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "fold_launch.h"

namespace mcclx {
namespace {

static __device__ __align__(256) unsigned char scratch[kStaticTableBytes];

constexpr int kMaxDevices = 64;
std::mutex g_mu;
void* g_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once resolved

struct Words {
    uint64_t w[kUploadWords];
};

// dst[i] = a.w[i] for i < n: the payload travels in the kernel arguments.
__global__ void __launch_bounds__(kUploadWords) table_write_kernel(Words a, uint64_t* __restrict__ dst, uint32_t n) {
    const uint32_t i = threadIdx.x;
    if (i < n) dst[i] = a.w[i];
}

}  // namespace

hipError_t static_table_resolve(int device, void** out) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_ptr[device]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // for the current device
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_ptr[device] = p;
    }
    *out = g_ptr[device];
    return hipSuccess;
}

hipError_t launch_table_write(hipStream_t st, void* dst_words, const uint64_t* words, uint32_t n) {
    if (n == 0) return hipSuccess;
    if (n > kUploadWords) return hipErrorInvalidValue;
    Words a;
    for (uint32_t i = 0; i < n; ++i) a.w[i] = words[i];
    for (uint32_t i = n; i < kUploadWords; ++i) a.w[i] = 0;
    table_write_kernel<<<dim3(1), dim3(kUploadWords), 0, st>>>(a, static_cast<uint64_t*>(dst_words), n);
    return hipGetLastError();
}

}  // namespace mcclx
