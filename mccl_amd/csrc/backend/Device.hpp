// Device.hpp -- the four things the backend asks of the device runtime, in one place:
// which GPU the calling thread uses, the stream it produces and consumes tensors on, raw
// device memory for scratch buffers, and whether a tensor lives on the GPU.  (The
// reference gets the same from csrc/metal/MPSInterop: its MPS stream, its shared-storage
// buffers, check_mps_.)
//
// -DMCCL_NULL_DEVICE swaps in a host stand-in -- GPU 0, the null stream, host memory, every
// tensor accepted -- so that the group, Work and completion logic can be compiled without a
// HIP runtime and run under ThreadSanitizer / AddressSanitizer against a stand-in of the C
// ABI (tests/native/pg_stress.cpp).  The shipped extension is never built that way.
#pragma once

#include <ATen/ATen.h>

#ifndef MCCL_NULL_DEVICE
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#endif

namespace mccl {
namespace dev {

#ifndef MCCL_NULL_DEVICE
inline int current_device() { return static_cast<int>(c10::hip::current_device()); }
inline void* current_stream(int device) {
    return static_cast<void*>(c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(device)).stream());
}
inline at::Tensor empty_bytes(int64_t nbytes, int device) {
    return at::empty({nbytes}, at::TensorOptions().dtype(at::kByte).device(at::kCUDA, device));
}
inline bool on_device(const at::Tensor& t) { return t.is_cuda(); }
#else
inline int current_device() { return 0; }
inline void* current_stream(int) { return nullptr; }
inline at::Tensor empty_bytes(int64_t nbytes, int) { return at::empty({nbytes}, at::TensorOptions().dtype(at::kByte)); }
inline bool on_device(const at::Tensor&) { return true; }
#endif

}  // namespace dev
}  // namespace mccl
