// GPU allocator: one hipMalloc per buffer, no pooling (reference: kuiper/source/base/alloc_cu.cpp:8-23,
// which does one cudaMalloc per buffer).  A failed allocation is fatal, as there.
#include <hip/hip_runtime_api.h>

#include "base/alloc.h"

namespace base {

CUDADeviceAllocator::CUDADeviceAllocator() : DeviceAllocator(DeviceType::DeviceCUDA) {}

void* CUDADeviceAllocator::allocate(size_t byte_size) const {
    if (byte_size == 0) {
        return nullptr;
    }
    void* ptr = nullptr;
    hipError_t err = hipMalloc(&ptr, byte_size);
    CHECK_EQ(err, hipSuccess) << "hipMalloc of " << byte_size << " bytes: " << hipGetErrorString(err);
    return ptr;
}

void CUDADeviceAllocator::release(void* ptr) const {
    if (ptr != nullptr) {
        (void)hipFree(ptr);
    }
}

std::shared_ptr<CUDADeviceAllocator> CUDADeviceAllocatorFactory::instance = nullptr;

}  // namespace base
