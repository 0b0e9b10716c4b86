// Host allocator: plain malloc / free (reference: kuiper/source/base/alloc_cpu.cpp:7-20).
#include <cstdlib>

#include "base/alloc.h"

namespace base {

CPUDeviceAllocator::CPUDeviceAllocator() : DeviceAllocator(DeviceType::DeviceCPU) {}

void* CPUDeviceAllocator::allocate(size_t byte_size) const {
    return byte_size == 0 ? nullptr : std::malloc(byte_size);
}

void CPUDeviceAllocator::release(void* ptr) const {
    if (ptr != nullptr) {
        std::free(ptr);
    }
}

std::shared_ptr<CPUDeviceAllocator> CPUDeviceAllocatorFactory::instance = nullptr;

}  // namespace base
