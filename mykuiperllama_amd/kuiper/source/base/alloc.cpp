// memcpy / memset_zero shared by both allocators (reference: kuiper/source/base/alloc.cpp:6-74).
#include "base/alloc.h"

#include <hip/hip_runtime_api.h>

#include <cstring>

namespace base {
namespace {

// The reference ignores the runtime's return codes here; this build reports them and carries on.
void report(hipError_t err, const char* what) {
    if (err != hipSuccess) {
        LOG(ERROR) << what << " failed: " << hipGetErrorString(err);
    }
}

hipMemcpyKind to_hip(MemcpyKind kind) {
    switch (kind) {
        case MemcpyKind::MemcpyCPU2CUDA: return hipMemcpyHostToDevice;
        case MemcpyKind::MemcpyCUDA2CPU: return hipMemcpyDeviceToHost;
        default: return hipMemcpyDeviceToDevice;
    }
}

}  // namespace

void DeviceAllocator::memcpy(void* dest_ptr, const void* src_ptr, size_t byte_size,
                             MemcpyKind memcpy_kind, void* stream, bool need_sync) const {
    CHECK_NE(dest_ptr, nullptr);
    CHECK_NE(src_ptr, nullptr);
    if (byte_size == 0) {
        return;
    }
    switch (memcpy_kind) {
        case MemcpyKind::MemcpyCPU2CPU:
            std::memcpy(dest_ptr, src_ptr, byte_size);
            break;
        case MemcpyKind::MemcpyCPU2CUDA:
        case MemcpyKind::MemcpyCUDA2CPU:
        case MemcpyKind::MemcpyCUDA2CUDA:
            if (stream == nullptr) {
                report(hipMemcpy(dest_ptr, src_ptr, byte_size, to_hip(memcpy_kind)), "hipMemcpy");
            } else {
                report(hipMemcpyAsync(dest_ptr, src_ptr, byte_size, to_hip(memcpy_kind),
                                      static_cast<hipStream_t>(stream)),
                       "hipMemcpyAsync");
            }
            break;
        default:
            LOG(FATAL) << "Unknown memcpy kind: " << int(memcpy_kind);
    }
    if (need_sync) {
        report(hipDeviceSynchronize(), "hipDeviceSynchronize");
    }
}

void DeviceAllocator::memset_zero(void* ptr, size_t byte_size, void* stream, bool need_sync) {
    CHECK(device_type_ != DeviceType::DeviceUnknown);
    if (device_type_ == DeviceType::DeviceCPU) {
        std::memset(ptr, 0, byte_size);
    } else if (stream == nullptr) {
        report(hipMemset(ptr, 0, byte_size), "hipMemset");
    } else {
        report(hipMemsetAsync(ptr, 0, byte_size, static_cast<hipStream_t>(stream)), "hipMemsetAsync");
    }
    if (need_sync) {
        report(hipDeviceSynchronize(), "hipDeviceSynchronize");
    }
}

}  // namespace base
