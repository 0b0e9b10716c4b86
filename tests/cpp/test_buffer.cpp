// Buffer semantics.  Restates the assertions of the reference's test/test_tensor/test_buffer.cpp
// (cases allocate :7-28, use_external :30-38, cuda_memory1/2/3 :40-114) on this build's classes.
#include <hip/hip_runtime_api.h>

#include <vector>

#include "base/buffer.h"
#include "mini_test.h"
#include "utils.h"

using namespace base;

TEST_CPU(test_buffer, allocate_cpu) {
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    Buffer buffer(32, allocator);
    ASSERT_NE(buffer.ptr(), nullptr);
    ASSERT_EQ(buffer.byte_size(), 32u);
    ASSERT_EQ(buffer.is_external(), false);
    ASSERT_EQ(buffer.allocator(), allocator);
    ASSERT_TRUE(buffer.device_type() == DeviceType::DeviceCPU);
    buffer.set_device_type(DeviceType::DeviceCUDA);
    ASSERT_TRUE(buffer.device_type() == DeviceType::DeviceCUDA);
    ASSERT_EQ(CPUDeviceAllocatorFactory::get_instance(), allocator);  // one shared instance
}

TEST_GPU(test_buffer, allocate_cuda) {
    auto allocator_cu = CUDADeviceAllocatorFactory::get_instance();
    Buffer buffer_cu(32, allocator_cu);
    ASSERT_NE(buffer_cu.ptr(), nullptr);
    ASSERT_EQ(buffer_cu.byte_size(), 32u);
    ASSERT_EQ(buffer_cu.is_external(), false);
    ASSERT_EQ(buffer_cu.allocator(), allocator_cu);
    ASSERT_TRUE(buffer_cu.device_type() == DeviceType::DeviceCUDA);
}

TEST_CPU(test_buffer, use_external) {
    std::vector<float> storage(32);
    Buffer buffer(32, nullptr, storage.data(), true);
    ASSERT_EQ(buffer.is_external(), true);
    ASSERT_EQ(buffer.byte_size(), 32u);
    ASSERT_EQ(buffer.ptr(), static_cast<void*>(storage.data()));
    // a wrapped pointer has no device until one is set
    ASSERT_TRUE(buffer.device_type() == DeviceType::DeviceUnknown);
}

TEST_CPU(test_buffer, wrapped_pointer_with_allocator_keeps_unknown_device) {
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    void* mem = allocator->allocate(64);
    {
        Buffer owned(64, allocator, mem, false);  // owns mem, releases it through the allocator
        ASSERT_TRUE(owned.device_type() == DeviceType::DeviceUnknown);
        ASSERT_EQ(owned.is_external(), false);
    }
}

TEST_CPU(test_buffer, copy_from_cpu_to_cpu_takes_the_smaller_size) {
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    Buffer src(8 * sizeof(float), allocator), dst(4 * sizeof(float), allocator);
    for (int i = 0; i < 8; i++) static_cast<float*>(src.ptr())[i] = float(i + 1);
    dst.copy_from(src);
    for (int i = 0; i < 4; i++) ASSERT_EQ(static_cast<float*>(dst.ptr())[i], float(i + 1));
    Buffer big(16 * sizeof(float), allocator);
    for (int i = 0; i < 16; i++) static_cast<float*>(big.ptr())[i] = -1.f;
    big.copy_from(&src);
    ASSERT_EQ(static_cast<float*>(big.ptr())[7], 8.f);
    ASSERT_EQ(static_cast<float*>(big.ptr())[8], -1.f);
}

TEST_CPU(test_buffer, copy_from_checks) {
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    std::vector<float> storage(4, 1.f);
    Buffer borrowed(16, nullptr, storage.data(), true);  // no allocator, unknown device
    Buffer owned(16, allocator);
    ASSERT_FATAL(borrowed.copy_from(owned));  // the destination performs the copy: needs an allocator
    ASSERT_FATAL(owned.copy_from(borrowed));  // source device unknown
    borrowed.set_device_type(DeviceType::DeviceCPU);
    owned.copy_from(borrowed);
    ASSERT_EQ(static_cast<float*>(owned.ptr())[3], 1.f);
    Buffer empty;
    ASSERT_EQ(empty.allocate(), false);
    ASSERT_FATAL(owned.copy_from(empty));  // null source pointer
}

TEST_CPU(test_buffer, zero_size_allocation_is_null) {
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    ASSERT_EQ(allocator->allocate(0), nullptr);
    allocator->release(nullptr);
    Buffer b(0, allocator);
    ASSERT_EQ(b.ptr(), nullptr);
}

TEST_GPU(test_buffer, cuda_memory1) {
    auto allocator_cu = CUDADeviceAllocatorFactory::get_instance();
    const int32_t size = 32;
    std::vector<float> host(size);
    for (int32_t i = 0; i < size; i++) host[i] = float(i);
    Buffer buffer(size * sizeof(float), nullptr, host.data(), true);
    buffer.set_device_type(DeviceType::DeviceCPU);
    ASSERT_EQ(buffer.is_external(), true);
    Buffer buffer_cu(size * sizeof(float), allocator_cu);
    buffer_cu.copy_from(buffer);
    std::vector<float> back(size, -1.f);
    allocator_cu->memcpy(back.data(), buffer_cu.ptr(), size * sizeof(float), MemcpyKind::MemcpyCUDA2CPU);
    for (int32_t i = 0; i < size; i++) ASSERT_EQ(back[i], host[i]);
}

TEST_GPU(test_buffer, cuda_memory2) {
    auto allocator_cu = CUDADeviceAllocatorFactory::get_instance();
    const int32_t size = 32;
    Buffer buffer_cu1(size * sizeof(float), allocator_cu);
    Buffer buffer_cu2(size * sizeof(float), allocator_cu);
    ASSERT_TRUE(buffer_cu1.device_type() == DeviceType::DeviceCUDA);
    ASSERT_TRUE(buffer_cu2.device_type() == DeviceType::DeviceCUDA);
    set_value_cu(static_cast<float*>(buffer_cu1.ptr()), size, 1.f);
    buffer_cu2.copy_from(buffer_cu1);
    std::vector<float> back(size, 0.f);
    ASSERT_EQ(hipMemcpy(back.data(), buffer_cu2.ptr(), size * sizeof(float), hipMemcpyDeviceToHost), hipSuccess);
    for (int32_t i = 0; i < size; i++) ASSERT_EQ(back[i], 1.f);
}

TEST_GPU(test_buffer, cuda_memory3) {
    auto allocator_cu = CUDADeviceAllocatorFactory::get_instance();
    auto allocator = CPUDeviceAllocatorFactory::get_instance();
    const int32_t size = 32;
    Buffer buffer_cu(size * sizeof(float), allocator_cu);
    Buffer buffer(size * sizeof(float), allocator);
    ASSERT_TRUE(buffer_cu.device_type() == DeviceType::DeviceCUDA);
    ASSERT_TRUE(buffer.device_type() == DeviceType::DeviceCPU);
    set_value_cu(static_cast<float*>(buffer_cu.ptr()), size, 1.f);
    buffer.copy_from(buffer_cu);
    const float* p = static_cast<const float*>(buffer.ptr());
    for (int32_t i = 0; i < size; i++) ASSERT_EQ(p[i], 1.f);
}

TEST_GPU(test_buffer, memset_zero_and_async_copy) {
    auto allocator_cu = CUDADeviceAllocatorFactory::get_instance();
    const int32_t size = 1000;
    Buffer buffer_cu(size * sizeof(float), allocator_cu);
    set_value_cu(static_cast<float*>(buffer_cu.ptr()), size, 3.f);
    hipStream_t stream;
    ASSERT_EQ(hipStreamCreate(&stream), hipSuccess);
    allocator_cu->memset_zero(buffer_cu.ptr(), size * sizeof(float), stream, true);
    std::vector<float> back(size, 7.f);
    allocator_cu->memcpy(back.data(), buffer_cu.ptr(), size * sizeof(float), MemcpyKind::MemcpyCUDA2CPU, stream, true);
    for (int32_t i = 0; i < size; i++) ASSERT_EQ(back[i], 0.f);
    ASSERT_EQ(hipStreamDestroy(stream), hipSuccess);
}
