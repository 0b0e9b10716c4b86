// The pooled GPU allocator behind base::CUDADeviceAllocator: blocks come back from the pool instead
// of the device, within the limits the header states.
#include <hip/hip_runtime_api.h>

#include <vector>

#include "base/alloc.h"
#include "base/buffer.h"
#include "mini_test.h"
#include "tensor/tensor.h"

namespace {
using Stats = base::CUDADeviceAllocator::PoolStats;
}

TEST_GPU(test_alloc, released_blocks_are_reused) {
    base::CUDADeviceAllocator alloc;
    void* a = alloc.allocate(1000);
    ASSERT_TRUE(a != nullptr);
    ASSERT_EQ(reinterpret_cast<uintptr_t>(a) % 256, uintptr_t(0));
    alloc.release(a);
    Stats s = alloc.stats();
    ASSERT_EQ(s.device_allocations, size_t(1));
    ASSERT_EQ(s.device_frees, size_t(0));
    ASSERT_EQ(s.idle_bytes, size_t(1024));
    void* b = alloc.allocate(900);  // fits the 1024-byte block and wastes less than half of it
    ASSERT_EQ(b, a);
    s = alloc.stats();
    ASSERT_EQ(s.device_allocations, size_t(1));
    ASSERT_EQ(s.reuses, size_t(1));
    ASSERT_EQ(s.busy_bytes, size_t(1024));
    void* c = alloc.allocate(900);  // the pool is empty now
    ASSERT_TRUE(c != b);
    alloc.release(b);
    void* d = alloc.allocate(256);  // a quarter of the idle block: not taken from it
    ASSERT_TRUE(d != b);
    alloc.release(c);
    alloc.release(d);
    alloc.trim();
    s = alloc.stats();
    ASSERT_EQ(s.idle_bytes, size_t(0));
    ASSERT_EQ(s.busy_bytes, size_t(0));
    ASSERT_EQ(s.device_frees, s.device_allocations);
}

TEST_GPU(test_alloc, idle_limit_bounds_the_pool) {
    base::CUDADeviceAllocator alloc;
    alloc.set_idle_limit(1 << 20);
    std::vector<void*> blocks;
    for (int i = 0; i < 4; i++) blocks.push_back(alloc.allocate(512 << 10));
    for (void* p : blocks) alloc.release(p);
    Stats s = alloc.stats();
    ASSERT_LE(s.idle_bytes, size_t(1 << 20));
    ASSERT_EQ(s.device_frees, size_t(2));
    alloc.set_idle_limit(0);  // pooling off: a release goes straight back to the device
    s = alloc.stats();
    ASSERT_EQ(s.idle_bytes, size_t(0));
    void* p = alloc.allocate(4096);
    alloc.release(p);
    ASSERT_EQ(alloc.stats().idle_bytes, size_t(0));
    ASSERT_EQ(alloc.stats().device_frees, alloc.stats().device_allocations);
}

TEST_GPU(test_alloc, a_loop_of_tensors_stops_calling_the_device) {
    auto alloc = base::CUDADeviceAllocatorFactory::get_instance();
    // what a decode loop that builds its activations per step does
    for (int step = 0; step < 3; step++) {
        tensor::Tensor x(base::DataType::DataTypeBf16, 4096, true, alloc);
        tensor::Tensor y(base::DataType::DataTypeBf16, 12288, true, alloc);
        ASSERT_TRUE(x.ptr<uint16_t>() != nullptr && y.ptr<uint16_t>() != nullptr);
    }
    const size_t before = alloc->stats().device_allocations;
    for (int step = 0; step < 50; step++) {
        tensor::Tensor x(base::DataType::DataTypeBf16, 4096, true, alloc);
        tensor::Tensor y(base::DataType::DataTypeBf16, 12288, true, alloc);
        ASSERT_EQ(hipMemset(x.ptr<uint16_t>(), 0, x.byte_size()), hipSuccess);
    }
    ASSERT_EQ(alloc->stats().device_allocations, before);
}

TEST_GPU(test_alloc, foreign_pointers_are_passed_to_the_runtime) {
    base::CUDADeviceAllocator alloc;
    void* p = nullptr;
    ASSERT_EQ(hipMalloc(&p, 4096), hipSuccess);
    alloc.release(p);
    ASSERT_EQ(alloc.stats().device_frees, size_t(1));
    ASSERT_EQ(alloc.stats().idle_bytes, size_t(0));
    alloc.release(nullptr);
    ASSERT_TRUE(alloc.allocate(0) == nullptr);
}
