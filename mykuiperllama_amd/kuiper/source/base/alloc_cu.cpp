// GPU allocator with a pool of idle blocks (see base/alloc.h).  A failed allocation is fatal, as
// in the reference (kuiper/source/base/alloc_cu.cpp:13-18); before giving up the pool is emptied
// and the allocation tried once more.
#include <hip/hip_runtime_api.h>

#include <map>
#include <unordered_map>

#include "base/alloc.h"

namespace base {

struct CUDADeviceAllocator::Pool {
    std::multimap<size_t, void*> idle;          // block size -> block
    std::unordered_map<void*, size_t> busy;     // block -> block size
    size_t idle_limit = size_t(1) << 30;
    PoolStats stats;

    void free_block(void* ptr, size_t bytes) {
        (void)hipFree(ptr);
        stats.device_frees++;
        stats.idle_bytes -= bytes;
    }
    void shrink_to(size_t limit) {
        while (stats.idle_bytes > limit && !idle.empty()) {
            auto largest = std::prev(idle.end());
            void* ptr = largest->second;
            const size_t bytes = largest->first;
            idle.erase(largest);
            free_block(ptr, bytes);
        }
    }
};

namespace {
// Blocks are multiples of 256 bytes: what the GEMV workspace and 16-byte vector loads ask of a base
// address holds for every block, and sizes that differ by a few bytes share blocks.
size_t round_up(size_t bytes) {
    return (bytes + 255) & ~size_t(255);
}
}  // namespace

CUDADeviceAllocator::CUDADeviceAllocator() : DeviceAllocator(DeviceType::DeviceCUDA), pool_(new Pool) {}

CUDADeviceAllocator::~CUDADeviceAllocator() {
    // The shared instance lives until the process ends, when the HIP runtime may already be gone:
    // idle blocks are left to the driver.
}

void* CUDADeviceAllocator::allocate(size_t byte_size) const {
    if (byte_size == 0) {
        return nullptr;
    }
    Pool& pool = *pool_;
    const size_t want = round_up(byte_size);
    auto fit = pool.idle.lower_bound(want);
    if (fit != pool.idle.end() && fit->first <= 2 * want) {
        void* ptr = fit->second;
        const size_t bytes = fit->first;
        pool.idle.erase(fit);
        pool.busy[ptr] = bytes;
        pool.stats.idle_bytes -= bytes;
        pool.stats.busy_bytes += bytes;
        pool.stats.reuses++;
        return ptr;
    }
    void* ptr = nullptr;
    hipError_t err = hipMalloc(&ptr, want);
    if (err != hipSuccess) {
        (void)hipGetLastError();
        pool.shrink_to(0);
        err = hipMalloc(&ptr, want);
    }
    CHECK_EQ(err, hipSuccess) << "hipMalloc of " << want << " bytes: " << hipGetErrorString(err);
    pool.stats.device_allocations++;
    pool.busy[ptr] = want;
    pool.stats.busy_bytes += want;
    return ptr;
}

void CUDADeviceAllocator::release(void* ptr) const {
    if (ptr == nullptr) {
        return;
    }
    Pool& pool = *pool_;
    auto it = pool.busy.find(ptr);
    if (it == pool.busy.end()) {
        // not handed out by this allocator: pass it to the runtime, as the reference does with
        // every pointer
        (void)hipFree(ptr);
        pool.stats.device_frees++;
        return;
    }
    const size_t bytes = it->second;
    pool.busy.erase(it);
    pool.stats.busy_bytes -= bytes;
    pool.idle.emplace(bytes, ptr);
    pool.stats.idle_bytes += bytes;
    pool.shrink_to(pool.idle_limit);
}

void CUDADeviceAllocator::set_idle_limit(size_t bytes) {
    pool_->idle_limit = bytes;
    pool_->shrink_to(bytes);
}

void CUDADeviceAllocator::trim() {
    pool_->shrink_to(0);
}

CUDADeviceAllocator::PoolStats CUDADeviceAllocator::stats() const {
    return pool_->stats;
}

std::shared_ptr<CUDADeviceAllocator> CUDADeviceAllocatorFactory::instance = nullptr;

}  // namespace base
