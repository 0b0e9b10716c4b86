// Device allocators of the kuiper host API: host memory through malloc, GPU memory through
// hipMalloc.  Interface, defaults and the lazily created shared singletons follow
// kuiper/include/base/alloc.h:8-64 of the reference; the GPU side talks to the HIP runtime.
#ifndef KUIPER_INCLUDE_BASE_ALLOC_H
#define KUIPER_INCLUDE_BASE_ALLOC_H

#include <memory>

#include "base/base.h"

namespace base {

enum class MemcpyKind {
    MemcpyCPU2CPU = 0,
    MemcpyCPU2CUDA = 1,
    MemcpyCUDA2CPU = 2,
    MemcpyCUDA2CUDA = 3,
};

class DeviceAllocator {
public:
    explicit DeviceAllocator(DeviceType device_type) : device_type_(device_type) {}
    virtual ~DeviceAllocator() = default;
    virtual DeviceType device_type() const { return device_type_; }
    virtual void* allocate(size_t byte_size) const = 0;
    virtual void release(void* ptr) const = 0;
    // Copies byte_size bytes.  With a stream the GPU copies are asynchronous on that stream,
    // without one they block; need_sync adds a device-wide synchronisation afterwards.
    virtual void memcpy(void* dest_ptr, const void* src_ptr, size_t byte_size,
                        MemcpyKind memcpy_kind = MemcpyKind::MemcpyCPU2CPU, void* stream = nullptr,
                        bool need_sync = false) const;
    virtual void memset_zero(void* ptr, size_t byte_size, void* stream, bool need_sync = false);

private:
    DeviceType device_type_ = DeviceType::DeviceUnknown;
};

class CPUDeviceAllocator : public DeviceAllocator {
public:
    explicit CPUDeviceAllocator();
    void* allocate(size_t byte_size) const override;
    void release(void* ptr) const override;
};

// GPU memory with a free-block pool.  release() keeps the block; allocate() takes the smallest idle
// block that fits without wasting more than half of it, else calls hipMalloc.  hipMalloc and
// hipFree cost tens of microseconds to milliseconds and hipFree waits for the device, which a
// decode loop that creates tensors per step cannot afford; the reference does one cudaMalloc and
// one cudaFree per buffer (kuiper/source/base/alloc_cu.cpp:8-23).  Blocks are handed out again in
// program order, so work that still uses a released block must be on the stream that the next
// user launches on, or finished (the rule of any caching allocator).
class CUDADeviceAllocator : public DeviceAllocator {
public:
    struct PoolStats {
        size_t device_allocations = 0;  // hipMalloc calls
        size_t device_frees = 0;        // hipFree calls
        size_t reuses = 0;              // allocate() calls served from the pool
        size_t idle_bytes = 0;          // bytes held in idle blocks
        size_t busy_bytes = 0;          // bytes handed out
    };

    explicit CUDADeviceAllocator();
    ~CUDADeviceAllocator() override;
    void* allocate(size_t byte_size) const override;
    void release(void* ptr) const override;

    // Idle blocks beyond this many bytes are returned to the device, largest first (default 1 GiB;
    // 0 switches pooling off: every release is a hipFree, as in the reference).
    void set_idle_limit(size_t bytes);
    void trim();  // returns every idle block to the device
    PoolStats stats() const;

private:
    struct Pool;
    std::unique_ptr<Pool> pool_;
};

// One shared allocator per kind, created on first use (not synchronised: the host API is
// single-threaded, as in the reference).
class CPUDeviceAllocatorFactory {
public:
    static std::shared_ptr<CPUDeviceAllocator> get_instance() {
        if (instance == nullptr) {
            instance = std::make_shared<CPUDeviceAllocator>();
        }
        return instance;
    }

private:
    static std::shared_ptr<CPUDeviceAllocator> instance;
};

class CUDADeviceAllocatorFactory {
public:
    static std::shared_ptr<CUDADeviceAllocator> get_instance() {
        if (instance == nullptr) {
            instance = std::make_shared<CUDADeviceAllocator>();
        }
        return instance;
    }

private:
    static std::shared_ptr<CUDADeviceAllocator> instance;
};

}  // namespace base

#endif  // KUIPER_INCLUDE_BASE_ALLOC_H
