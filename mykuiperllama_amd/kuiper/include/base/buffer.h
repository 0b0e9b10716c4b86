// A run of bytes on one device, either owned (allocated through a DeviceAllocator and released
// with the Buffer) or borrowed (external pointer, never released).  Mirrors
// kuiper/include/base/buffer.h:17-45.
#ifndef KUIPER_INCLUDE_BASE_BUFFER_H
#define KUIPER_INCLUDE_BASE_BUFFER_H

#include "base/alloc.h"

namespace base {

// enable_shared_from_this is a private base, as in the reference (buffer.h:17): a Buffer is
// never handed out through get_shared_from_this() by the library itself.
class Buffer : public NoCopyable, std::enable_shared_from_this<Buffer> {
public:
    explicit Buffer() = default;
    // ptr == nullptr with an allocator: allocate byte_size bytes and own them.
    // ptr != nullptr: wrap it; the device type stays DeviceUnknown until set_device_type().
    explicit Buffer(size_t byte_size, std::shared_ptr<DeviceAllocator> allocator = nullptr,
                    void* ptr = nullptr, bool use_external = false);
    virtual ~Buffer();

    bool allocate();
    // Copies min(byte_size(), other.byte_size()) bytes; both device types must be known and this
    // buffer needs an allocator (it performs the copy).
    void copy_from(const Buffer& buffer) const;
    void copy_from(const Buffer* buffer) const;

    void* ptr();
    const void* ptr() const;
    size_t byte_size() const;
    std::shared_ptr<DeviceAllocator> allocator() const;
    DeviceType device_type() const;
    void set_device_type(DeviceType device_type);
    std::shared_ptr<Buffer> get_shared_from_this();
    bool is_external() const;

private:
    size_t byte_size_ = 0;
    void* ptr_ = nullptr;
    bool use_external_ = false;
    DeviceType device_type_ = DeviceType::DeviceUnknown;
    std::shared_ptr<DeviceAllocator> allocator_;
};

}  // namespace base

#endif  // KUIPER_INCLUDE_BASE_BUFFER_H
