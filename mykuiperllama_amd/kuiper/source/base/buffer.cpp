// Buffer: ownership and device-to-device copies (reference: kuiper/source/base/buffer.cpp:4-103).
#include "base/buffer.h"

#include <algorithm>

namespace base {
namespace {

// Any pair that is not CPU/CPU, CPU/GPU or GPU/CPU is treated as GPU/GPU (reference
// buffer.cpp:35-49).
MemcpyKind copy_kind(DeviceType src, DeviceType dst) {
    const bool src_cpu = src == DeviceType::DeviceCPU;
    const bool dst_cpu = dst == DeviceType::DeviceCPU;
    if (src_cpu && dst_cpu) return MemcpyKind::MemcpyCPU2CPU;
    if (src_cpu && dst == DeviceType::DeviceCUDA) return MemcpyKind::MemcpyCPU2CUDA;
    if (src == DeviceType::DeviceCUDA && dst_cpu) return MemcpyKind::MemcpyCUDA2CPU;
    return MemcpyKind::MemcpyCUDA2CUDA;
}

}  // namespace

Buffer::Buffer(size_t byte_size, std::shared_ptr<DeviceAllocator> allocator, void* ptr, bool use_external)
    : byte_size_(byte_size), ptr_(ptr), use_external_(use_external), allocator_(std::move(allocator)) {
    if (ptr_ == nullptr && allocator_ != nullptr) {
        device_type_ = allocator_->device_type();
        use_external_ = false;
        ptr_ = allocator_->allocate(byte_size_);
    }
}

Buffer::~Buffer() {
    if (!use_external_ && ptr_ != nullptr && allocator_ != nullptr) {
        allocator_->release(ptr_);
        ptr_ = nullptr;
    }
}

bool Buffer::allocate() {
    if (allocator_ == nullptr || byte_size_ == 0) {
        return false;
    }
    use_external_ = false;
    ptr_ = allocator_->allocate(byte_size_);
    return ptr_ != nullptr;
}

void Buffer::copy_from(const Buffer& buffer) const {
    copy_from(&buffer);
}

void Buffer::copy_from(const Buffer* buffer) const {
    CHECK(allocator_ != nullptr);
    CHECK(buffer != nullptr && buffer->ptr_ != nullptr);
    const DeviceType dst = device_type_;
    const DeviceType src = buffer->device_type_;
    CHECK(src != DeviceType::DeviceUnknown && dst != DeviceType::DeviceUnknown);
    allocator_->memcpy(ptr_, buffer->ptr_, std::min(byte_size_, buffer->byte_size_), copy_kind(src, dst));
}

void* Buffer::ptr() { return ptr_; }
const void* Buffer::ptr() const { return ptr_; }
size_t Buffer::byte_size() const { return byte_size_; }
std::shared_ptr<DeviceAllocator> Buffer::allocator() const { return allocator_; }
DeviceType Buffer::device_type() const { return device_type_; }
void Buffer::set_device_type(DeviceType device_type) { device_type_ = device_type; }
std::shared_ptr<Buffer> Buffer::get_shared_from_this() { return shared_from_this(); }
bool Buffer::is_external() const { return use_external_; }

}  // namespace base
