// Tensor behaviour (reference: kuiper/source/tensor/tensor.cpp:6-254).
#include "tensor/tensor.h"

#include <utility>

namespace tensor {
namespace {

// Product of the dims; an empty list has zero elements (reference tensor.cpp:6-13).
size_t element_count(const std::vector<int32_t>& dims) {
    if (dims.empty()) {
        return 0;
    }
    size_t n = 1;
    for (int32_t d : dims) {
        n *= static_cast<size_t>(d);
    }
    return n;
}

}  // namespace

Tensor::Tensor(base::DataType data_type, int32_t dim0, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : dims_{dim0}, data_type_(data_type) {
    size_ = element_count(dims_);
    init_buffer(std::move(allocator), need_alloc, ptr);
}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : dims_{dim0, dim1}, data_type_(data_type) {
    size_ = element_count(dims_);
    init_buffer(std::move(allocator), need_alloc, ptr);
}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, int32_t dim2, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : dims_{dim0, dim1, dim2}, data_type_(data_type) {
    size_ = element_count(dims_);
    init_buffer(std::move(allocator), need_alloc, ptr);
}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, int32_t dim2, int32_t dim3,
               bool need_alloc, std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : dims_{dim0, dim1, dim2, dim3}, data_type_(data_type) {
    size_ = element_count(dims_);
    init_buffer(std::move(allocator), need_alloc, ptr);
}

Tensor::Tensor(base::DataType data_type, std::vector<int32_t> dims, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : dims_(std::move(dims)), data_type_(data_type) {
    size_ = element_count(dims_);
    init_buffer(std::move(allocator), need_alloc, ptr);
}

void Tensor::init_buffer(std::shared_ptr<base::DeviceAllocator> allocator, bool need_alloc, void* ptr) {
    if (allocator == nullptr) {
        // no allocator: the tensor can only borrow memory
        CHECK_NE(ptr, nullptr);
        CHECK_EQ(need_alloc, false);
        buffer_ = std::make_shared<base::Buffer>(byte_size(), nullptr, ptr, true);
        return;
    }
    if (need_alloc) {
        allocate(allocator, false);
    } else if (ptr != nullptr) {
        buffer_ = std::make_shared<base::Buffer>(byte_size(), allocator, ptr, false);
    } else {
        allocate(allocator, true);  // an allocator without a pointer allocates all the same
    }
}

bool Tensor::allocate(std::shared_ptr<base::DeviceAllocator> allocator, bool need_realloc) {
    if (allocator == nullptr) {
        LOG(ERROR) << "The allocator parameter in the allocate function is null pointer!";
        return false;
    }
    const size_t bytes = byte_size();
    if (bytes == 0) {
        LOG(ERROR) << "The byte_size parameter in the allocate function is equal to zero!";
        return false;
    }
    if (buffer_ && bytes <= buffer_->byte_size() && !need_realloc) {
        return true;  // the present buffer is large enough
    }
    buffer_ = std::make_shared<base::Buffer>(bytes, allocator, nullptr);
    if (buffer_->ptr() == nullptr) {
        LOG(ERROR) << "The memory allocated is a null pointer!";
        return false;
    }
    return true;
}

bool Tensor::assgin(std::shared_ptr<base::Buffer> buffer) {
    if (buffer == nullptr) {
        LOG(ERROR) << "The buffer parameter in the assign function is null pointer!";
        return false;
    }
    if (buffer_ && buffer_->device_type() != buffer->device_type()) {
        // reported, not refused
        LOG(ERROR) << "The device type of the new buffer is different from the original one.";
    }
    if (buffer->byte_size() < byte_size()) {
        LOG(ERROR) << "The size of buffer is too small for the tensor!";
        return false;
    }
    buffer_ = std::move(buffer);
    return true;
}

void Tensor::to_cpu() {
    CHECK_NE(buffer_, nullptr);
    const base::DeviceType where = device_type();
    if (where == base::DeviceType::DeviceCUDA) {
        const size_t bytes = byte_size();
        auto host_alloc = base::CPUDeviceAllocatorFactory::get_instance();
        auto host_buffer = std::make_shared<base::Buffer>(bytes, host_alloc);
        host_alloc->memcpy(host_buffer->ptr(), buffer_->ptr(), bytes, base::MemcpyKind::MemcpyCUDA2CPU);
        buffer_ = host_buffer;
    } else if (where == base::DeviceType::DeviceCPU) {
        LOG(INFO) << "The device type of the tensor is already cpu.";
    } else {
        LOG(ERROR) << "The device type of the tensor is unknown.";
    }
}

void Tensor::to_cuda(hipStream_t stream) {
    UNUSED(stream);  // the reference ignores it too and copies synchronously (tensor.cpp:146-154)
    CHECK_NE(buffer_, nullptr);
    const base::DeviceType where = device_type();
    if (where == base::DeviceType::DeviceCPU) {
        const size_t bytes = byte_size();
        auto gpu_alloc = base::CUDADeviceAllocatorFactory::get_instance();
        auto gpu_buffer = std::make_shared<base::Buffer>(bytes, gpu_alloc);
        gpu_alloc->memcpy(gpu_buffer->ptr(), buffer_->ptr(), bytes, base::MemcpyKind::MemcpyCPU2CUDA);
        buffer_ = gpu_buffer;
    } else if (where == base::DeviceType::DeviceCUDA) {
        LOG(INFO) << "The device type of the tensor is already cuda.";
    } else {
        LOG(ERROR) << "The device type of the tensor is unknown.";
    }
}

void Tensor::reshape(const std::vector<int32_t>& dims) {
    const size_t new_size = element_count(dims);
    if (buffer_ && size_ < new_size) {
        // grow: new storage from the same allocator, old contents copied over
        auto grown = std::make_shared<base::Buffer>(new_size * base::data_type_size(data_type_), buffer_->allocator());
        grown->copy_from(buffer_.get());
        buffer_ = grown;
    }
    dims_ = dims;
    size_ = new_size;
}

int32_t Tensor::dims_size() const {
    return static_cast<int32_t>(dims_.size());
}

int32_t Tensor::get_dim(int32_t index) const {
    CHECK_GE(index, 0);
    CHECK_LT(static_cast<size_t>(index), dims_.size());
    return dims_[index];
}

const std::vector<int32_t>& Tensor::dims() const {
    return dims_;
}

std::vector<size_t> Tensor::strides() const {
    std::vector<size_t> out(dims_.size(), 1);
    for (size_t i = dims_.size(); i-- > 1;) {
        out[i - 1] = out[i] * static_cast<size_t>(dims_[i]);
    }
    return out;
}

Tensor Tensor::clone() const {
    Tensor copy = *this;
    copy.buffer_ = std::make_shared<base::Buffer>(byte_size(), buffer_->allocator());
    copy.buffer_->copy_from(buffer_.get());
    return copy;
}

void Tensor::reset(base::DataType data_type, const std::vector<int32_t>& dims) {
    data_type_ = data_type;
    dims_ = dims;
    size_ = element_count(dims);
    buffer_ = nullptr;
}

bool Tensor::is_empty() const {
    return size_ == 0 || buffer_ == nullptr || buffer_->ptr() == nullptr;
}

size_t Tensor::size() const { return size_; }

size_t Tensor::byte_size() const {
    return size_ * base::data_type_size(data_type_);
}

base::DataType Tensor::data_type() const { return data_type_; }

base::DeviceType Tensor::device_type() const {
    return buffer_ ? buffer_->device_type() : base::DeviceType::DeviceUnknown;
}

void Tensor::set_device_type(base::DeviceType device_type) const {
    // const on purpose (reference tensor.cpp:244-249): the flag lives in the shared buffer
    if (buffer_ && buffer_->device_type() != device_type) {
        buffer_->set_device_type(device_type);
    }
}

std::shared_ptr<base::Buffer> Tensor::get_buffer() const { return buffer_; }

}  // namespace tensor
