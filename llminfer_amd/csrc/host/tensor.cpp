#include "tensor.h"

#include <cstdio>

namespace tensor {

static size_t element_count(const std::vector<int32_t>& dims) {
    if (dims.empty()) return 0;
    size_t n = 1;
    for (int32_t d : dims) n *= static_cast<size_t>(d);
    return n;
}

Tensor::Tensor(base::DataType data_type, int32_t dim0, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : Tensor(data_type, std::vector<int32_t>{dim0}, need_alloc, std::move(allocator), ptr) {}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : Tensor(data_type, std::vector<int32_t>{dim0, dim1}, need_alloc, std::move(allocator), ptr) {}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, int32_t dim2, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : Tensor(data_type, std::vector<int32_t>{dim0, dim1, dim2}, need_alloc, std::move(allocator), ptr) {}

Tensor::Tensor(base::DataType data_type, int32_t dim0, int32_t dim1, int32_t dim2, int32_t dim3, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : Tensor(data_type, std::vector<int32_t>{dim0, dim1, dim2, dim3}, need_alloc, std::move(allocator), ptr) {}

Tensor::Tensor(base::DataType data_type, std::vector<int32_t> dims, bool need_alloc,
               std::shared_ptr<base::DeviceAllocator> allocator, void* ptr)
    : size_(element_count(dims)), dims_(std::move(dims)), data_type_(data_type) {
    init_buffer(std::move(allocator), need_alloc, ptr);
}

void Tensor::init_buffer(std::shared_ptr<base::DeviceAllocator> allocator, bool need_alloc, void* ptr) {
    if (!allocator) {
        LLMI_CHECK(!need_alloc);  // tensor.cpp:62
        if (ptr) buffer_ = std::make_shared<base::Buffer>(byte_size(), nullptr, ptr, true);  // borrowed view
        return;
    }
    if (need_alloc) {
        allocate(allocator, false);
    } else if (ptr) {
        buffer_ = std::make_shared<base::Buffer>(byte_size(), allocator, ptr, false);  // adopted
    } else {
        allocate(allocator, true);
    }
}

bool Tensor::allocate(std::shared_ptr<base::DeviceAllocator> allocator, bool need_realloc) {
    if (!allocator) {
        std::fprintf(stderr, "Tensor::allocate: null allocator\n");
        return false;
    }
    const size_t bytes = byte_size();
    if (!bytes) {
        std::fprintf(stderr, "Tensor::allocate: zero bytes\n");
        return false;
    }
    if (buffer_ && bytes <= buffer_->byte_size() && !need_realloc) return true;
    buffer_ = std::make_shared<base::Buffer>(bytes, allocator, nullptr);
    if (!buffer_->ptr()) {
        std::fprintf(stderr, "Tensor::allocate: the allocator returned a null pointer\n");
        return false;
    }
    return true;
}

bool Tensor::assgin(std::shared_ptr<base::Buffer> buffer) {
    if (!buffer) {
        std::fprintf(stderr, "Tensor::assgin: null buffer\n");
        return false;
    }
    if (buffer_ && buffer_->device_type() != buffer->device_type())
        std::fprintf(stderr, "Tensor::assgin: the new buffer is on another device than the old one\n");
    if (buffer->byte_size() < byte_size()) {
        std::fprintf(stderr, "Tensor::assgin: buffer too small for the tensor\n");
        return false;
    }
    buffer_ = std::move(buffer);
    return true;
}

void Tensor::to_cpu() {
    LLMI_CHECK(buffer_ != nullptr);
    if (device_type() != base::DeviceType::DeviceHIP) return;  // already on the host (or unknown: left alone)
    auto cpu = base::CPUDeviceAllocatorFactory::get_instance();
    auto host = std::make_shared<base::Buffer>(byte_size(), cpu);
    cpu->memcpy(host->ptr(), buffer_->ptr(), byte_size(), base::MemcpyKind::MemcpyHIP2CPU);
    buffer_ = host;
}

void Tensor::to_hip(hipStream_t stream) {
    LLMI_CHECK(buffer_ != nullptr);
    if (device_type() != base::DeviceType::DeviceCPU) return;
    auto hip = base::HIPDeviceAllocatorFactory::get_instance();
    auto dev = std::make_shared<base::Buffer>(byte_size(), hip);
    LLMI_CHECK(dev->ptr() != nullptr);
    hip->memcpy(dev->ptr(), buffer_->ptr(), byte_size(), base::MemcpyKind::MemcpyCPU2HIP, stream);
    buffer_ = dev;
}

void Tensor::reshape(const std::vector<int32_t>& dims) {
    const size_t n = element_count(dims);
    if (buffer_ && size_ < n) {  // grow: new block, old contents copied over (tensor.cpp:176-181)
        auto bigger = std::make_shared<base::Buffer>(n * base::data_type_size(data_type_), buffer_->allocator());
        bigger->copy_from(buffer_.get());
        buffer_ = bigger;
    }
    dims_ = dims;
    size_ = n;
}

int32_t Tensor::get_dim(int32_t index) const {
    LLMI_CHECK(index >= 0 && static_cast<size_t>(index) < dims_.size());
    return dims_[index];
}

std::vector<size_t> Tensor::strides() const {
    std::vector<size_t> s(dims_.size(), 1);
    for (int i = static_cast<int>(dims_.size()) - 1; i >= 1; --i) s[i - 1] = s[i] * dims_[i];
    return s;
}

Tensor Tensor::clone() const {
    Tensor t = *this;
    t.buffer_ = std::make_shared<base::Buffer>(byte_size(), buffer_->allocator());
    t.buffer_->copy_from(buffer_.get());
    return t;
}

void Tensor::reset(base::DataType data_type, const std::vector<int32_t>& dims) {
    size_ = element_count(dims);
    dims_ = dims;
    buffer_ = nullptr;
    data_type_ = data_type;
}

}  // namespace tensor
