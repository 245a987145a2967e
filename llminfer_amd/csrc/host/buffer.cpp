#include "buffer.h"

namespace base {

Buffer::Buffer(size_t byte_size, std::shared_ptr<DeviceAllocator> allocator, void* ptr, bool use_external)
    : byte_size_(byte_size), allocator_(std::move(allocator)), ptr_(ptr), use_external_(use_external) {
    if (allocator_) device_type_ = allocator_->device_type();
    if (!ptr_ && allocator_) {
        use_external_ = false;
        ptr_ = allocator_->allocate(byte_size_);
    }
}

Buffer::~Buffer() {
    if (!use_external_ && ptr_ && allocator_) {
        allocator_->release(ptr_);
        ptr_ = nullptr;
    }
}

bool Buffer::allocate() {
    if (!allocator_ || !byte_size_) return false;
    use_external_ = false;
    ptr_ = allocator_->allocate(byte_size_);
    return ptr_ != nullptr;
}

void Buffer::copy_from(const Buffer& src) const {
    LLMI_CHECK(allocator_ != nullptr);
    LLMI_CHECK(src.ptr_ != nullptr);
    const size_t n = byte_size_ < src.byte_size_ ? byte_size_ : src.byte_size_;  // the smaller of the two
    const DeviceType to = device_type_, from = src.device_type_;
    LLMI_CHECK(to != DeviceType::DeviceUnknown && from != DeviceType::DeviceUnknown);
    MemcpyKind kind;
    if (from == DeviceType::DeviceCPU)
        kind = to == DeviceType::DeviceCPU ? MemcpyKind::MemcpyCPU2CPU : MemcpyKind::MemcpyCPU2HIP;
    else
        kind = to == DeviceType::DeviceCPU ? MemcpyKind::MemcpyHIP2CPU : MemcpyKind::MemcpyHIP2HIP;
    allocator_->memcpy(ptr_, src.ptr_, n, kind);
}

void Buffer::copy_from(const Buffer* src) const {
    LLMI_CHECK(src != nullptr);
    copy_from(*src);
}

}  // namespace base
