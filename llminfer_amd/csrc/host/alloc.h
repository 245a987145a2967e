// Device allocators behind Buffer/Tensor: plain malloc on the host, the pooled
// hipMalloc allocator of libllmi_hip.so on the device.
// Mirrors code/include/base/alloc.h:10-85 of the reference.
#ifndef LLMI_HOST_ALLOC_H
#define LLMI_HOST_ALLOC_H

#include <memory>

#include "base.h"

namespace base {

enum class MemcpyKind : uint8_t {
    MemcpyCPU2CPU = 0,
    MemcpyCPU2HIP = 1,
    MemcpyHIP2CPU = 2,
    MemcpyHIP2HIP = 3,
};

class DeviceAllocator {
public:
    explicit DeviceAllocator(DeviceType device_type) : device_type_(device_type) {}
    virtual ~DeviceAllocator() = default;
    virtual DeviceType device_type() const { return device_type_; }
    virtual void* allocate(size_t byte_size) = 0;
    virtual void release(void* ptr) = 0;
    // alloc.cpp:11-53: NULL stream = synchronous copy, need_sync adds a device synchronise.
    virtual void memcpy(void* dest_ptr, const void* src_ptr, size_t byte_size,
                        MemcpyKind memcpy_kind = MemcpyKind::MemcpyCPU2CPU, void* stream = nullptr,
                        bool need_sync = false) const;
    virtual void memset_zero(void* ptr, size_t byte_size, void* stream, bool need_sync = false);

private:
    DeviceType device_type_ = DeviceType::DeviceUnknown;
};

class CPUDeviceAllocator : public DeviceAllocator {
public:
    CPUDeviceAllocator() : DeviceAllocator(DeviceType::DeviceCPU) {}
    void* allocate(size_t byte_size) override;
    void release(void* ptr) override;
};

// Two size classes split at 1 MiB, best-fit reuse, blocks never handed back
// (alloc_cu.cpp:7-119); the policy itself lives in libllmi_hip.so (llmi_pool_*).
class HIPDeviceAllocator : public DeviceAllocator {
public:
    HIPDeviceAllocator() : DeviceAllocator(DeviceType::DeviceHIP) {}
    void* allocate(size_t byte_size) override;
    void release(void* ptr) override;
};

class CPUDeviceAllocatorFactory {
public:
    static std::shared_ptr<CPUDeviceAllocator> get_instance();
};

class HIPDeviceAllocatorFactory {
public:
    static std::shared_ptr<HIPDeviceAllocator> get_instance();
};

}  // namespace base
#endif
