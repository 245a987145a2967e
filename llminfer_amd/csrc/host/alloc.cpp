#include "alloc.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "llmi_hip.h"

namespace base {

void fatal(const char* file, int line, const std::string& msg) {
    std::ostringstream oss;
    oss << file << ":" << line << ": " << msg;
    throw FatalError(oss.str());
}

size_t data_type_size(DataType data_type) {
    switch (data_type) {
        case DataType::DataTypeBf16:
        case DataType::DataTypeFp16: return sizeof(uint16_t);
        case DataType::DataTypeFp32:
        case DataType::DataTypeInt32:
        case DataType::DataTypeInt4x8: return sizeof(int32_t);
        default: LLMI_FATAL("Unknown data type size for " << int(data_type));
    }
}

void DeviceAllocator::memcpy(void* dest_ptr, const void* src_ptr, size_t byte_size, MemcpyKind memcpy_kind,
                             void* stream, bool need_sync) const {
    LLMI_CHECK(dest_ptr != nullptr);
    LLMI_CHECK(src_ptr != nullptr);
    if (!byte_size) return;
    if (memcpy_kind == MemcpyKind::MemcpyCPU2CPU) {
        std::memcpy(dest_ptr, src_ptr, byte_size);
        return;
    }
    const int rc = llmi_hip_memcpy(dest_ptr, src_ptr, byte_size, static_cast<int32_t>(memcpy_kind), stream,
                                   need_sync ? 1 : 0);
    if (rc != LLMI_OK) LLMI_FATAL("memcpy kind " << int(memcpy_kind) << " failed: " << llmi_hip_last_error());
}

void DeviceAllocator::memset_zero(void* ptr, size_t byte_size, void* stream, bool need_sync) {
    LLMI_CHECK(device_type_ != DeviceType::DeviceUnknown);
    if (device_type_ == DeviceType::DeviceCPU) {
        std::memset(ptr, 0, byte_size);
        return;
    }
    const int rc = llmi_hip_memset_zero(ptr, byte_size, stream, need_sync ? 1 : 0);
    if (rc != LLMI_OK) LLMI_FATAL("memset_zero failed: " << llmi_hip_last_error());
}

void* CPUDeviceAllocator::allocate(size_t byte_size) {
    if (!byte_size) return nullptr;
    return std::malloc(byte_size);
}

void CPUDeviceAllocator::release(void* ptr) { std::free(ptr); }

void* HIPDeviceAllocator::allocate(size_t byte_size) {
    void* p = llmi_hip_pool_alloc(byte_size);
    if (!p && byte_size)
        std::fprintf(stderr, "HIPDeviceAllocator: cannot allocate %zu bytes: %s\n", byte_size, llmi_hip_last_error());
    return p;  // nullptr on failure, like alloc_cu.cpp:35-42
}

void HIPDeviceAllocator::release(void* ptr) {
    // Releasing a pointer the pool does not own is fatal (alloc_cu.cpp:86-87).
    if (llmi_hip_pool_free(ptr) != LLMI_OK) LLMI_FATAL("release of a pointer the device pool does not own");
}

std::shared_ptr<CPUDeviceAllocator> CPUDeviceAllocatorFactory::get_instance() {
    static std::shared_ptr<CPUDeviceAllocator> instance = std::make_shared<CPUDeviceAllocator>();
    return instance;
}

std::shared_ptr<HIPDeviceAllocator> HIPDeviceAllocatorFactory::get_instance() {
    static std::shared_ptr<HIPDeviceAllocator> instance = std::make_shared<HIPDeviceAllocator>();
    return instance;
}

}  // namespace base
