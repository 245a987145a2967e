// One HIP stream, created on demand and destroyed with the object
// (role of kernel::CudaConfig, code/include/base/cuda_config.h:17-21).
#ifndef LLMI_HOST_HIP_CONFIG_H
#define LLMI_HOST_HIP_CONFIG_H

#include <hip/hip_runtime_api.h>

namespace kernel {
struct HipConfig {
    HipConfig() = default;
    HipConfig(const HipConfig&) = delete;
    HipConfig& operator=(const HipConfig&) = delete;
    ~HipConfig();
    void create();  // default priority, like every stream this backend uses
    hipStream_t stream = nullptr;
};
}  // namespace kernel
#endif
