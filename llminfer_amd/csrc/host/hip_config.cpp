#include "hip_config.h"

#include "base.h"

namespace kernel {
HipConfig::~HipConfig() {
    if (stream) (void)hipStreamDestroy(stream);
}

void HipConfig::create() {
    if (stream) return;
    const hipError_t err = hipStreamCreate(&stream);
    if (err != hipSuccess) LLMI_FATAL("hipStreamCreate failed: " << hipGetErrorString(err));
}
}  // namespace kernel
