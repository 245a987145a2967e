// The operator registry of the attention path: one function-pointer type per
// op and a getter that picks the implementation by DeviceType.
// Mirrors code/source/op/kernel/kernel_interface.h (MHAKernel :168-183,
// FusedQKNormRoPEKernel :154-166, SinCosCacheKernel :132-139, SoftmaxKernel
// :185-189, ScaleSumKernel :194-202) and kernel_interface.cpp:25-219.
//
// Argument order of MHAKernel. The typedef names its second parameter "score",
// which is what the CPU kernel takes (cpu/mha_kernel.h:7-21); the GPU kernel
// takes (query, key_cache, value_cache, kv_split_output, output, ...)
// (cuda/mha_kernel.cuh:7-21) and that is the order the only caller passes
// (op/mha.cpp:54-56). Both orders are kept as they are in the reference:
//   DeviceHIP arm: (query, key_cache, value_cache, workspace, output, ...)
//   DeviceCPU arm: (query, score, key_cache, value_cache, output, ...)
//
// The DeviceHIP arms are built in. This backend ships no CPU compute: a CPU
// arm exists only if the embedding program registers one (register_*_kernel),
// otherwise asking for it is fatal, as asking the reference for an
// unregistered device is (kernel_interface.cpp:186-189).
#ifndef LLMI_HOST_KERNEL_INTERFACE_H
#define LLMI_HOST_KERNEL_INTERFACE_H

#include "tensor.h"

namespace kernel {

using MHAKernel = void (*)(const tensor::Tensor& query, const tensor::Tensor& score,
                           const tensor::Tensor& key_cache, const tensor::Tensor& value_cache,
                           const tensor::Tensor& output, int32_t layer_id, int32_t pos, int32_t kv_dim,
                           int32_t kv_mul, int32_t head_num, int32_t head_dim, int32_t max_seq_len, void* stream);
MHAKernel get_mha_kernel(base::DeviceType device_type);
void register_mha_kernel(base::DeviceType device_type, MHAKernel fn);

using FusedQKNormRoPEKernel = void (*)(const tensor::Tensor& query, const tensor::Tensor& key,
                                       const tensor::Tensor& weight, const tensor::Tensor& token_pos,
                                       const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache, int32_t dim,
                                       int32_t kv_dim, int32_t head_dim, void* stream);
FusedQKNormRoPEKernel get_fused_qk_norm_rope_kernel(base::DeviceType device_type);

using SinCosCacheKernel = void (*)(const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache,
                                   int32_t head_dim, int32_t max_seq_len, void* stream);
SinCosCacheKernel get_sin_cos_cache_kernel(base::DeviceType device_type);

// The bf16 GEMVs either side of the attention (kernel_interface.h:49-65,76-84 of the reference).
using GEMVKernel = void (*)(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& output,
                            bool lm_head, void* stream);
GEMVKernel get_gemv_kernel(base::DeviceType device_type);

using FusedGEMVAddKernel = void (*)(const tensor::Tensor& input, const tensor::Tensor& weight,
                                    const tensor::Tensor& output, void* stream);
FusedGEMVAddKernel get_fused_gemv_add_kernel(base::DeviceType device_type);

using FusedQKVGEMVKernel = void (*)(const tensor::Tensor& input, const tensor::Tensor& weight,
                                    const tensor::Tensor& query, const tensor::Tensor& key,
                                    const tensor::Tensor& value, void* stream);
FusedQKVGEMVKernel get_fused_qkv_gemv_kernel(base::DeviceType device_type);

// The gfx950 implementations (thin shims over the C ABI of libllmi_hip.so).
// A 3-D key/value cache tensor [layers, max_seq_len, kv_dim] is the
// reference's position-major layout; a 4-D one [layers, kv_heads, max_seq_len,
// head_dim] is the head-major layout.
void mha_kernel_hip(const tensor::Tensor& query, const tensor::Tensor& key_cache, const tensor::Tensor& value_cache,
                    const tensor::Tensor& kv_split_output, const tensor::Tensor& output, int32_t layer_id,
                    int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num, int32_t head_dim,
                    int32_t max_seq_len, void* stream);
void fused_qk_norm_rope_kernel_hip(const tensor::Tensor& query, const tensor::Tensor& key,
                                   const tensor::Tensor& weight, const tensor::Tensor& token_pos,
                                   const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache, int32_t dim,
                                   int32_t kv_dim, int32_t head_dim, void* stream);
void gemv_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& output,
                     bool lm_head, void* stream);
void fused_gemv_add_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight,
                               const tensor::Tensor& output, void* stream);
void fused_qkv_gemv_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& query,
                               const tensor::Tensor& key, const tensor::Tensor& value, void* stream);
void sin_cos_cache_precompute_hip(const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache, int32_t head_dim,
                                  int32_t max_seq_len, void* stream);

// Tuning overrides read by mha_kernel_hip (0 = let the library decide). The
// registry signature has no room for them; they are process-wide, like the
// reference's compile-time constants (mha_kernel.cu:478,505-517).
struct MhaHipOptions {
    int32_t force_path = 0;
    int32_t num_splits = 0;
    int32_t waves_per_group = 0;
};
MhaHipOptions& mha_hip_options();

// What llmi_hip_mha_workspace_side says about a split workspace (which of its 8 KiB blocks lie near which side of the
// package), measured the first time a workspace is seen outside stream capture and remembered by its address; 0 (the
// plain layout) where it cannot be measured now. The measurement overwrites the start of the workspace and
// synchronises `stream`.
int32_t workspace_side_of(const void* workspace, size_t bytes, void* stream);

}  // namespace kernel
#endif
