// Owner of the device buffers of the attention path: K/V caches (either
// layout), split workspace, query / output vectors, sin/cos tables, and the
// addressing of one token's cache slot.
// Role of Qwen3FusedModel::allocate_model_buffers (code/source/model/qwen3_fused.cpp:453-515,
// the rows :482-503), Model::get_buffer and Model::slice_kv_cache
// (code/source/model/model.cpp:90-107) of the reference.
#ifndef LLMI_HOST_ATTENTION_BUFFERS_H
#define LLMI_HOST_ATTENTION_BUFFERS_H

#include <map>
#include <utility>

#include "llmi_hip.h"
#include "tensor.h"

namespace model {

struct AttentionConfig {
    int32_t layer_num = 0;
    int32_t max_seq_len = 0;
    int32_t head_num = 0;     // query heads
    int32_t kv_head_num = 0;
    int32_t head_dim = 128;
    int32_t kv_layout = LLMI_KV_LAYOUT_HEAD_MAJOR;
    int32_t dim() const { return head_num * head_dim; }
    int32_t kv_dim() const { return kv_head_num * head_dim; }
    int32_t kv_mul() const { return head_num / kv_head_num; }
};

class AttentionBuffers {
public:
    // Allocates everything through `allocator` (the pooled device allocator in production).
    AttentionBuffers(const AttentionConfig& config, std::shared_ptr<base::DeviceAllocator> allocator);

    const AttentionConfig& config() const { return config_; }
    tensor::Tensor& get_buffer(ModelBufferType type);
    const tensor::Tensor& get_buffer(ModelBufferType type) const;

    // Element offset of (layer, pos, kv_head, 0) inside a cache, 64-bit
    // (the reference's int32 product, model.cpp:92-93, overflows on large caches).
    int64_t kv_offset(int32_t layer_id, int32_t token_pos, int32_t kv_head) const;

    // One token's K and V rows as borrowed [kv_dim] views. Only the
    // position-major layout stores a row contiguously; asking for it in the
    // head-major layout is fatal (use kv_offset per KV head there).
    std::pair<tensor::Tensor, tensor::Tensor> slice_kv_cache(int32_t layer_id, int32_t token_pos) const;

private:
    AttentionConfig config_;
    base::DeviceType device_type_;
    std::map<ModelBufferType, tensor::Tensor> buffers_;
};

}  // namespace model
#endif
