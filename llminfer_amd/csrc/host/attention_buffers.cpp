#include "attention_buffers.h"

namespace model {

AttentionBuffers::AttentionBuffers(const AttentionConfig& c, std::shared_ptr<base::DeviceAllocator> allocator)
    : config_(c), device_type_(allocator->device_type()) {
    LLMI_CHECK(c.layer_num > 0 && c.max_seq_len > 0 && c.head_num > 0 && c.kv_head_num > 0);
    LLMI_CHECK(c.head_num % c.kv_head_num == 0);
    using base::DataType;
    auto put = [&](ModelBufferType type, tensor::Tensor t) {
        LLMI_CHECK(!t.is_empty());
        buffers_.emplace(type, std::move(t));
    };
    if (c.kv_layout == LLMI_KV_LAYOUT_POS_MAJOR) {
        put(ModelBufferType::KeyCache, tensor::Tensor(DataType::DataTypeBf16, c.layer_num, c.max_seq_len, c.kv_dim(), true, allocator));
        put(ModelBufferType::ValueCache, tensor::Tensor(DataType::DataTypeBf16, c.layer_num, c.max_seq_len, c.kv_dim(), true, allocator));
    } else {
        put(ModelBufferType::KeyCache, tensor::Tensor(DataType::DataTypeBf16, c.layer_num, c.kv_head_num, c.max_seq_len, c.head_dim, true, allocator));
        put(ModelBufferType::ValueCache, tensor::Tensor(DataType::DataTypeBf16, c.layer_num, c.kv_head_num, c.max_seq_len, c.head_dim, true, allocator));
    }
    put(ModelBufferType::Query, tensor::Tensor(DataType::DataTypeBf16, c.dim(), true, allocator));
    put(ModelBufferType::MHAOutput, tensor::Tensor(DataType::DataTypeBf16, c.dim(), true, allocator));
    // Split workspace: [head_num, n] fp32 with n at least the reference's 4*max_seq_len
    // (qwen3_fused.cpp:502) and at least what the kernels ask for at this max_seq_len.
    const size_t need = llmi_hip_mha_workspace_bytes(c.head_num, c.head_dim, c.max_seq_len);
    int32_t per_head = 4 * c.max_seq_len;
    const size_t need_per_head = (need / sizeof(float) + c.head_num - 1) / c.head_num;
    if (static_cast<size_t>(per_head) < need_per_head) per_head = static_cast<int32_t>(need_per_head);
    put(ModelBufferType::KVSplitOutput, tensor::Tensor(DataType::DataTypeFp32, c.head_num, per_head, true, allocator));
    put(ModelBufferType::SinCache, tensor::Tensor(DataType::DataTypeFp32, c.max_seq_len, c.head_dim / 2, true, allocator));
    put(ModelBufferType::CosCache, tensor::Tensor(DataType::DataTypeFp32, c.max_seq_len, c.head_dim / 2, true, allocator));
    put(ModelBufferType::TokenPosition,
        tensor::Tensor(DataType::DataTypeInt32, 1, true, base::CPUDeviceAllocatorFactory::get_instance()));
}

tensor::Tensor& AttentionBuffers::get_buffer(ModelBufferType type) {
    auto it = buffers_.find(type);
    LLMI_CHECK(it != buffers_.end());
    return it->second;
}

const tensor::Tensor& AttentionBuffers::get_buffer(ModelBufferType type) const {
    auto it = buffers_.find(type);
    LLMI_CHECK(it != buffers_.end());
    return it->second;
}

int64_t AttentionBuffers::kv_offset(int32_t layer_id, int32_t token_pos, int32_t kv_head) const {
    const AttentionConfig& c = config_;
    LLMI_CHECK(layer_id >= 0 && layer_id < c.layer_num && token_pos >= 0 && token_pos < c.max_seq_len);
    LLMI_CHECK(kv_head >= 0 && kv_head < c.kv_head_num);
    const int64_t layer = static_cast<int64_t>(layer_id) * c.max_seq_len * c.kv_dim();
    if (c.kv_layout == LLMI_KV_LAYOUT_POS_MAJOR)
        return layer + static_cast<int64_t>(token_pos) * c.kv_dim() + static_cast<int64_t>(kv_head) * c.head_dim;
    return layer + (static_cast<int64_t>(kv_head) * c.max_seq_len + token_pos) * c.head_dim;
}

std::pair<tensor::Tensor, tensor::Tensor> AttentionBuffers::slice_kv_cache(int32_t layer_id, int32_t token_pos) const {
    if (config_.kv_layout != LLMI_KV_LAYOUT_POS_MAJOR)
        LLMI_FATAL("slice_kv_cache: a token's row is contiguous only in the position-major layout");
    const int64_t off = kv_offset(layer_id, token_pos, 0);
    const tensor::Tensor& kc = get_buffer(ModelBufferType::KeyCache);
    const tensor::Tensor& vc = get_buffer(ModelBufferType::ValueCache);
    tensor::Tensor key(base::DataType::DataTypeBf16, config_.kv_dim(), false, nullptr,
                       const_cast<uint16_t*>(kc.ptr<uint16_t>(off)));
    tensor::Tensor value(base::DataType::DataTypeBf16, config_.kv_dim(), false, nullptr,
                         const_cast<uint16_t*>(vc.ptr<uint16_t>(off)));
    key.set_device_type(device_type_);
    value.set_device_type(device_type_);
    return {key, value};
}

}  // namespace model
