// The engine's on-disk weight file for the dense bf16 model, read the way the
// engine reads it: an 8 x int32 header followed by one flat bf16 payload in a
// fixed order, mapped into memory and addressed by element offset.
// Role of model::ModelConfig (code/include/model/config.h:7-16),
// Model::read_model_file (code/source/model/model.cpp:130-179),
// Model::generate_model_info (:210-236) and the offset walk of
// Qwen3FusedModel::create_param_layers (code/source/model/qwen3_fused.cpp:233-319).
// The file is written by tools/qwen3/qwen3_dense_unified_converter.py:43-57
// (header int32[8], then the tensors in the order below).
#ifndef LLMI_HOST_WEIGHT_FILE_H
#define LLMI_HOST_WEIGHT_FILE_H

#include <memory>
#include <string>

#include "base.h"

namespace model {

// The header as stored (config.h:7-16). `dim` is the query width, `hidden_dim`
// the embedding width, `immediate_dim` the FFN width.
struct ModelConfig {
    int32_t dim = 0;
    int32_t hidden_dim = 0;
    int32_t layer_num = 0;
    int32_t head_num = 0;
    int32_t kv_head_num = 0;
    int32_t vocab_size = 0;
    int32_t max_seq_len = 0;
    int32_t immediate_dim = 0;
};

class WeightFile : private base::NoCopyable {
public:
    // Maps `path` read-only, reads the header, derives head_dim / kv_dim and checks that
    // the payload is exactly as long as the layout says (qwen3_fused.cpp:317-318).
    // `header_ints` is 8; 7 reads the older header without immediate_dim (the layout of
    // the engine's loader fixture): header and raw payload only, no derived sizes, no tensors.
    static base::Status open(const std::string& path, std::unique_ptr<WeightFile>* out, int32_t header_ints = 8);
    ~WeightFile();

    const ModelConfig& config() const { return config_; }
    int32_t head_dim() const { return head_dim_; }
    int32_t kv_dim() const { return kv_dim_; }
    int32_t kv_mul() const { return config_.head_num / config_.kv_head_num; }
    int32_t vocab_size() const { return vocab_size_; }  // |vocab_size| (model.cpp:233)
    size_t file_size() const { return file_size_; }
    size_t payload_elements() const { return payload_elems_; }

    // Start of the payload; element offset `offset` (RawModelDataBf16::weight_ptr).
    const uint16_t* weight_ptr(size_t offset) const {
        LLMI_CHECK(offset <= payload_elems_);
        return payload_ + offset;
    }
    const void* payload_bytes() const { return payload_; }

    // The tensors in file order (qwen3_fused.cpp:246-314).
    const uint16_t* embedding() const { return weight_ptr(off_embedding_); }           // [vocab][hidden]
    const uint16_t* pre_rmsnorm(int32_t layer) const;                                    // [hidden]
    const uint16_t* qkv_proj(int32_t layer) const;                                       // [dim + 2*kv_dim][hidden]
    const uint16_t* qk_norm(int32_t layer) const;                                        // [2*head_dim]
    const uint16_t* o_proj(int32_t layer) const;                                         // [hidden][dim]
    const uint16_t* ffn_rmsnorm(int32_t layer) const;                                    // [hidden]
    const uint16_t* gate_up(int32_t layer) const;                                        // [2*immediate][hidden]
    const uint16_t* down_proj(int32_t layer) const;                                      // [hidden][immediate]
    const uint16_t* final_rmsnorm() const { return weight_ptr(off_final_norm_); }       // [hidden]
    const uint16_t* lm_head() const { return weight_ptr(0); }                           // tied to the embedding (:313)

private:
    WeightFile() = default;
    size_t layer_off(size_t base, int32_t layer, size_t per_layer) const;

    ModelConfig config_;
    int32_t head_dim_ = 0, kv_dim_ = 0, vocab_size_ = 0;
    int fd_ = -1;
    void* map_ = nullptr;
    size_t file_size_ = 0, payload_elems_ = 0;
    const uint16_t* payload_ = nullptr;
    size_t off_embedding_ = 0, off_pre_norm_ = 0, off_qkv_ = 0, off_qk_norm_ = 0, off_o_ = 0, off_ffn_norm_ = 0,
           off_gate_up_ = 0, off_down_ = 0, off_final_norm_ = 0, total_elems_ = 0;
};

}  // namespace model
#endif
