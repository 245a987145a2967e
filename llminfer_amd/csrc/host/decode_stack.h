// The attention part of one decode step over all layers, as the engine's layer
// loop issues it (code/source/model/qwen3_fused.cpp:115-127 with :517-553):
// per layer, fused QK-Norm + RoPE on the new token's Q and K with the K and V
// rows appended to the cache, then grouped-query attention over positions
// 0..pos. The sequence can be captured once into a HIP graph and replayed.
// Harness for benchmarks and tests, not part of the C ABI.
#ifndef LLMI_HOST_DECODE_STACK_H
#define LLMI_HOST_DECODE_STACK_H

#include <memory>
#include <vector>

#include "attention_buffers.h"
#include "hip_config.h"
#include "weight_file.h"

namespace model {

class DecodeStack {
public:
    explicit DecodeStack(const AttentionConfig& config);
    ~DecodeStack();
    DecodeStack(const DecodeStack&) = delete;
    DecodeStack& operator=(const DecodeStack&) = delete;

    AttentionBuffers& buffers() { return *buffers_; }
    hipStream_t stream() const { return hip_config_->stream; }
    // Per-layer inputs of the new token (raw, before QK-Norm) and norm weights, device bf16.
    uint16_t* query_raw(int32_t layer) { return raw_q_.ptr<uint16_t>(static_cast<int64_t>(layer) * config_.dim()); }
    uint16_t* key_raw(int32_t layer) { return raw_k_.ptr<uint16_t>(static_cast<int64_t>(layer) * config_.kv_dim()); }
    uint16_t* value_raw(int32_t layer) { return raw_v_.ptr<uint16_t>(static_cast<int64_t>(layer) * config_.kv_dim()); }
    uint16_t* norm_weight(int32_t layer) { return norm_w_.ptr<uint16_t>(static_cast<int64_t>(layer) * 2 * config_.head_dim); }
    // Per-layer attention outputs [layer][dim], device bf16.
    uint16_t* output(int32_t layer) { return outputs_.ptr<uint16_t>(static_cast<int64_t>(layer) * config_.dim()); }

    // Optional: the projections either side of the attention (packed QKV GEMV in front, output
    // projection with residual add behind; code/source/model/qwen3_fused.cpp:517-553). Allocates
    // per-layer weights [dim + 2*kv_dim][hidden] and [hidden][dim], per-layer inputs [hidden] and one
    // residual stream [hidden]; needed by mode kAttentionBlock.
    void enable_projections(int32_t hidden_dim);
    int32_t hidden_dim() const { return hidden_dim_; }
    uint16_t* qkv_weight(int32_t layer) { return wqkv_.ptr<uint16_t>(static_cast<int64_t>(layer) * (config_.dim() + 2 * config_.kv_dim()) * hidden_dim_); }
    uint16_t* out_weight(int32_t layer) { return wo_.ptr<uint16_t>(static_cast<int64_t>(layer) * hidden_dim_ * config_.dim()); }
    uint16_t* hidden_in(int32_t layer) { return hidden_.ptr<uint16_t>(static_cast<int64_t>(layer) * hidden_dim_); }
    uint16_t* residual() { return residual_.ptr<uint16_t>(); }

    // Uploads the attention block's weights of every layer of this stack from a mapped weight file
    // (packed QKV projection, q_norm/k_norm, output projection); enables the projections if needed.
    // The file must describe the stack's head layout; it may hold more layers than the stack.
    base::Status load_weights(const WeightFile& file);

    void build_sincos();
    // What one layer issues: attention alone on the raw query (0), the QK-Norm + RoPE + append kernel
    // followed by attention (1, the reference's sequence), or both fused into one launch (2).
    // kAttentionBlock (3): packed QKV GEMV -> fused append attention -> output projection + residual,
    // three launches per layer.
    // kFusedBlock (4): the same block in two launches per layer: packed QKV GEMV -> attention whose idle
    // workgroups also do the output projection + residual (llmi_hip_mha_decode_append_oproj).
    // kResidentStack (5): what kFusedAppend computes, as ONE launch for all layers (llmi_hip_mha_decode_append_stack):
    // the grid stays resident, the next layer's K/V tiles are on their way while this layer's results are merged,
    // and a layer reads its inputs only after the layer before has published its outputs.
    enum Mode : int32_t { kAttentionOnly = 0, kSeparateQkNormRope = 1, kFusedAppend = 2, kAttentionBlock = 3, kFusedBlock = 4,
                          kResidentStack = 5 };
    // Enqueues the whole stack for a token at `pos` on the stack's stream (no synchronisation).
    // `follow_device_pos`: the kernels read the position from the stack's device word (set_position)
    // and `pos` is the largest position they may see; modes 0 and 2 only (the separate QK-Norm/RoPE
    // launch takes its position from the host).
    void enqueue(int32_t pos, int32_t mode, bool follow_device_pos = false);
    // Captures enqueue(pos, mode, follow_device_pos) into a graph (replacing an earlier one).
    void capture(int32_t pos, int32_t mode, bool follow_device_pos = false);
    // Writes the position word the kernels follow (ordered on the stack's stream).
    void set_position(int32_t pos);
    // Replays the captured graph `times` times; returns the elapsed milliseconds (HIP events on the stream).
    float replay(int32_t times);
    void synchronize();

private:
    AttentionConfig config_;
    std::shared_ptr<kernel::HipConfig> hip_config_;
    std::unique_ptr<AttentionBuffers> buffers_;
    tensor::Tensor raw_q_, raw_k_, raw_v_, norm_w_, outputs_, pos_dev_;
    tensor::Tensor wqkv_, wo_, hidden_, residual_;
    int32_t hidden_dim_ = 0;
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t graph_exec_ = nullptr;
};

}  // namespace model
#endif
