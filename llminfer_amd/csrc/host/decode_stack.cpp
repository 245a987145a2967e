#include "decode_stack.h"

#include <hip/hip_runtime.h>

#include "kernel_interface.h"

namespace model {

#define HIP_OK(expr)                                                                     \
    do {                                                                                 \
        hipError_t llmi_e_ = (expr);                                                     \
        if (llmi_e_ != hipSuccess) LLMI_FATAL(#expr << ": " << hipGetErrorString(llmi_e_)); \
    } while (0)

DecodeStack::DecodeStack(const AttentionConfig& config) : config_(config) {
    hip_config_ = std::make_shared<kernel::HipConfig>();
    hip_config_->create();
    auto alloc = base::HIPDeviceAllocatorFactory::get_instance();
    buffers_ = std::make_unique<AttentionBuffers>(config, alloc);
    const int32_t L = config.layer_num;
    using base::DataType;
    raw_q_ = tensor::Tensor(DataType::DataTypeBf16, L, config.dim(), true, alloc);
    raw_k_ = tensor::Tensor(DataType::DataTypeBf16, L, config.kv_dim(), true, alloc);
    raw_v_ = tensor::Tensor(DataType::DataTypeBf16, L, config.kv_dim(), true, alloc);
    norm_w_ = tensor::Tensor(DataType::DataTypeBf16, L, 2 * config.head_dim, true, alloc);
    outputs_ = tensor::Tensor(DataType::DataTypeBf16, L, config.dim(), true, alloc);
    pos_dev_ = tensor::Tensor(DataType::DataTypeInt32, 4, true, alloc);
    LLMI_CHECK(!pos_dev_.is_empty());
    LLMI_CHECK(!raw_q_.is_empty() && !raw_k_.is_empty() && !raw_v_.is_empty() && !norm_w_.is_empty() && !outputs_.is_empty());
}

DecodeStack::~DecodeStack() {
    if (graph_exec_) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_) (void)hipGraphDestroy(graph_);
}

void DecodeStack::enable_projections(int32_t hidden_dim) {
    LLMI_CHECK(hidden_dim > 0 && hidden_dim % 8 == 0);
    auto alloc = base::HIPDeviceAllocatorFactory::get_instance();
    const int32_t L = config_.layer_num;
    using base::DataType;
    hidden_dim_ = hidden_dim;
    wqkv_ = tensor::Tensor(DataType::DataTypeBf16, L, config_.dim() + 2 * config_.kv_dim(), hidden_dim, true, alloc);
    wo_ = tensor::Tensor(DataType::DataTypeBf16, L, hidden_dim, config_.dim(), true, alloc);
    hidden_ = tensor::Tensor(DataType::DataTypeBf16, L, hidden_dim, true, alloc);
    residual_ = tensor::Tensor(DataType::DataTypeBf16, hidden_dim, true, alloc);
    LLMI_CHECK(!wqkv_.is_empty() && !wo_.is_empty() && !hidden_.is_empty() && !residual_.is_empty());
}

base::Status DecodeStack::load_weights(const WeightFile& file) {
    const ModelConfig& f = file.config();
    const AttentionConfig& c = config_;
    if (f.head_num != c.head_num || f.kv_head_num != c.kv_head_num || file.head_dim() != c.head_dim)
        return base::error::invalid_argument("The weight file's head layout differs from the stack's.");
    if (f.layer_num < c.layer_num) return base::error::invalid_argument("The weight file has fewer layers than the stack.");
    if (hidden_dim_ == 0) enable_projections(f.hidden_dim);
    if (hidden_dim_ != f.hidden_dim) return base::error::invalid_argument("The weight file's hidden_dim differs from the stack's.");
    const size_t qkv_bytes = static_cast<size_t>(c.dim() + 2 * c.kv_dim()) * hidden_dim_ * sizeof(uint16_t);
    const size_t o_bytes = static_cast<size_t>(hidden_dim_) * c.dim() * sizeof(uint16_t);
    const size_t norm_bytes = 2 * static_cast<size_t>(c.head_dim) * sizeof(uint16_t);
    for (int32_t l = 0; l < c.layer_num; ++l) {
        const std::pair<void*, std::pair<const void*, size_t>> copies[] = {
            {qkv_weight(l), {file.qkv_proj(l), qkv_bytes}},
            {norm_weight(l), {file.qk_norm(l), norm_bytes}},
            {out_weight(l), {file.o_proj(l), o_bytes}},
        };
        for (const auto& cp : copies) {
            const int rc = llmi_hip_memcpy(cp.first, cp.second.first, cp.second.second, 1, nullptr, 1);  // host to device
            if (rc != LLMI_OK) return base::error::internal_error(std::string("weight upload: ") + llmi_hip_strerror(rc));
        }
    }
    return base::error::success();
}

void DecodeStack::build_sincos() {
    kernel::get_sin_cos_cache_kernel(base::DeviceType::DeviceHIP)(
        buffers_->get_buffer(ModelBufferType::SinCache), buffers_->get_buffer(ModelBufferType::CosCache),
        config_.head_dim, config_.max_seq_len, stream());
    synchronize();
}

void DecodeStack::enqueue(int32_t pos, int32_t mode, bool follow_device_pos) {
    const bool with_qk_norm_rope = mode == kSeparateQkNormRope;
    LLMI_CHECK(!(follow_device_pos && with_qk_norm_rope));
    const bool fused_tail = mode == kFusedBlock;  // the block with attention + output projection in one launch
    const bool block = mode == kAttentionBlock || fused_tail;
    LLMI_CHECK(!block || hidden_dim_ > 0);
    const AttentionConfig& c = config_;
    tensor::Tensor& kc = buffers_->get_buffer(ModelBufferType::KeyCache);
    tensor::Tensor& vc = buffers_->get_buffer(ModelBufferType::ValueCache);
    tensor::Tensor& q = buffers_->get_buffer(ModelBufferType::Query);
    tensor::Tensor& ws = buffers_->get_buffer(ModelBufferType::KVSplitOutput);
    if (mode == kResidentStack) {
        LLMI_CHECK(!follow_device_pos);
        llmi_mha_stack_args t{};
        llmi_mha_args& m = t.first.mha;
        m.query = query_raw(0);
        m.key_cache = kc.ptr<uint16_t>();
        m.value_cache = vc.ptr<uint16_t>();
        m.workspace = ws.ptr<float>();
        m.workspace_bytes = ws.byte_size();
        m.output = output(0);
        m.layer_id = 0;
        m.pos = pos;
        m.kv_dim = c.kv_dim();
        m.kv_mul = c.kv_mul();
        m.head_num = c.head_num;
        m.head_dim = c.head_dim;
        m.max_seq_len = c.max_seq_len;
        m.kv_layout = c.kv_layout;
        const kernel::MhaHipOptions& o = kernel::mha_hip_options();
        m.force_path = o.force_path;
        m.num_splits = o.num_splits;
        m.waves_per_group = o.waves_per_group;
        m.stream = stream();
        m.workspace_side = kernel::workspace_side_of(m.workspace, m.workspace_bytes, stream());
        t.first.key_new = key_raw(0);
        t.first.value_new = value_raw(0);
        t.first.norm_weight = norm_weight(0);
        t.first.sin_cache = buffers_->get_buffer(ModelBufferType::SinCache).ptr<float>();
        t.first.cos_cache = buffers_->get_buffer(ModelBufferType::CosCache).ptr<float>();
        t.first.eps = 1e-6f;
        t.layer_count = c.layer_num;
        t.query_stride = c.dim();
        t.key_new_stride = c.kv_dim();
        t.value_new_stride = c.kv_dim();
        t.norm_weight_stride = 2 * c.head_dim;
        t.output_stride = c.dim();
        const int rc = llmi_hip_mha_decode_append_stack(&t);
        if (rc != LLMI_OK) LLMI_FATAL("llmi_hip_mha_decode_append_stack: " << llmi_hip_strerror(rc) << " " << llmi_hip_last_error());
        return;
    }
    for (int32_t layer = 0; layer < c.layer_num; ++layer) {
        const void* q_for_attention = query_raw(layer);
        if (with_qk_norm_rope) {
            llmi_qk_norm_rope_args a{};
            a.query = q.ptr<uint16_t>();
            a.query_src = query_raw(layer);
            a.key_new = key_raw(layer);
            a.value_new = value_raw(layer);
            a.key_cache = kc.ptr<uint16_t>();
            a.value_cache = vc.ptr<uint16_t>();
            a.norm_weight = norm_weight(layer);
            a.sin_cache = buffers_->get_buffer(ModelBufferType::SinCache).ptr<float>();
            a.cos_cache = buffers_->get_buffer(ModelBufferType::CosCache).ptr<float>();
            a.layer_id = layer;
            a.pos = pos;
            a.kv_dim = c.kv_dim();
            a.head_num = c.head_num;
            a.head_dim = c.head_dim;
            a.max_seq_len = c.max_seq_len;
            a.kv_layout = c.kv_layout;
            a.eps = 1e-6f;
            a.stream = stream();
            const int rc = llmi_hip_qk_norm_rope_append(&a);
            if (rc != LLMI_OK) LLMI_FATAL("llmi_hip_qk_norm_rope_append: " << llmi_hip_strerror(rc));
            q_for_attention = q.ptr<uint16_t>();
        }
        if (block) {
            llmi_qkv_gemv_args g{};
            g.input = hidden_in(layer);
            g.weight = qkv_weight(layer);
            g.query = query_raw(layer);
            g.key = key_raw(layer);
            g.value = value_raw(layer);
            g.dim = c.dim();
            g.kv_dim = c.kv_dim();
            g.k = hidden_dim_;
            g.stream = stream();
            const int rc = llmi_hip_qkv_gemv(&g);
            if (rc != LLMI_OK) LLMI_FATAL("llmi_hip_qkv_gemv: " << llmi_hip_strerror(rc));
        }
        llmi_mha_args m{};
        m.query = q_for_attention;
        m.key_cache = kc.ptr<uint16_t>();
        m.value_cache = vc.ptr<uint16_t>();
        m.workspace = ws.ptr<float>();
        m.workspace_bytes = ws.byte_size();
        m.output = output(layer);
        m.layer_id = layer;
        m.pos = pos;
        m.kv_dim = c.kv_dim();
        m.kv_mul = c.kv_mul();
        m.head_num = c.head_num;
        m.head_dim = c.head_dim;
        m.max_seq_len = c.max_seq_len;
        m.kv_layout = c.kv_layout;
        const kernel::MhaHipOptions& o = kernel::mha_hip_options();
        m.force_path = o.force_path;
        m.num_splits = o.num_splits;
        m.waves_per_group = o.waves_per_group;
        m.stream = stream();
        m.pos_device = follow_device_pos ? pos_dev_.ptr<int32_t>() : nullptr;
        m.workspace_side = kernel::workspace_side_of(m.workspace, m.workspace_bytes, stream());  // (measured once, before any capture)
        int rc;
        if (mode == kFusedAppend || block) {
            llmi_mha_append_args f{};
            f.mha = m;
            f.mha.query = query_raw(layer);
            f.key_new = key_raw(layer);
            f.value_new = value_raw(layer);
            f.norm_weight = norm_weight(layer);
            f.sin_cache = buffers_->get_buffer(ModelBufferType::SinCache).ptr<float>();
            f.cos_cache = buffers_->get_buffer(ModelBufferType::CosCache).ptr<float>();
            f.eps = 1e-6f;
            if (fused_tail) {
                llmi_attn_oproj_args t{};
                t.attn = f;
                t.o_weight = out_weight(layer);
                t.residual = residual();
                t.hidden = hidden_dim_;
                t.one_launch = 1;  // (this mode exists to run the one-launch form; the stack has the GPU to itself)
                rc = llmi_hip_mha_decode_append_oproj(&t);
            } else {
                rc = llmi_hip_mha_decode_append(&f);
            }
        } else {
            rc = llmi_hip_mha_decode(&m);
        }
        if (rc != LLMI_OK) LLMI_FATAL("decode attention: " << llmi_hip_strerror(rc) << " " << llmi_hip_last_error());
        if (block && !fused_tail) {
            llmi_gemv_args o{};
            o.input = output(layer);
            o.weight = out_weight(layer);
            o.output = residual();
            o.n = hidden_dim_;
            o.k = c.dim();
            o.mode = LLMI_GEMV_ADD_BF16;
            o.stream = stream();
            const int rc2 = llmi_hip_gemv(&o);
            if (rc2 != LLMI_OK) LLMI_FATAL("llmi_hip_gemv: " << llmi_hip_strerror(rc2));
        }
    }
}

void DecodeStack::set_position(int32_t pos) {
    // Synchronous small copy: the word is in place before anything enqueued afterwards runs.
    synchronize();
    const int rc = llmi_hip_memcpy(pos_dev_.ptr<int32_t>(), &pos, sizeof(pos), 1, nullptr, 1);
    if (rc != LLMI_OK) LLMI_FATAL("set_position: " << llmi_hip_strerror(rc));
}

void DecodeStack::capture(int32_t pos, int32_t mode, bool follow_device_pos) {
    if (graph_exec_) {
        HIP_OK(hipGraphExecDestroy(graph_exec_));
        graph_exec_ = nullptr;
    }
    if (graph_) {
        HIP_OK(hipGraphDestroy(graph_));
        graph_ = nullptr;
    }
    {   // the workspace's sides cannot be measured under capture: do it now if it has not been done
        tensor::Tensor& ws = buffers_->get_buffer(ModelBufferType::KVSplitOutput);
        (void)kernel::workspace_side_of(ws.ptr<float>(), ws.byte_size(), stream());
    }
    HIP_OK(hipStreamBeginCapture(stream(), hipStreamCaptureModeThreadLocal));
    try {
        enqueue(pos, mode, follow_device_pos);
    } catch (...) {
        hipGraph_t dead = nullptr;
        (void)hipStreamEndCapture(stream(), &dead);
        if (dead) (void)hipGraphDestroy(dead);
        throw;
    }
    HIP_OK(hipStreamEndCapture(stream(), &graph_));
    HIP_OK(hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0));
}

float DecodeStack::replay(int32_t times) {
    LLMI_CHECK(graph_exec_ != nullptr);
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    HIP_OK(hipEventRecord(e0, stream()));
    for (int32_t i = 0; i < times; ++i) HIP_OK(hipGraphLaunch(graph_exec_, stream()));
    HIP_OK(hipEventRecord(e1, stream()));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0.0f;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    return ms;
}

void DecodeStack::synchronize() { HIP_OK(hipStreamSynchronize(stream())); }

}  // namespace model
