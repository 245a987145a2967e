#include "host_hooks.h"

#include <cstring>
#include <string>

#include "decode_stack.h"
#include "kernel_interface.h"
#include "mha.h"

struct llmi_host_stack {
    std::unique_ptr<model::DecodeStack> impl;
};

namespace {
thread_local std::string g_err;

template <typename F>
int guarded(F&& f) {
    try {
        f();
        g_err.clear();
        return 0;
    } catch (const std::exception& e) {
        g_err = e.what();
        return -1;
    }
}
}  // namespace

extern "C" {

const char* llmi_host_last_error(void) { return g_err.c_str(); }

llmi_host_stack* llmi_host_stack_create(int32_t layer_num, int32_t max_seq_len, int32_t head_num,
                                        int32_t kv_head_num, int32_t kv_layout) {
    llmi_host_stack* s = nullptr;
    guarded([&] {
        model::AttentionConfig c;
        c.layer_num = layer_num;
        c.max_seq_len = max_seq_len;
        c.head_num = head_num;
        c.kv_head_num = kv_head_num;
        c.kv_layout = kv_layout;
        auto impl = std::make_unique<model::DecodeStack>(c);
        s = new llmi_host_stack{std::move(impl)};
    });
    return s;
}

void llmi_host_stack_destroy(llmi_host_stack* s) { delete s; }

void* llmi_host_stack_ptr(llmi_host_stack* s, int32_t which, int32_t layer) {
    void* p = nullptr;
    guarded([&] {
        model::DecodeStack& d = *s->impl;
        using model::ModelBufferType;
        switch (which) {
            case 0: p = d.buffers().get_buffer(ModelBufferType::KeyCache).ptr<uint16_t>(); break;
            case 1: p = d.buffers().get_buffer(ModelBufferType::ValueCache).ptr<uint16_t>(); break;
            case 2: p = d.query_raw(layer); break;
            case 3: p = d.key_raw(layer); break;
            case 4: p = d.value_raw(layer); break;
            case 5: p = d.norm_weight(layer); break;
            case 6: p = d.output(layer); break;
            case 7: p = d.buffers().get_buffer(ModelBufferType::SinCache).ptr<float>(); break;
            case 8: p = d.buffers().get_buffer(ModelBufferType::CosCache).ptr<float>(); break;
            case 9: p = d.buffers().get_buffer(ModelBufferType::Query).ptr<uint16_t>(); break;
            case 10: p = d.qkv_weight(layer); break;
            case 11: p = d.out_weight(layer); break;
            case 12: p = d.hidden_in(layer); break;
            case 13: p = d.residual(); break;
            default: LLMI_FATAL("unknown pointer selector " << which);
        }
    });
    return p;
}

int llmi_host_stack_enable_projections(llmi_host_stack* s, int32_t hidden_dim) {
    return guarded([&] { s->impl->enable_projections(hidden_dim); });
}

int llmi_host_stack_build_sincos(llmi_host_stack* s) { return guarded([&] { s->impl->build_sincos(); }); }

int llmi_host_stack_run(llmi_host_stack* s, int32_t pos, int32_t with_qk_norm_rope) {
    return guarded([&] {
        s->impl->enqueue(pos, with_qk_norm_rope);
        s->impl->synchronize();
    });
}

int llmi_host_stack_capture(llmi_host_stack* s, int32_t pos, int32_t with_qk_norm_rope) {
    return guarded([&] { s->impl->capture(pos, with_qk_norm_rope); });
}

int llmi_host_stack_capture_following(llmi_host_stack* s, int32_t max_pos, int32_t mode) {
    return guarded([&] { s->impl->capture(max_pos, mode, true); });
}

int llmi_host_stack_set_pos(llmi_host_stack* s, int32_t pos) {
    return guarded([&] { s->impl->set_position(pos); });
}

int llmi_host_stack_replay(llmi_host_stack* s, int32_t times, float* elapsed_ms) {
    return guarded([&] {
        const float ms = s->impl->replay(times);
        if (elapsed_ms) *elapsed_ms = ms;
    });
}

int llmi_host_stack_load_weights(llmi_host_stack* s, const char* path) {
    int code = -1;
    const int rc = guarded([&] {
        std::unique_ptr<model::WeightFile> file;
        base::Status st = model::WeightFile::open(path ? path : "", &file);
        if (st) st = s->impl->load_weights(*file);
        code = int(st);
        if (!st) g_err = st.get_err_msg();
    });
    return rc != 0 ? rc : code;
}

int llmi_host_weight_file_info(const char* path, int32_t header_ints, int64_t info[12], void* payload_out,
                               int64_t payload_bytes) {
    int code = -1;
    std::string msg;
    const int rc = guarded([&] {
        std::unique_ptr<model::WeightFile> file;
        const base::Status st = model::WeightFile::open(path ? path : "", &file, header_ints);
        code = int(st);
        msg = st.get_err_msg();
        if (!st) return;
        const model::ModelConfig& c = file->config();
        const int32_t raw[8] = {c.dim, c.hidden_dim, c.layer_num, c.head_num, c.kv_head_num, c.vocab_size, c.max_seq_len, c.immediate_dim};
        for (int i = 0; i < 8; ++i) info[i] = raw[i];
        info[8] = file->head_dim();
        info[9] = file->kv_dim();
        info[10] = file->vocab_size();
        info[11] = static_cast<int64_t>(file->payload_elements());
        if (payload_out && payload_bytes > 0) {
            const size_t have = file->payload_elements() * sizeof(uint16_t);
            std::memcpy(payload_out, file->payload_bytes(), static_cast<size_t>(payload_bytes) < have ? static_cast<size_t>(payload_bytes) : have);
        }
    });
    if (rc == 0 && code != 0) g_err = msg;
    return rc != 0 ? rc : code;
}

void llmi_host_set_mha_options(int32_t force_path, int32_t num_splits, int32_t waves_per_group) {
    kernel::MhaHipOptions& o = kernel::mha_hip_options();
    o.force_path = force_path;
    o.num_splits = num_splits;
    o.waves_per_group = waves_per_group;
}

int llmi_host_mha_forward(void* query, void* key_cache, void* value_cache, void* workspace, int64_t workspace_floats,
                          void* output, int32_t layer_num, int32_t layer_id, int32_t pos, int32_t kv_dim,
                          int32_t kv_mul, int32_t head_num, int32_t head_dim, int32_t max_seq_len,
                          int32_t cache_dims) {
    int status_code = -1;
    const int rc = guarded([&] {
        using base::DataType;
        const base::DeviceType dev = base::DeviceType::DeviceHIP;
        auto view = [&](DataType dt, std::vector<int32_t> dims, void* p) {
            tensor::Tensor t(dt, std::move(dims), false, nullptr, p);
            t.set_device_type(dev);
            return t;
        };
        const int32_t n_kv = kv_dim / head_dim;
        tensor::Tensor q = view(DataType::DataTypeBf16, {head_num * head_dim}, query);
        std::vector<int32_t> cdims = cache_dims == 4 ? std::vector<int32_t>{layer_num, n_kv, max_seq_len, head_dim}
                                                     : std::vector<int32_t>{layer_num, max_seq_len, kv_dim};
        tensor::Tensor kc = view(DataType::DataTypeBf16, cdims, key_cache);
        tensor::Tensor vc = view(DataType::DataTypeBf16, cdims, value_cache);
        tensor::Tensor ws = view(DataType::DataTypeFp32, {head_num, static_cast<int32_t>(workspace_floats / head_num)}, workspace);
        tensor::Tensor out = view(DataType::DataTypeBf16, {head_num * head_dim}, output);
        op::MultiHeadAttention mha(dev, kv_dim, kv_mul, head_num, head_dim, max_seq_len);
        auto cfg = std::make_shared<kernel::HipConfig>();
        cfg->create();
        mha.set_hip_config(cfg);
        mha.set_pos(pos);
        mha.set_layer_id(layer_id);
        const base::Status st = mha.forward(q, kc, vc, ws, out);
        if (st) {
            const hipError_t e = hipStreamSynchronize(cfg->stream);
            if (e != hipSuccess) LLMI_FATAL("hipStreamSynchronize: " << hipGetErrorString(e));
        } else {
            g_err = st.get_err_msg();
        }
        status_code = int(st);
    });
    return rc == 0 ? status_code : -1;
}

}  // extern "C"
