#include "kernel_interface.h"

#include <map>
#include <mutex>
#include <utility>

#include "llmi_hip.h"

namespace kernel {

namespace {
MHAKernel g_cpu_mha = nullptr;

// Same conversion trick the reference relies on: the HIP kernel's parameter
// list has the same types as MHAKernel, only the meaning of slots 2-4 differs.
void mha_kernel_hip_slot(const tensor::Tensor& query, const tensor::Tensor& key_cache,
                         const tensor::Tensor& value_cache, const tensor::Tensor& kv_split_output,
                         const tensor::Tensor& output, int32_t layer_id, int32_t pos, int32_t kv_dim, int32_t kv_mul,
                         int32_t head_num, int32_t head_dim, int32_t max_seq_len, void* stream) {
    mha_kernel_hip(query, key_cache, value_cache, kv_split_output, output, layer_id, pos, kv_dim, kv_mul, head_num,
                   head_dim, max_seq_len, stream);
}
}  // namespace

// The library this layer was linked against must speak the ABI of the header it was compiled with: a struct that
// grew since would be read past its end. Checked once, the first time a HIP arm is handed out.
static void ensure_abi() {
    static const bool ok = [] {
        const int got = llmi_hip_abi_version();
        if (got != LLMI_HIP_ABI_VERSION)
            LLMI_FATAL("libllmi_hip.so speaks ABI version " << got << ", this host layer was built for " << LLMI_HIP_ABI_VERSION);
        return true;
    }();
    (void)ok;
}

MHAKernel get_mha_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return mha_kernel_hip_slot;
    }
    if (device_type == base::DeviceType::DeviceCPU && g_cpu_mha) return g_cpu_mha;
    LLMI_FATAL("Unknown device type for get a mha kernel.");
}

void register_mha_kernel(base::DeviceType device_type, MHAKernel fn) {
    if (device_type != base::DeviceType::DeviceCPU) LLMI_FATAL("only the CPU arm of the mha kernel can be registered");
    g_cpu_mha = fn;
}

FusedQKNormRoPEKernel get_fused_qk_norm_rope_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return fused_qk_norm_rope_kernel_hip;
    }
    LLMI_FATAL("Unknown device type for get a fused_qk_norm_rope kernel.");  // kernel_interface.cpp:172-178: GPU only
}

SinCosCacheKernel get_sin_cos_cache_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return sin_cos_cache_precompute_hip;
    }
    LLMI_FATAL("Unknown device type for get a sin_cos_cache kernel.");
}

GEMVKernel get_gemv_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return gemv_kernel_hip;
    }
    LLMI_FATAL("Unknown device type for get a gemv kernel.");
}

FusedGEMVAddKernel get_fused_gemv_add_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return fused_gemv_add_kernel_hip;
    }
    LLMI_FATAL("Unknown device type for get a fused_gemv_add kernel.");
}

FusedQKVGEMVKernel get_fused_qkv_gemv_kernel(base::DeviceType device_type) {
    if (device_type == base::DeviceType::DeviceHIP) {
        ensure_abi();
        return fused_qkv_gemv_kernel_hip;
    }
    LLMI_FATAL("Unknown device type for get a fused_qkv_gemv kernel.");
}

MhaHipOptions& mha_hip_options() {
    static MhaHipOptions opts;
    return opts;
}

static void fail_on(int rc, const char* what) {
    if (rc != LLMI_OK)
        LLMI_FATAL(what << " failed with status " << rc << " (" << llmi_hip_strerror(rc) << ") " << llmi_hip_last_error());
}

int32_t workspace_side_of(const void* workspace, size_t bytes, void* stream) {
    static std::mutex mu;
    static std::map<const void*, std::pair<size_t, int32_t>> known;
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find(workspace);
    if (it != known.end() && it->second.first == bytes) return it->second.second;
    int32_t sides = 0;
    if (llmi_hip_mha_workspace_side(const_cast<void*>(workspace), bytes, stream, &sides) != LLMI_OK)
        return 0;  // under capture, or too small to measure: the plain layout this time, nothing remembered
    known[workspace] = {bytes, sides};
    return sides;
}

void mha_kernel_hip(const tensor::Tensor& query, const tensor::Tensor& key_cache, const tensor::Tensor& value_cache,
                    const tensor::Tensor& kv_split_output, const tensor::Tensor& output, int32_t layer_id,
                    int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num, int32_t head_dim,
                    int32_t max_seq_len, void* stream) {
    // mha_kernel.cu:455-471: emptiness, dtype and device of every operand.
    LLMI_CHECK(!query.is_empty() && !key_cache.is_empty() && !value_cache.is_empty());
    LLMI_CHECK(!kv_split_output.is_empty() && !output.is_empty());
    LLMI_CHECK(query.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(key_cache.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(value_cache.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(kv_split_output.data_type() == base::DataType::DataTypeFp32);
    LLMI_CHECK(output.data_type() == base::DataType::DataTypeBf16);
    for (const tensor::Tensor* t : {&query, &key_cache, &value_cache, &kv_split_output, &output})
        LLMI_CHECK(t->device_type() == base::DeviceType::DeviceHIP);
    LLMI_CHECK(key_cache.dims_size() == value_cache.dims_size());
    // The cache must hold the layer that is asked for (the reference trusts the caller here).
    LLMI_CHECK(key_cache.size() >= static_cast<size_t>(layer_id + 1) * max_seq_len * kv_dim);
    LLMI_CHECK(value_cache.size() >= static_cast<size_t>(layer_id + 1) * max_seq_len * kv_dim);

    llmi_mha_args a{};
    a.query = query.ptr<uint16_t>();
    a.key_cache = key_cache.ptr<uint16_t>();
    a.value_cache = value_cache.ptr<uint16_t>();
    a.workspace = const_cast<float*>(kv_split_output.ptr<float>());
    a.workspace_bytes = kv_split_output.byte_size();
    a.output = const_cast<uint16_t*>(output.ptr<uint16_t>());
    a.output_f32 = nullptr;
    a.layer_id = layer_id;
    a.pos = pos;
    a.kv_dim = kv_dim;
    a.kv_mul = kv_mul;
    a.head_num = head_num;
    a.head_dim = head_dim;
    a.max_seq_len = max_seq_len;
    a.kv_layout = key_cache.dims_size() == 4 ? LLMI_KV_LAYOUT_HEAD_MAJOR : LLMI_KV_LAYOUT_POS_MAJOR;
    const MhaHipOptions& o = mha_hip_options();
    a.force_path = o.force_path;
    a.num_splits = o.num_splits;
    a.waves_per_group = o.waves_per_group;
    a.stream = stream;
    a.workspace_side = workspace_side_of(a.workspace, a.workspace_bytes, stream);
    fail_on(llmi_hip_mha_decode(&a), "llmi_hip_mha_decode");
}

void fused_qk_norm_rope_kernel_hip(const tensor::Tensor& query, const tensor::Tensor& key,
                                   const tensor::Tensor& weight, const tensor::Tensor& token_pos,
                                   const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache, int32_t dim,
                                   int32_t kv_dim, int32_t head_dim, void* stream) {
    // rmsnorm_kernel.cu:260-274
    LLMI_CHECK(query.data_type() == base::DataType::DataTypeBf16 && key.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(weight.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(token_pos.data_type() == base::DataType::DataTypeInt32);
    LLMI_CHECK(sin_cache.data_type() == base::DataType::DataTypeFp32 && cos_cache.data_type() == base::DataType::DataTypeFp32);
    LLMI_CHECK(query.device_type() == base::DeviceType::DeviceHIP && key.device_type() == base::DeviceType::DeviceHIP);
    LLMI_CHECK(weight.device_type() == base::DeviceType::DeviceHIP);
    LLMI_CHECK(token_pos.device_type() == base::DeviceType::DeviceCPU);  // read on the host (rmsnorm_kernel.cu:281)
    LLMI_CHECK(sin_cache.device_type() == base::DeviceType::DeviceHIP && cos_cache.device_type() == base::DeviceType::DeviceHIP);
    const int32_t pos = token_pos.index<int32_t>(0);
    LLMI_CHECK(pos >= 0 && static_cast<size_t>(pos + 1) * (head_dim / 2) <= sin_cache.size());

    // In place on the query and on `key`, which in the reference is the K-cache
    // row of this token (position-major slice): hand the row in as a one-row
    // "cache" so that slot (layer 0, pos 0) is the row itself, and point the
    // sin/cos tables at this position's row.
    llmi_qk_norm_rope_args a{};
    a.query = const_cast<uint16_t*>(query.ptr<uint16_t>());
    a.query_src = nullptr;
    a.key_new = key.ptr<uint16_t>();
    a.value_new = nullptr;
    a.key_cache = const_cast<uint16_t*>(key.ptr<uint16_t>());
    a.value_cache = nullptr;
    a.norm_weight = weight.ptr<uint16_t>();
    a.sin_cache = sin_cache.ptr<float>(static_cast<int64_t>(pos) * (head_dim / 2));
    a.cos_cache = cos_cache.ptr<float>(static_cast<int64_t>(pos) * (head_dim / 2));
    a.layer_id = 0;
    a.pos = 0;
    a.kv_dim = kv_dim;
    a.head_num = dim / head_dim;
    a.head_dim = head_dim;
    a.max_seq_len = 1;
    a.kv_layout = LLMI_KV_LAYOUT_POS_MAJOR;
    a.eps = 1e-6f;  // rmsnorm_kernel.cu:284
    a.stream = stream;
    fail_on(llmi_hip_qk_norm_rope_append(&a), "llmi_hip_qk_norm_rope_append");
}

void sin_cos_cache_precompute_hip(const tensor::Tensor& sin_cache, const tensor::Tensor& cos_cache, int32_t head_dim,
                                  int32_t max_seq_len, void* stream) {
    LLMI_CHECK(!sin_cache.is_empty() && !cos_cache.is_empty());  // rope_kernel.cu:30-37
    LLMI_CHECK(sin_cache.data_type() == base::DataType::DataTypeFp32 && cos_cache.data_type() == base::DataType::DataTypeFp32);
    LLMI_CHECK(sin_cache.device_type() == base::DeviceType::DeviceHIP && cos_cache.device_type() == base::DeviceType::DeviceHIP);
    LLMI_CHECK(sin_cache.size() >= static_cast<size_t>(max_seq_len) * (head_dim / 2));
    LLMI_CHECK(cos_cache.size() >= static_cast<size_t>(max_seq_len) * (head_dim / 2));
    fail_on(llmi_hip_sincos_table(const_cast<float*>(sin_cache.ptr<float>()), const_cast<float*>(cos_cache.ptr<float>()),
                                  head_dim, max_seq_len, stream),
            "llmi_hip_sincos_table");
}

// matmul_kernel.cu:107-128: shapes, dtypes and devices of a GEMV's operands.
static void check_gemv_operands(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& output,
                                base::DataType out_type) {
    LLMI_CHECK(!input.is_empty() && input.dims_size() == 1);
    LLMI_CHECK(!weight.is_empty() && weight.dims_size() == 2);
    LLMI_CHECK(!output.is_empty() && output.dims_size() == 1);
    LLMI_CHECK(input.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(weight.data_type() == base::DataType::DataTypeBf16);
    LLMI_CHECK(output.data_type() == out_type);
    for (const tensor::Tensor* t : {&input, &weight, &output}) LLMI_CHECK(t->device_type() == base::DeviceType::DeviceHIP);
    LLMI_CHECK(input.get_dim(0) == weight.get_dim(1));
}

static void run_gemv(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& output,
                     int32_t mode, void* stream) {
    LLMI_CHECK(output.get_dim(0) == weight.get_dim(0));
    llmi_gemv_args a{};
    a.input = input.ptr<uint16_t>();
    a.weight = weight.ptr<uint16_t>();
    a.output = const_cast<void*>(static_cast<const void*>(output.ptr<uint8_t>()));  // outputs arrive const, like the reference's
    a.n = weight.get_dim(0);
    a.k = weight.get_dim(1);
    a.mode = mode;
    a.stream = stream;
    fail_on(llmi_hip_gemv(&a), "llmi_hip_gemv");
}

void gemv_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& output,
                     bool lm_head, void* stream) {
    check_gemv_operands(input, weight, output, lm_head ? base::DataType::DataTypeFp32 : base::DataType::DataTypeBf16);
    run_gemv(input, weight, output, lm_head ? LLMI_GEMV_OUT_F32 : LLMI_GEMV_OUT_BF16, stream);
}

void fused_gemv_add_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight,
                               const tensor::Tensor& output, void* stream) {
    check_gemv_operands(input, weight, output, base::DataType::DataTypeBf16);
    run_gemv(input, weight, output, LLMI_GEMV_ADD_BF16, stream);
}

void fused_qkv_gemv_kernel_hip(const tensor::Tensor& input, const tensor::Tensor& weight, const tensor::Tensor& query,
                               const tensor::Tensor& key, const tensor::Tensor& value, void* stream) {
    // matmul_kernel.cu:256-292
    LLMI_CHECK(!input.is_empty() && input.dims_size() == 1);
    LLMI_CHECK(!weight.is_empty() && weight.dims_size() == 2);
    for (const tensor::Tensor* t : {&query, &key, &value}) LLMI_CHECK(!t->is_empty() && t->dims_size() == 1);
    for (const tensor::Tensor* t : {&input, &weight, &query, &key, &value}) {
        LLMI_CHECK(t->data_type() == base::DataType::DataTypeBf16);
        LLMI_CHECK(t->device_type() == base::DeviceType::DeviceHIP);
    }
    const int32_t dim = query.get_dim(0), kv_dim = key.get_dim(0);
    LLMI_CHECK(value.get_dim(0) == kv_dim);
    LLMI_CHECK(weight.get_dim(0) == dim + 2 * kv_dim);
    LLMI_CHECK(weight.get_dim(1) == input.get_dim(0));
    llmi_qkv_gemv_args a{};
    a.input = input.ptr<uint16_t>();
    a.weight = weight.ptr<uint16_t>();
    a.query = const_cast<uint16_t*>(query.ptr<uint16_t>());
    a.key = const_cast<uint16_t*>(key.ptr<uint16_t>());
    a.value = const_cast<uint16_t*>(value.ptr<uint16_t>());
    a.dim = dim;
    a.kv_dim = kv_dim;
    a.k = weight.get_dim(1);
    a.stream = stream;
    fail_on(llmi_hip_qkv_gemv(&a), "llmi_hip_qkv_gemv");
}

}  // namespace kernel
