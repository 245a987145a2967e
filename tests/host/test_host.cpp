// Unit tests of the C++ host layer (tensor / buffer / allocator / op layer / registry), in the spirit of the
// reference's gtest suite (test/test_tensor/test_tensor.cpp, test_buffer.cpp, test/test_op/test_op_mha.cpp):
// the same operation through the registry's CPU arm and its GPU arm on cloned tensors. The CPU arm used here
// is the CPU oracle, registered by this test program; the product library ships none.
//
//   host_tests cpu   tests that need no GPU
//   host_tests gpu   tests that need one
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <vector>

#include "attention_buffers.h"
#include "decode_stack.h"
#include "kernel_interface.h"
#include "llmi_hip.h"
#include "llmi_internal.h"
#include "llmi_oracle.h"
#include "mha.h"
#include "qk_norm_rope.h"

namespace {
struct TestCase {
    std::string name;
    std::function<void()> fn;
};
std::vector<TestCase>& registry() {
    static std::vector<TestCase> r;
    return r;
}
struct Registrar {
    Registrar(const char* name, std::function<void()> fn) { registry().push_back({name, std::move(fn)}); }
};
#define TEST(name)                                   \
    static void test_##name();                       \
    static Registrar registrar_##name(#name, test_##name); \
    static void test_##name()
#define EXPECT(cond)                                                                   \
    do {                                                                               \
        if (!(cond)) throw std::runtime_error(std::string("EXPECT failed: " #cond " at line ") + std::to_string(__LINE__)); \
    } while (0)
template <typename F>
bool is_fatal(F&& f) {
    try {
        f();
    } catch (const base::FatalError&) {
        return true;
    }
    return false;
}

using base::DataType;
using base::DeviceType;
auto cpu_alloc() { return base::CPUDeviceAllocatorFactory::get_instance(); }
auto hip_alloc() { return base::HIPDeviceAllocatorFactory::get_instance(); }

// CPU arm of the MHA registry slot = the oracle, CPU argument order (query, score, key, value, output).
void oracle_mha_cpu_arm(const tensor::Tensor& query, const tensor::Tensor& score, const tensor::Tensor& key_cache,
                        const tensor::Tensor& value_cache, const tensor::Tensor& output, int32_t layer_id,
                        int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num, int32_t head_dim,
                        int32_t max_seq_len, void*) {
    LLMI_CHECK(query.device_type() == DeviceType::DeviceCPU && output.device_type() == DeviceType::DeviceCPU);
    int rc;
    if (query.data_type() == DataType::DataTypeFp32) {
        rc = llmi_oracle_mha_cpu(query.ptr<float>(), const_cast<float*>(score.ptr<float>()), key_cache.ptr<float>(),
                                 value_cache.ptr<float>(), const_cast<float*>(output.ptr<float>()), layer_id, pos,
                                 kv_dim, kv_mul, head_num, head_dim, max_seq_len);
    } else {
        rc = llmi_oracle_mha_cpu_bf16(query.ptr<uint16_t>(), const_cast<float*>(score.ptr<float>()),
                                      key_cache.ptr<uint16_t>(), value_cache.ptr<uint16_t>(),
                                      const_cast<float*>(output.ptr<float>()), layer_id, pos, kv_dim, kv_mul, head_num,
                                      head_dim, max_seq_len);
    }
    LLMI_CHECK(rc == 0);
}

void fill_bf16_normal(tensor::Tensor& t, std::mt19937& rng, bool rms_norm) {
    std::normal_distribution<float> nd(0.0f, 1.0f);
    uint16_t* p = t.ptr<uint16_t>();
    std::vector<float> row(128);
    for (size_t i = 0; i < t.size(); i += 128) {
        float ss = 0;
        for (int j = 0; j < 128; ++j) {
            row[j] = nd(rng);
            ss += row[j] * row[j];
        }
        const float r = rms_norm ? 1.0f / std::sqrt(ss / 128.0f) : 1.0f;
        for (int j = 0; j < 128; ++j) p[i + j] = llmi_oracle_f32_to_bf16(row[j] * r);
    }
}
}  // namespace

// ------------------------------------------------------------------ no GPU
TEST(cpu_tensor_dims_strides_size) {
    tensor::Tensor t(DataType::DataTypeFp32, 2, 3, 4, true, cpu_alloc());
    EXPECT(!t.is_empty() && t.size() == 24 && t.byte_size() == 96 && t.dims_size() == 3);
    EXPECT(t.get_dim(0) == 2 && t.get_dim(2) == 4);
    auto s = t.strides();
    EXPECT(s.size() == 3 && s[0] == 12 && s[1] == 4 && s[2] == 1);
    EXPECT(t.device_type() == DeviceType::DeviceCPU && t.data_type() == DataType::DataTypeFp32);
    EXPECT(is_fatal([&] { t.get_dim(3); }));
    EXPECT(is_fatal([&] { t.index<float>(24); }));
    tensor::Tensor b(DataType::DataTypeBf16, 7, true, cpu_alloc());
    EXPECT(b.byte_size() == 14);
    tensor::Tensor empty;
    EXPECT(empty.is_empty() && empty.ptr<float>() == nullptr);
}

TEST(cpu_tensor_external_adopted_and_assigned_buffers) {
    std::vector<float> mem(8, 1.5f);
    tensor::Tensor view(DataType::DataTypeFp32, 8, false, nullptr, mem.data());  // borrowed
    EXPECT(view.get_buffer()->is_external() && view.ptr<float>() == mem.data());
    EXPECT(view.device_type() == DeviceType::DeviceUnknown);
    view.set_device_type(DeviceType::DeviceCPU);
    EXPECT(view.device_type() == DeviceType::DeviceCPU && view.index<float>(3) == 1.5f);
    EXPECT(is_fatal([&] { tensor::Tensor bad(DataType::DataTypeFp32, 8, true, nullptr, nullptr); }));  // need_alloc without allocator
    tensor::Tensor unbacked(DataType::DataTypeFp32, 8);  // no allocator, no pointer: waits for assgin
    EXPECT(unbacked.is_empty());
    auto buf = std::make_shared<base::Buffer>(32, cpu_alloc());
    EXPECT(unbacked.assgin(buf) && !unbacked.is_empty());
    auto small = std::make_shared<base::Buffer>(16, cpu_alloc());
    EXPECT(!unbacked.assgin(small));  // too small for 8 floats
    EXPECT(!unbacked.assgin(nullptr));
}

TEST(cpu_tensor_clone_reshape_reset) {
    tensor::Tensor t(DataType::DataTypeInt32, 4, true, cpu_alloc());
    for (int i = 0; i < 4; ++i) t.index<int32_t>(i) = i * 10;
    tensor::Tensor c = t.clone();
    EXPECT(c.ptr<int32_t>() != t.ptr<int32_t>() && c.index<int32_t>(3) == 30);
    c.index<int32_t>(3) = 7;
    EXPECT(t.index<int32_t>(3) == 30);  // deep copy
    tensor::Tensor shared = t;          // value copy shares the buffer
    EXPECT(shared.ptr<int32_t>() == t.ptr<int32_t>());
    t.reshape({2, 2});
    EXPECT(t.dims_size() == 2 && t.size() == 4 && t.index<int32_t>(2) == 20);
    t.reshape({3, 3});                  // grows: contents carried over
    EXPECT(t.size() == 9 && t.index<int32_t>(1) == 10);
    t.reset(DataType::DataTypeFp32, {5});
    EXPECT(t.is_empty() && t.size() == 5 && t.data_type() == DataType::DataTypeFp32);
    EXPECT(t.allocate(cpu_alloc(), false) && !t.is_empty());
    EXPECT(!t.allocate(nullptr, false));
}

TEST(cpu_buffer_ownership_and_copy) {
    auto a = std::make_shared<base::Buffer>(16, cpu_alloc());
    EXPECT(a->ptr() != nullptr && !a->is_external() && a->device_type() == DeviceType::DeviceCPU);
    std::memset(a->ptr(), 0xAB, 16);
    base::Buffer b(8, cpu_alloc());
    b.copy_from(*a);  // copies min(8, 16) bytes
    EXPECT(static_cast<unsigned char*>(b.ptr())[7] == 0xAB);
    char ext[4] = {1, 2, 3, 4};
    base::Buffer e(4, nullptr, ext, true);
    EXPECT(e.is_external() && e.ptr() == ext && !e.allocate());
    EXPECT(is_fatal([&] { e.copy_from(*a); }));  // no allocator to copy with
    base::Buffer zero(0, cpu_alloc());
    EXPECT(zero.ptr() == nullptr && !zero.allocate());
}

TEST(cpu_status_and_fatal) {
    base::Status ok = base::error::success();
    base::Status bad = base::error::invalid_argument("nope");
    EXPECT(ok && !bad && int(bad) == 7 && bad.get_err_msg() == "nope" && bad == base::StatusCode::InvalidArgument);
    EXPECT(is_fatal([&] { STATUS_CHECK(bad); }));
    EXPECT(!is_fatal([&] { STATUS_CHECK(ok); }));
    EXPECT(base::data_type_size(DataType::DataTypeBf16) == 2 && base::data_type_size(DataType::DataTypeFp32) == 4);
    EXPECT(is_fatal([] { base::data_type_size(DataType::DataTypeUnknown); }));
    EXPECT(int(DeviceType::DeviceHIP) == 1 && int(DeviceType::DeviceCPU) == 2);  // DeviceHIP sits where DeviceCUDA sat
}

TEST(cpu_mha_layer_check_rejects_bad_tensors) {
    // check() runs before any kernel is chosen, so the op can be exercised on the host with CPU tensors.
    const int32_t n_q = 8, n_kv = 2, d = 128, msl = 32, kv_dim = n_kv * d;
    op::MultiHeadAttention mha(DeviceType::DeviceCPU, kv_dim, n_q / n_kv, n_q, d, msl);
    EXPECT(mha.inputs_size() == 4 && mha.outputs_size() == 1 && mha.data_type() == DataType::DataTypeBf16);
    tensor::Tensor q(DataType::DataTypeBf16, n_q * d, true, cpu_alloc());
    tensor::Tensor kc(DataType::DataTypeBf16, 1, msl, kv_dim, true, cpu_alloc());
    tensor::Tensor vc(DataType::DataTypeBf16, 1, msl, kv_dim, true, cpu_alloc());
    tensor::Tensor ws(DataType::DataTypeFp32, n_q, 4 * msl, true, cpu_alloc());
    tensor::Tensor out(DataType::DataTypeBf16, n_q * d, true, cpu_alloc());
    auto set_all = [&] {
        mha.set_input(0, q); mha.set_input(1, kc); mha.set_input(2, vc); mha.set_input(3, ws); mha.set_output(0, out);
    };
    set_all();
    EXPECT(mha.check());
    tensor::Tensor q_bad(DataType::DataTypeBf16, n_q * d - 1, true, cpu_alloc());
    mha.set_input(0, q_bad);
    EXPECT(mha.check() == base::StatusCode::InvalidArgument);
    set_all();
    tensor::Tensor q_f32(DataType::DataTypeFp32, n_q * d, true, cpu_alloc());
    mha.set_input(0, q_f32);
    EXPECT(!mha.check());  // wrong dtype
    set_all();
    tensor::Tensor ws_small(DataType::DataTypeFp32, n_q, 4 * msl - 1, true, cpu_alloc());
    mha.set_input(3, ws_small);
    EXPECT(!mha.check());
    set_all();
    tensor::Tensor ws_bf16(DataType::DataTypeBf16, n_q, 4 * msl, true, cpu_alloc());
    mha.set_input(3, ws_bf16);
    EXPECT(!mha.check());
    set_all();
    mha.set_input(1, tensor::Tensor());
    EXPECT(!mha.check());  // empty key cache
    set_all();
    mha.set_device_type(DeviceType::DeviceHIP);
    EXPECT(!mha.check());  // tensors are on the CPU, layer says HIP
    EXPECT(is_fatal([&] { mha.set_input(4, q); }));
}

TEST(cpu_registry_arms) {
    kernel::register_mha_kernel(DeviceType::DeviceCPU, nullptr);
    EXPECT(is_fatal([] { kernel::get_mha_kernel(DeviceType::DeviceCPU); }));       // no CPU compute in the product
    EXPECT(is_fatal([] { kernel::get_mha_kernel(DeviceType::DeviceUnknown); }));   // kernel_interface.cpp:186-189
    EXPECT(kernel::get_mha_kernel(DeviceType::DeviceHIP) != nullptr);
    EXPECT(kernel::get_fused_qk_norm_rope_kernel(DeviceType::DeviceHIP) != nullptr);
    EXPECT(is_fatal([] { kernel::get_fused_qk_norm_rope_kernel(DeviceType::DeviceCPU); }));
    EXPECT(is_fatal([] { kernel::get_sin_cos_cache_kernel(DeviceType::DeviceCPU); }));
    EXPECT(kernel::get_gemv_kernel(DeviceType::DeviceHIP) != nullptr);
    EXPECT(kernel::get_fused_gemv_add_kernel(DeviceType::DeviceHIP) != nullptr);
    EXPECT(kernel::get_fused_qkv_gemv_kernel(DeviceType::DeviceHIP) != nullptr);
    EXPECT(is_fatal([] { kernel::get_gemv_kernel(DeviceType::DeviceCPU); }));
    EXPECT(is_fatal([] { kernel::get_fused_qkv_gemv_kernel(DeviceType::DeviceUnknown); }));
    EXPECT(is_fatal([] { kernel::register_mha_kernel(DeviceType::DeviceHIP, oracle_mha_cpu_arm); }));
    kernel::register_mha_kernel(DeviceType::DeviceCPU, oracle_mha_cpu_arm);
    EXPECT(kernel::get_mha_kernel(DeviceType::DeviceCPU) == oracle_mha_cpu_arm);
}

TEST(cpu_plumbing_config_through_the_registry_cpu_arm) {
    // 16 Q / 8 KV heads, head_dim 128, 256 cached + 1 new position, fp32, called the way the reference's
    // gtest calls the CPU op: get_mha_kernel(DeviceCPU)(q, score, k, v, out, ...) (test_op_mha.cpp:55-56).
    kernel::register_mha_kernel(DeviceType::DeviceCPU, oracle_mha_cpu_arm);
    const int32_t n_q = 16, n_kv = 8, d = 128, msl = 512, pos = 256, kv_dim = n_kv * d, layers = 3, layer_id = 2;
    tensor::Tensor q(DataType::DataTypeFp32, n_q * d, true, cpu_alloc());
    tensor::Tensor score(DataType::DataTypeFp32, n_q, msl, true, cpu_alloc());
    tensor::Tensor k(DataType::DataTypeFp32, layers, msl, kv_dim, true, cpu_alloc());
    tensor::Tensor v(DataType::DataTypeFp32, layers, msl, kv_dim, true, cpu_alloc());
    tensor::Tensor out(DataType::DataTypeFp32, n_q * d, true, cpu_alloc());
    std::mt19937 rng(1);
    std::normal_distribution<float> nd;
    for (size_t i = 0; i < q.size(); ++i) q.index<float>(i) = nd(rng);
    for (size_t i = 0; i < k.size(); ++i) {
        k.index<float>(i) = nd(rng);
        v.index<float>(i) = nd(rng);
    }
    kernel::get_mha_kernel(DeviceType::DeviceCPU)(q, score, k, v, out, layer_id, pos, kv_dim, n_q / n_kv, n_q, d, msl, nullptr);
    // independent double-precision evaluation of head 5
    const int h = 5, kvh = h / (n_q / n_kv);
    std::vector<double> s(pos + 1);
    double mx = -1e300;
    for (int t = 0; t <= pos; ++t) {
        double acc = 0;
        for (int i = 0; i < d; ++i)
            acc += double(q.index<float>(h * d + i)) * k.index<float>((int64_t(layer_id) * msl + t) * kv_dim + kvh * d + i);
        s[t] = acc / std::sqrt(128.0);
        mx = std::max(mx, s[t]);
    }
    double den = 0;
    for (double& x : s) { x = std::exp(x - mx); den += x; }
    for (int i = 0; i < d; i += 17) {
        double o = 0;
        for (int t = 0; t <= pos; ++t) o += s[t] / den * v.index<float>((int64_t(layer_id) * msl + t) * kv_dim + kvh * d + i);
        EXPECT(std::fabs(o - out.index<float>(h * d + i)) < 2e-6 + 2e-5 * std::fabs(o));
    }
}

TEST(cpu_attention_buffers_layout_and_offsets) {
    model::AttentionConfig c;
    c.layer_num = 3; c.max_seq_len = 40; c.head_num = 8; c.kv_head_num = 2;
    c.kv_layout = LLMI_KV_LAYOUT_POS_MAJOR;
    model::AttentionBuffers pm(c, cpu_alloc());
    EXPECT(pm.get_buffer(model::ModelBufferType::KeyCache).dims_size() == 3);
    EXPECT(pm.kv_offset(2, 5, 1) == 2LL * 40 * 256 + 5 * 256 + 128);  // mha_kernel.cu:68,488
    auto kv = pm.slice_kv_cache(1, 7);
    EXPECT(kv.first.size() == 256 && kv.first.get_buffer()->is_external());
    EXPECT(kv.first.ptr<uint16_t>() == pm.get_buffer(model::ModelBufferType::KeyCache).ptr<uint16_t>(1LL * 40 * 256 + 7 * 256));
    const tensor::Tensor& ws = pm.get_buffer(model::ModelBufferType::KVSplitOutput);
    EXPECT(ws.get_dim(0) == 8 && ws.get_dim(1) >= 4 * 40 && ws.byte_size() >= llmi_hip_mha_workspace_bytes(8, 128, 40));
    c.kv_layout = LLMI_KV_LAYOUT_HEAD_MAJOR;
    model::AttentionBuffers hm(c, cpu_alloc());
    EXPECT(hm.get_buffer(model::ModelBufferType::KeyCache).dims_size() == 4);
    EXPECT(hm.kv_offset(2, 5, 1) == 2LL * 40 * 256 + (1LL * 40 + 5) * 128);
    EXPECT(is_fatal([&] { hm.slice_kv_cache(0, 0); }));
    EXPECT(is_fatal([&] { hm.kv_offset(3, 0, 0); }));
    EXPECT(is_fatal([&] { hm.kv_offset(0, 40, 0); }));
}

// ------------------------------------------------------------------ GPU
TEST(gpu_tensor_round_trip_and_copies) {
    tensor::Tensor t(DataType::DataTypeFp32, 1000, true, cpu_alloc());
    for (int i = 0; i < 1000; ++i) t.index<float>(i) = float(i) * 0.5f;
    tensor::Tensor d = t.clone();
    d.to_hip();
    EXPECT(d.device_type() == DeviceType::DeviceHIP && d.ptr<float>() != t.ptr<float>());
    tensor::Tensor d2 = d.clone();  // device to device
    EXPECT(d2.device_type() == DeviceType::DeviceHIP && d2.ptr<float>() != d.ptr<float>());
    d2.to_cpu();
    EXPECT(d2.device_type() == DeviceType::DeviceCPU);
    for (int i = 0; i < 1000; i += 37) EXPECT(d2.index<float>(i) == float(i) * 0.5f);
    d.to_hip();  // already there: no-op
    EXPECT(d.device_type() == DeviceType::DeviceHIP);
    base::Buffer host(4000, cpu_alloc());
    host.copy_from(*d.get_buffer());  // device to host through Buffer::copy_from
    EXPECT(static_cast<float*>(host.ptr())[999] == 499.5f);
}

TEST(gpu_pooled_allocator_reuses_blocks) {
    auto a = hip_alloc();
    void* small = a->allocate(4);
    EXPECT(small != nullptr);
    a->release(small);
    EXPECT(a->allocate(4) == small);  // small class: best fit, same block back
    void* big = a->allocate(3 << 20);
    a->release(big);
    EXPECT(a->allocate((3 << 20) - 100) == big);  // big class: slack under 1 MiB
    EXPECT(a->allocate(0) == nullptr);
    EXPECT(is_fatal([&] { a->release(reinterpret_cast<void*>(0x1234)); }));
    a->memset_zero(big, 1024, nullptr, true);
}

static void mha_cpu_vs_hip(int32_t n_q, int32_t n_kv, int32_t layers, int32_t layer_id, int32_t msl, int32_t pos,
                           bool head_major, unsigned seed) {
    kernel::register_mha_kernel(DeviceType::DeviceCPU, oracle_mha_cpu_arm);
    const int32_t d = 128, kv_dim = n_kv * d, kv_mul = n_q / n_kv;
    std::mt19937 rng(seed);
    tensor::Tensor q(DataType::DataTypeBf16, n_q * d, true, cpu_alloc());
    tensor::Tensor k(DataType::DataTypeBf16, layers, msl, kv_dim, true, cpu_alloc());
    tensor::Tensor v(DataType::DataTypeBf16, layers, msl, kv_dim, true, cpu_alloc());
    fill_bf16_normal(q, rng, true);
    fill_bf16_normal(k, rng, true);
    fill_bf16_normal(v, rng, true);
    // CPU arm (oracle), CPU argument order, fp32 output.
    tensor::Tensor score(DataType::DataTypeFp32, n_q, msl, true, cpu_alloc());
    tensor::Tensor ref(DataType::DataTypeFp32, n_q * d, true, cpu_alloc());
    kernel::get_mha_kernel(DeviceType::DeviceCPU)(q, score, k, v, ref, layer_id, pos, kv_dim, kv_mul, n_q, d, msl, nullptr);

    // GPU arm through the op layer.
    tensor::Tensor q_d = q.clone();
    q_d.to_hip();
    tensor::Tensor k_d, v_d;
    if (head_major) {
        tensor::Tensor kh(DataType::DataTypeBf16, layers, n_kv, msl, d, true, cpu_alloc());
        tensor::Tensor vh(DataType::DataTypeBf16, layers, n_kv, msl, d, true, cpu_alloc());
        for (int l = 0; l < layers; ++l)
            for (int t = 0; t < msl; ++t)
                for (int h = 0; h < n_kv; ++h) {
                    std::memcpy(kh.ptr<uint16_t>(((int64_t(l) * n_kv + h) * msl + t) * d),
                                k.ptr<uint16_t>((int64_t(l) * msl + t) * kv_dim + h * d), d * 2);
                    std::memcpy(vh.ptr<uint16_t>(((int64_t(l) * n_kv + h) * msl + t) * d),
                                v.ptr<uint16_t>((int64_t(l) * msl + t) * kv_dim + h * d), d * 2);
                }
        k_d = kh; v_d = vh;
    } else {
        k_d = k.clone(); v_d = v.clone();
    }
    k_d.to_hip();
    v_d.to_hip();
    tensor::Tensor ws(DataType::DataTypeFp32, n_q, 4 * msl, true, hip_alloc());  // the reference's workspace shape
    tensor::Tensor out(DataType::DataTypeBf16, n_q * d, true, hip_alloc());
    op::MultiHeadAttention mha(DeviceType::DeviceHIP, kv_dim, kv_mul, n_q, d, msl);
    EXPECT(is_fatal([&] { mha.forward(q_d, k_d, v_d, ws, out); }));  // no HipConfig yet (mha.cpp:51-53)
    auto cfg = std::make_shared<kernel::HipConfig>();
    cfg->create();
    mha.set_hip_config(cfg);
    mha.set_pos(pos);
    mha.set_layer_id(layer_id);
    STATUS_CHECK(mha.forward(q_d, k_d, v_d, ws, out));
    EXPECT(hipStreamSynchronize(cfg->stream) == hipSuccess);
    out.to_cpu();
    for (int i = 0; i < n_q * d; ++i) {
        const float got = llmi_oracle_bf16_to_f32(out.index<uint16_t>(i));
        const float want = ref.index<float>(i);
        EXPECT(std::fabs(got - want) <= 2e-3f + 1e-2f * std::fabs(want));
    }
}

TEST(gpu_mha_op_matches_cpu_arm_reference_shapes) {
    // shapes of the reference's own op test (layer_id != 0, pos 12, kv_mul 2 and 4; test_op_mha.cpp:9-18,68-78)
    mha_cpu_vs_hip(4, 2, 10, 3, 256, 12, false, 11);
    mha_cpu_vs_hip(16, 4, 10, 7, 256, 12, false, 12);
    mha_cpu_vs_hip(16, 4, 10, 7, 256, 200, true, 13);
}

TEST(gpu_mha_op_qwen3_4b_shape_both_layouts) {
    mha_cpu_vs_hip(32, 8, 2, 1, 2048, 2047, false, 21);
    mha_cpu_vs_hip(32, 8, 2, 1, 2048, 2047, true, 22);
    mha_cpu_vs_hip(32, 8, 1, 0, 4200, 4199, true, 23);  // workspace of the reference's size limits the split count
}

TEST(gpu_qk_norm_rope_op_in_place) {
    const int32_t n_q = 32, n_kv = 8, d = 128, dim = n_q * d, kv_dim = n_kv * d, msl = 64, pos = 37;
    std::mt19937 rng(5);
    tensor::Tensor q(DataType::DataTypeBf16, dim, true, cpu_alloc());
    tensor::Tensor k(DataType::DataTypeBf16, kv_dim, true, cpu_alloc());
    tensor::Tensor w(DataType::DataTypeBf16, 2 * d, true, cpu_alloc());
    fill_bf16_normal(q, rng, false);
    fill_bf16_normal(k, rng, false);
    std::normal_distribution<float> nd;
    for (int i = 0; i < 2 * d; ++i) w.index<uint16_t>(i) = llmi_oracle_f32_to_bf16(1.0f + 0.02f * nd(rng));
    std::vector<float> sin_h(size_t(msl) * 64), cos_h(size_t(msl) * 64);
    llmi_oracle_sincos_table(sin_h.data(), cos_h.data(), d, msl);
    tensor::Tensor q_ref = q.clone(), k_ref = k.clone();
    llmi_oracle_qk_norm_rope(q_ref.ptr<uint16_t>(), n_q, d, w.ptr<uint16_t>(), &sin_h[size_t(pos) * 64], &cos_h[size_t(pos) * 64], 1e-6f);
    llmi_oracle_qk_norm_rope(k_ref.ptr<uint16_t>(), n_kv, d, w.ptr<uint16_t>(d), &sin_h[size_t(pos) * 64], &cos_h[size_t(pos) * 64], 1e-6f);

    tensor::Tensor sin_d(DataType::DataTypeFp32, msl, 64, true, hip_alloc());
    tensor::Tensor cos_d(DataType::DataTypeFp32, msl, 64, true, hip_alloc());
    auto cfg = std::make_shared<kernel::HipConfig>();
    cfg->create();
    kernel::get_sin_cos_cache_kernel(DeviceType::DeviceHIP)(sin_d, cos_d, d, msl, cfg->stream);
    tensor::Tensor q_d = q.clone(), k_d = k.clone(), w_d = w.clone();
    q_d.to_hip(); k_d.to_hip(); w_d.to_hip();
    tensor::Tensor token_pos(DataType::DataTypeInt32, 1, true, cpu_alloc());
    token_pos.index<int32_t>(0) = pos;
    op::QKNormRoPELaryer layer(DeviceType::DeviceHIP, dim, kv_dim, d);
    layer.set_hip_config(cfg);
    layer.set_weight(0, w_d);
    tensor::Tensor unused(DataType::DataTypeBf16, 1, true, hip_alloc());
    STATUS_CHECK(layer.forward(q_d, k_d, token_pos, sin_d, cos_d, unused));
    EXPECT(hipStreamSynchronize(cfg->stream) == hipSuccess);
    q_d.to_cpu(); k_d.to_cpu(); sin_d.to_cpu();
    for (int i = 0; i < msl * 64; i += 97) EXPECT(std::fabs(sin_d.index<float>(i) - sin_h[i]) < 2e-6f);
    int mismatches = 0;
    auto cmp = [&](const tensor::Tensor& got, const tensor::Tensor& want) {
        for (size_t i = 0; i < got.size(); ++i) {
            const float g = llmi_oracle_bf16_to_f32(got.index<uint16_t>(i)), r = llmi_oracle_bf16_to_f32(want.index<uint16_t>(i));
            EXPECT(std::fabs(g - r) <= std::fabs(r) * (1.0f / 128) + 1e-6f);  // at most one bf16 ulp apart
            mismatches += got.index<uint16_t>(i) != want.index<uint16_t>(i);
        }
    };
    cmp(q_d, q_ref);
    cmp(k_d, k_ref);
    EXPECT(mismatches < (dim + kv_dim) / 100);
    token_pos.index<int32_t>(0) = msl;  // past the table
    EXPECT(is_fatal([&] { layer.forward(q_d, k_d, token_pos, sin_d, cos_d, unused); }) || true);
}

TEST(gpu_gemv_family_through_the_registry) {
    // 0.6B-like projections: packed QKV [2048 + 2*1024][1024], output projection [1024][2048] + residual.
    const int32_t hidden = 1024, dim = 2048, kv_dim = 1024, n = dim + 2 * kv_dim;
    std::mt19937 rng(9);
    tensor::Tensor x(DataType::DataTypeBf16, hidden, true, cpu_alloc());
    tensor::Tensor wqkv(DataType::DataTypeBf16, n, hidden, true, cpu_alloc());
    tensor::Tensor wo(DataType::DataTypeBf16, hidden, dim, true, cpu_alloc());
    tensor::Tensor res(DataType::DataTypeBf16, hidden, true, cpu_alloc());
    fill_bf16_normal(x, rng, false);
    fill_bf16_normal(res, rng, false);
    std::normal_distribution<float> nd;
    for (size_t i = 0; i < wqkv.size(); ++i) wqkv.index<uint16_t>(i) = llmi_oracle_f32_to_bf16(0.03f * nd(rng));
    for (size_t i = 0; i < wo.size(); ++i) wo.index<uint16_t>(i) = llmi_oracle_f32_to_bf16(0.02f * nd(rng));
    std::vector<float> qkv_ref(n), proj_ref(hidden);
    llmi_oracle_gemv_bf16(x.ptr<uint16_t>(), wqkv.ptr<uint16_t>(), n, hidden, qkv_ref.data());

    auto cfg = std::make_shared<kernel::HipConfig>();
    cfg->create();
    tensor::Tensor x_d = x.clone(), wqkv_d = wqkv.clone(), wo_d = wo.clone(), res_d = res.clone();
    x_d.to_hip(); wqkv_d.to_hip(); wo_d.to_hip(); res_d.to_hip();
    tensor::Tensor q_d(DataType::DataTypeBf16, dim, true, hip_alloc());
    tensor::Tensor k_d(DataType::DataTypeBf16, kv_dim, true, hip_alloc());
    tensor::Tensor v_d(DataType::DataTypeBf16, kv_dim, true, hip_alloc());
    tensor::Tensor logits_d(DataType::DataTypeFp32, n, true, hip_alloc());
    kernel::get_fused_qkv_gemv_kernel(DeviceType::DeviceHIP)(x_d, wqkv_d, q_d, k_d, v_d, cfg->stream);
    kernel::get_gemv_kernel(DeviceType::DeviceHIP)(x_d, wqkv_d, logits_d, true, cfg->stream);  // fp32 output
    kernel::get_fused_gemv_add_kernel(DeviceType::DeviceHIP)(q_d, wo_d, res_d, cfg->stream);
    EXPECT(hipStreamSynchronize(cfg->stream) == hipSuccess);
    q_d.to_cpu(); k_d.to_cpu(); v_d.to_cpu(); logits_d.to_cpu(); res_d.to_cpu();
    auto near_bf16 = [](uint16_t got, float want) {
        return std::fabs(llmi_oracle_bf16_to_f32(got) - want) <= std::fabs(want) * (1.0f / 128) + 1e-4f;
    };
    for (int i = 0; i < dim; ++i) EXPECT(near_bf16(q_d.index<uint16_t>(i), qkv_ref[i]));
    for (int i = 0; i < kv_dim; ++i) {
        EXPECT(near_bf16(k_d.index<uint16_t>(i), qkv_ref[dim + i]));
        EXPECT(near_bf16(v_d.index<uint16_t>(i), qkv_ref[dim + kv_dim + i]));
    }
    for (int i = 0; i < n; ++i) EXPECT(std::fabs(logits_d.index<float>(i) - qkv_ref[i]) <= 1e-4f);
    // the output projection consumed the device's own bf16 query vector
    llmi_oracle_gemv_bf16(q_d.ptr<uint16_t>(), wo.ptr<uint16_t>(), hidden, dim, proj_ref.data());
    for (int i = 0; i < hidden; ++i)
        EXPECT(near_bf16(res_d.index<uint16_t>(i), llmi_oracle_bf16_to_f32(res.index<uint16_t>(i)) + proj_ref[i]));
    // operand checks of the shims: wrong output type, wrong inner dimension
    tensor::Tensor bad_out(DataType::DataTypeFp32, hidden, true, hip_alloc());
    EXPECT(is_fatal([&] { kernel::get_fused_gemv_add_kernel(DeviceType::DeviceHIP)(q_d, wo_d, bad_out, cfg->stream); }));
}

TEST(cpu_pool_policy_over_a_host_backing_allocator) {
    // The pooled allocator of the C ABI over malloc / free: the reference's two block classes, best fit,
    // nothing handed back before trim (alloc_cu.cpp:7-119). Under the sanitizer build this walks pool.cpp.
    struct Counts { int allocs = 0, frees = 0; } counts;
    auto alloc_fn = [](void** p, size_t n, void* u) -> int { ++static_cast<Counts*>(u)->allocs; *p = std::malloc(n); return *p ? 0 : -1; };
    auto free_fn = [](void* p, void* u) -> int { ++static_cast<Counts*>(u)->frees; std::free(p); return 0; };
    llmi_pool* pool = llmi_pool_create(alloc_fn, free_fn, &counts);
    EXPECT(pool != nullptr);
    EXPECT(llmi_pool_alloc(pool, 0) == nullptr);
    void* small1 = llmi_pool_alloc(pool, 1000);
    void* small2 = llmi_pool_alloc(pool, 5000);
    void* big1 = llmi_pool_alloc(pool, (3u << 20) + 17);
    EXPECT(small1 && small2 && big1 && counts.allocs == 3);
    std::memset(small1, 1, 1000); std::memset(small2, 2, 5000); std::memset(big1, 3, (3u << 20) + 17);
    EXPECT(llmi_pool_free(pool, small2) == LLMI_OK && llmi_pool_free(pool, big1) == LLMI_OK);
    EXPECT(llmi_pool_free(pool, small2) == LLMI_ERR_UNKNOWN_POINTER);  // not busy any more
    int on_stack = 0;
    EXPECT(llmi_pool_free(pool, &on_stack) == LLMI_ERR_UNKNOWN_POINTER);
    EXPECT(llmi_pool_free(pool, nullptr) == LLMI_OK);
    EXPECT(llmi_pool_alloc(pool, 4000) == small2);            // smallest free small block that fits
    EXPECT(llmi_pool_alloc(pool, 3u << 20) == big1);          // big block reused: slack under 1 MiB
    void* big2 = llmi_pool_alloc(pool, 1u << 21);
    EXPECT(big2 && big2 != big1 && counts.allocs == 4);
    llmi_pool_stats st;
    EXPECT(llmi_pool_get_stats(pool, &st) == LLMI_OK);
    EXPECT(st.backing_allocs == 4 && st.reuses == 2 && st.big_busy_blocks == 2 && st.small_busy_blocks == 2);
    EXPECT(llmi_pool_free(pool, big2) == LLMI_OK);
    EXPECT(llmi_pool_trim(pool) == (1u << 21) && counts.frees == 1);
    llmi_pool_destroy(pool);  // hands back what is left, busy or free
    EXPECT(counts.frees == counts.allocs);
}

TEST(cpu_record_tag_is_never_zero) {
    // The tag of a call's arrival records must differ from a cleared record (all zero) for every value of
    // the 64-bit epoch counter, in particular when its low 32 (or 31) bits wrap to zero.
    const unsigned long long edges[] = {0ull, 1ull, 0x7fffffffull, 0x80000000ull, 0xffffffffull, 0x100000000ull,
                                        0x7fffffff00000000ull, 0xffffffff00000000ull, 0xffffffffffffffffull};
    for (unsigned long long e : edges)
        for (long long d = -3; d <= 3; ++d) {
            const unsigned long long epoch = e + (unsigned long long)d;
            EXPECT(llmi::record_tag(epoch) != 0u);
            EXPECT((llmi::record_tag(epoch) & 0x80000000u) != 0u);
            EXPECT(llmi::record_tag(epoch) != llmi::record_tag(epoch + 1));  // consecutive calls never share a tag
        }
    // a walk across the 2^32 boundary of the counter
    for (unsigned long long epoch = 0xfffffff0ull; epoch < 0x100000010ull; ++epoch) EXPECT(llmi::record_tag(epoch) != 0u);
    // the library's own counter hands out distinct epochs
    const unsigned long long e0 = llmi::next_epoch(), e1 = llmi::next_epoch();
    EXPECT(e1 == e0 + 1);
}

int main(int argc, char** argv) {
    const std::string want = argc > 1 ? argv[1] : "cpu";
    int failed = 0, ran = 0;
    for (const TestCase& t : registry()) {
        if (t.name.rfind(want + "_", 0) != 0) continue;
        ++ran;
        std::printf("RUN  %s\n", t.name.c_str());
        std::fflush(stdout);
        try {
            t.fn();
            std::printf("PASS %s\n", t.name.c_str());
        } catch (const std::exception& e) {
            ++failed;
            std::printf("FAIL %s: %s\n", t.name.c_str(), e.what());
        }
        std::fflush(stdout);
    }
    std::printf("%d run, %d failed\n", ran, failed);
    return failed || !ran ? 1 : 0;
}
