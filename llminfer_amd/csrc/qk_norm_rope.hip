// The per-token writers that feed decode attention on gfx950:
//   * fused per-head RMSNorm * weight + half-rotation RoPE on the query (in
//     place) and on the new K row, which lands in its cache slot in either
//     layout together with the new V row
//     (role of fused_qk_norm_rope_kernel, code/source/op/kernel/cuda/rmsnorm_kernel.cu:205-290,
//     plus the slot addressing of Model::slice_kv_cache, code/source/model/model.cpp:90-107);
//   * the sin/cos table (role of sin_cos_cache_kernel, code/source/op/kernel/cuda/rope_kernel.cu:6-21);
//   * a position-major -> head-major cache copy.
// One wavefront per head: lane i owns the rotation pair (i, i+64), the sum of
// squares is folded across the 64 lanes with DPP row steps and scalar reads, no LDS.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmi_internal.h"
#include "wave_ops.h"

namespace llmi {
namespace {

constexpr int kHeadDim = 128;
constexpr int kHalf = 64;

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if (x != x) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

struct AppendArgs {
    uint16_t* query;
    const uint16_t* query_src;
    const uint16_t* key_new;
    const uint16_t* value_new;
    uint16_t* key_slot;    // cache address of (layer, pos, kv_head 0)
    uint16_t* value_slot;
    const uint16_t* weight;
    const float* sin_row;
    const float* cos_row;
    int64_t slot_head_stride;  // elements between KV heads inside the slot
    int32_t head_num;
    int32_t n_kv;
    float eps;
};

__global__ __launch_bounds__(kHalf) void qk_norm_rope_append_kernel(AppendArgs a) {
    const int b = blockIdx.x;
    const int i = threadIdx.x;
    if (b >= a.head_num + a.n_kv) {
        // V row: plain copy into the slot, 4 bytes per lane.
        const int kh = b - a.head_num - a.n_kv;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(a.value_new + kh * kHeadDim);
        uint32_t* dst = reinterpret_cast<uint32_t*>(a.value_slot + kh * a.slot_head_stride);
        dst[i] = src[i];
        return;
    }
    const uint16_t* src;
    uint16_t* dst;
    const uint16_t* w;
    if (b < a.head_num) {
        src = a.query_src + b * kHeadDim;
        dst = a.query + b * kHeadDim;
        w = a.weight;
    } else {
        const int kh = b - a.head_num;
        src = a.key_new + kh * kHeadDim;
        dst = a.key_slot + kh * a.slot_head_stride;
        w = a.weight + kHeadDim;
    }
    const float x0 = bf16_to_f32(src[i]);
    const float x1 = bf16_to_f32(src[i + kHalf]);
    float ss = x0 * x0 + x1 * x1;
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)kHeadDim + a.eps);
    const float av = x0 * bf16_to_f32(w[i]) * r;
    const float bv = x1 * bf16_to_f32(w[i + kHalf]) * r;
    const float sn = a.sin_row[i];
    const float cs = a.cos_row[i];
    dst[i] = f32_to_bf16(av * cs - bv * sn);
    dst[i + kHalf] = f32_to_bf16(av * sn + bv * cs);
}

__global__ void sincos_table_kernel(float* __restrict__ sin_cache, float* __restrict__ cos_cache, int32_t half,
                                    int64_t total, float inv_head_dim, float ln_base) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int32_t i = (int32_t)(idx % half);
    const int32_t pos = (int32_t)(idx / half);
    // Same expression as the reference's host table (cpu/rope_kernel.cpp:12):
    // the exponent is formed in double and the frequency stored as float.
    const float freq = (float)exp(-2.0 * i * (double)inv_head_dim * (double)ln_base);
    const float theta = (float)pos * freq;
    float s, c;
    sincosf(theta, &s, &c);
    sin_cache[idx] = s;
    cos_cache[idx] = c;
}

__global__ void kv_restride_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int32_t max_seq_len,
                                   int32_t n_kv, int32_t num_pos, int64_t total) {
    // One 16-byte chunk (8 bf16) per thread; 16 chunks per 128-wide head row.
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int c = (int)(idx & 15);
    int64_t r = idx >> 4;
    const int kh = (int)(r % n_kv);
    r /= n_kv;
    const int t = (int)(r % num_pos);
    const int64_t layer = r / num_pos;
    const int64_t layer_chunks = (int64_t)max_seq_len * n_kv * 16;
    const int64_t s = layer * layer_chunks + ((int64_t)t * n_kv + kh) * 16 + c;
    const int64_t d = layer * layer_chunks + ((int64_t)kh * max_seq_len + t) * 16 + c;
    dst[d] = src[s];
}

}  // namespace

int launch_qk_norm_rope_append(const llmi_qk_norm_rope_args& args) {
    const int n_kv = args.kv_dim / args.head_dim;
    const int64_t layer_off = (int64_t)args.layer_id * args.max_seq_len * args.kv_dim;
    int64_t slot_off, slot_head_stride;
    if (args.kv_layout == LLMI_KV_LAYOUT_POS_MAJOR) {
        slot_off = layer_off + (int64_t)args.pos * args.kv_dim;
        slot_head_stride = args.head_dim;
    } else {
        slot_off = layer_off + (int64_t)args.pos * args.head_dim;
        slot_head_stride = (int64_t)args.max_seq_len * args.head_dim;
    }
    AppendArgs a;
    a.query = static_cast<uint16_t*>(args.query);
    a.query_src = args.query_src ? static_cast<const uint16_t*>(args.query_src) : a.query;
    a.key_new = static_cast<const uint16_t*>(args.key_new);
    a.value_new = static_cast<const uint16_t*>(args.value_new);
    a.key_slot = static_cast<uint16_t*>(args.key_cache) + slot_off;
    a.value_slot = args.value_cache ? static_cast<uint16_t*>(args.value_cache) + slot_off : nullptr;
    a.weight = static_cast<const uint16_t*>(args.norm_weight);
    a.sin_row = args.sin_cache + (int64_t)args.pos * (args.head_dim / 2);
    a.cos_row = args.cos_cache + (int64_t)args.pos * (args.head_dim / 2);
    a.slot_head_stride = slot_head_stride;
    a.head_num = args.head_num;
    a.n_kv = n_kv;
    a.eps = args.eps;
    const int blocks = args.head_num + n_kv + (args.value_new ? n_kv : 0);
    hipLaunchKernelGGL(qk_norm_rope_append_kernel, dim3(blocks), dim3(kHalf), 0,
                       static_cast<hipStream_t>(args.stream), a);
    return check_launch();
}

int launch_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim, int32_t max_seq_len,
                        hipStream_t stream) {
    const int32_t half = head_dim / 2;
    const int64_t total = (int64_t)half * max_seq_len;
    const int threads = 256;
    const int64_t blocks = (total + threads - 1) / threads;
    hipLaunchKernelGGL(sincos_table_kernel, dim3((unsigned)blocks), dim3(threads), 0, stream, sin_cache, cos_cache,
                       half, total, 1.0f / (float)head_dim, logf(1000000.0f));
    return check_launch();
}

int launch_kv_restride(const void* src, void* dst, int32_t layer_num, int32_t max_seq_len, int32_t kv_dim,
                       int32_t head_dim, int32_t num_pos, hipStream_t stream) {
    const int n_kv = kv_dim / head_dim;
    const int64_t total = (int64_t)layer_num * num_pos * n_kv * 16;
    if (total == 0) return LLMI_OK;
    const int threads = 256;
    const int64_t blocks = (total + threads - 1) / threads;
    hipLaunchKernelGGL(kv_restride_kernel, dim3((unsigned)blocks), dim3(threads), 0, stream,
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), max_seq_len, n_kv, num_pos, total);
    return check_launch();
}

}  // namespace llmi
