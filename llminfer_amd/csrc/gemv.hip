// The bf16 GEMVs that sit either side of decode attention in the layer loop, on
// gfx950: the packed QKV projection that produces the new token's raw q/k/v rows
// (role of fused_qkv_gemv_bf16x8_kernel, code/source/op/kernel/cuda/matmul_kernel.cu:211-246),
// the plain projection with bf16 or fp32 output (gemv_bf16x8_{bf16,fp32}_kernel, :38-98)
// and the output projection with the residual add folded in
// (fused_gemv_add_bf16x8_kernel, :143-172).
//
// HBM-bound weight streams: every weight byte is read once, with non-temporal
// 16-byte loads. A wavefront owns kRows consecutive rows and walks K in steps of
// 512 elements (64 lanes x 8 bf16); the input chunk a lane needs is the same for all
// of its rows and comes from L1/L2. Measured on the Qwen3-4B projections, many small
// workgroups of one row per wavefront beat fewer, fatter ones (6144 x 2560: 7.1 vs
// 7.7 us; 2560 x 4096: 5.6 vs 6.9 us): the matrices are a few microseconds of stream
// and what counts is how fast the whole chip has loads in flight. Products are formed in fp32 by v_dot2_f32_bf16
// (two bf16 pairs per instruction, fp32 accumulate), the 64 lanes fold with DPP row
// steps and four scalar reads, lane 0 rounds once and writes.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "llmi_internal.h"
#include "wave_ops.h"

namespace llmi {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

#ifndef LLMI_GEMV_ROWS
#define LLMI_GEMV_ROWS 1
#endif
#ifndef LLMI_GEMV_UNROLL
#define LLMI_GEMV_UNROLL 4
#endif
constexpr int kRows = LLMI_GEMV_ROWS;      // rows per wavefront
#ifndef LLMI_GEMV_WAVES
#define LLMI_GEMV_WAVES 2
#endif
constexpr int kWaves = LLMI_GEMV_WAVES;    // wavefronts per workgroup
constexpr int kUnroll = LLMI_GEMV_UNROLL;  // K steps whose loads are issued together

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if (x != x) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

struct GemvArgs {
    const uint16_t* x;   // [k]
    const uint16_t* w;   // [n][k]
    void* out[3];        // row segments (one for the plain GEMV, query/key/value for the packed one)
    int32_t seg_end[3];  // exclusive end row of each segment
    int32_t n;
    int32_t k8;          // k / 8
    int32_t mode;        // LLMI_GEMV_*
};

__global__ __launch_bounds__(kWaves * 64) void gemv_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int row0 = (blockIdx.x * kWaves + wave) * kRows;
    if (row0 >= a.n) return;
    const u32x4* x4 = reinterpret_cast<const u32x4*>(a.x);
    const u32x4* w4[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r)  // rows past the end re-read the last row and are not written
        w4[r] = reinterpret_cast<const u32x4*>(a.w) + (int64_t)min(row0 + r, a.n - 1) * a.k8;
    float acc[kRows] = {};
    int c = lane;
    for (; c + 64 * (kUnroll - 1) < a.k8; c += 64 * kUnroll) {
        u32x4 xv[kUnroll], wv[kUnroll][kRows];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            xv[u] = x4[c + 64 * u];
#pragma unroll
            for (int r = 0; r < kRows; ++r) wv[u][r] = __builtin_nontemporal_load(w4[r] + c + 64 * u);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
#pragma unroll
            for (int r = 0; r < kRows; ++r) acc[r] = dot8_bf16(xv[u], wv[u][r], acc[r]);
    }
    for (; c < a.k8; c += 64) {
        const u32x4 xv = x4[c];
#pragma unroll
        for (int r = 0; r < kRows; ++r) acc[r] = dot8_bf16(xv, __builtin_nontemporal_load(w4[r] + c), acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = wave_sum(acc[r]);
    if (lane < kRows) {
        float sum = acc[0];
#pragma unroll
        for (int r = 1; r < kRows; ++r) sum = lane == r ? acc[r] : sum;
        const int row = row0 + lane;
        if (row < a.n) {
            const int seg = row < a.seg_end[0] ? 0 : (row < a.seg_end[1] ? 1 : 2);
            const int local = row - (seg == 0 ? 0 : a.seg_end[seg - 1]);
            if (a.mode == LLMI_GEMV_OUT_F32) {
                static_cast<float*>(a.out[seg])[local] = sum;
            } else {
                uint16_t* o = static_cast<uint16_t*>(a.out[seg]) + local;
                if (a.mode == LLMI_GEMV_ADD_BF16) sum += bf16_to_f32(*o);  // fp32 + fp32 -> bf16 (:169-170)
                *o = f32_to_bf16(sum);
            }
        }
    }
}

}  // namespace

int launch_gemv(const void* input, const void* weight, void* const out[3], const int32_t seg_end[3], int32_t n,
                int32_t k, int32_t mode, hipStream_t stream) {
    GemvArgs a;
    a.x = static_cast<const uint16_t*>(input);
    a.w = static_cast<const uint16_t*>(weight);
    for (int i = 0; i < 3; ++i) {
        a.out[i] = out[i];
        a.seg_end[i] = seg_end[i];
    }
    a.n = n;
    a.k8 = k / 8;
    a.mode = mode;
    const int rows_per_group = kRows * kWaves;
    hipLaunchKernelGGL(gemv_kernel, dim3((n + rows_per_group - 1) / rows_per_group), dim3(kWaves * 64), 0, stream, a);
    return check_launch();
}

}  // namespace llmi
