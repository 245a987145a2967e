// Folds over the 64 lanes of a gfx950 wavefront without trips through the LDS crossbar
// (role of the reference's warp_reduce_sum / warp_reduce_max shuffles,
// code/source/op/kernel/cuda/mha_kernel.cu:6-13,390-397): four DPP steps inside the 16-lane
// rows, then the four row results are read into scalar registers.
#ifndef LLMI_WAVE_OPS_H
#define LLMI_WAVE_OPS_H

#include <hip/hip_runtime.h>

namespace llmi {

// x of the lane's DPP partner: quad_perm [1,0,3,2] (0xB1), [2,3,0,1] (0x4E), row_half_mirror (0x141),
// row_mirror (0x140). Applied in this order with a commutative fold they leave the fold of all 16
// lanes of a row in every lane, at VALU speed.
template <int CTRL>
__device__ __forceinline__ float dpp_partner(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_lane0(float x, int row) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 16 * row));
}
// Folds over all 64 lanes, the result in every lane.
__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_partner<0xB1>(x));
    x = fmaxf(x, dpp_partner<0x4E>(x));
    x = fmaxf(x, dpp_partner<0x141>(x));
    x = fmaxf(x, dpp_partner<0x140>(x));
    return fmaxf(fmaxf(row_lane0(x, 0), row_lane0(x, 1)), fmaxf(row_lane0(x, 2), row_lane0(x, 3)));
}
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_partner<0xB1>(x);
    x += dpp_partner<0x4E>(x);
    x += dpp_partner<0x141>(x);
    x += dpp_partner<0x140>(x);
    return (row_lane0(x, 0) + row_lane0(x, 1)) + (row_lane0(x, 2) + row_lane0(x, 3));
}

// acc + the dot product of eight bf16 pairs (two 16-byte operands), fp32 accumulate, left to right.
typedef uint32_t wave_ops_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float dot8_bf16(wave_ops_u32x4 a, wave_ops_u32x4 b, float acc) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t ai = a[i], bi = b[i];  // (bit_cast straight from a vector element reads element 0)
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, ai), __builtin_bit_cast(bf16x2, bi), acc, false);
    }
    return acc;
}

}  // namespace llmi

#endif
