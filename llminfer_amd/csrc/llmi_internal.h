// Internal declarations shared by the translation units of libllmi_hip.so.
#ifndef LLMI_INTERNAL_H
#define LLMI_INTERNAL_H

#include <hip/hip_runtime.h>

#include "llmi_hip.h"

namespace llmi {

constexpr int kMaxSplits = 256;     // upper bound on the KV split count
constexpr int kMaxGroup = 16;       // query heads per KV head the kernels accept
constexpr int kMaxGroupWaves = 64;  // group_pad * waves_per_group that fits the LDS merge
constexpr int kMaxWaves = 8;        // wavefronts per workgroup the kernels are instantiated for

// Records a failed HIP call for llmi_hip_last_error() and maps it to LLMI_ERR_LAUNCH.
int record_hip_error(hipError_t err, const char* what);
// hipGetLastError() after a kernel launch.
int check_launch();

// A fresh number per decode call, for the arrival records of the fused combine.
unsigned long long next_epoch();
// The 32-bit tag a call's records carry, from its epoch: bit 31 is always set, so that a tag never
// equals a cleared record (all zero) whatever the epoch counter reads -- also when its low bits wrap
// to zero; the low 31 bits are the epoch's.
constexpr uint32_t record_tag(unsigned long long epoch) { return 0x80000000u | (uint32_t)(epoch & 0x7fffffffull); }
// The workspace llmi_hip_mha_decode_static uses instead of a caller's: a fixed array in device memory that
// belongs to the library's code object (one copy per GPU). static_scratch() returns its address on the
// current device and its size; it allocates nothing.
#define LLMI_STATIC_SCRATCH_BYTES (4u << 20)
int static_scratch(void** ptr, size_t* bytes);
// Waits of the fused combine that gave up since the library was loaded (device counter of the current device).
int read_poll_timeouts(unsigned long long* count);
// Polls (each followed by a short sleep) the fused combine waits for the other splits.
int poll_limit();

// `append` non-null: the fused QK-Norm + RoPE + K/V append variant.
// `oproj` non-null (with `append`): the attention launch also computes the output projection + residual add.
int launch_mha_decode(const llmi_mha_args& args, const llmi_mha_plan& plan, const llmi_mha_append_args* append = nullptr,
                      const llmi_attn_oproj_args* oproj = nullptr);
// What the fused projection holds per wavefront: weight rows, and the widest attention output (elements).
int oproj_limits(int32_t* rows_per_wave, int32_t* max_k);
int launch_qk_norm_rope_append(const llmi_qk_norm_rope_args& args);
int launch_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim, int32_t max_seq_len,
                        hipStream_t stream);
int launch_gemv(const void* input, const void* weight, void* const out[3], const int32_t seg_end[3], int32_t n,
                int32_t k, int32_t mode, hipStream_t stream);
int launch_kv_restride(const void* src, void* dst, int32_t layer_num, int32_t max_seq_len,
                       int32_t kv_dim, int32_t head_dim, int32_t num_pos, hipStream_t stream);

}  // namespace llmi

#endif
