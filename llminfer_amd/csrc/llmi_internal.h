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
// Byte layout of the fused combine's workspace for `num_splits` splits of `head_num` query heads.
// Plain (side == 0): partials [head][split][128] fp32 at 0, records [head][split] x 16 bytes behind them.
// By package side: both arrays start on a 16 KiB boundary (side_pad() bytes into the workspace) and every row has a
// home in each 8 KiB block of a 16 KiB pair (see WsHead in mha_decode.hip).
struct FusedWorkspace {
    size_t partial_bytes, record_bytes;  // record array right behind the partial array
    size_t bytes() const { return partial_bytes + record_bytes + 16; }
};
constexpr size_t kSideBlock = 8192;
inline FusedWorkspace fused_workspace(int head_num, int head_dim, int num_splits, bool by_side) {
    const size_t row = (size_t)head_dim * sizeof(float), rec = 2 * sizeof(unsigned long long);
    FusedWorkspace w;
    if (!by_side) {
        w.partial_bytes = ((size_t)head_num * num_splits * row + 15) & ~(size_t)15;
        w.record_bytes = (size_t)head_num * num_splits * rec;
    } else {
        const size_t rows = (size_t)head_num * num_splits;  // each with two homes
        const size_t per_pblock = row <= kSideBlock ? kSideBlock / row : 1, per_rblock = kSideBlock / rec;  // (row = 512 bytes for the kernels' head_dim)
        w.partial_bytes = 2 * ((rows + per_pblock - 1) / per_pblock) * kSideBlock;
        w.record_bytes = 2 * ((rows + per_rblock - 1) / per_rblock) * kSideBlock;
    }
    return w;
}
// Which address parity (bit 13) is nearest to XCDs 0-3, measured on the workspace with the ping-pong probe, for every
// 2 MiB-aligned region the workspace reaches into (the answer is the same within one and changes between them): two
// bits per region, counted from the region the workspace starts in (16 regions at most), 1 = clear, 2 = set,
// 0 = no statement. Synchronises the stream.
int measure_workspace_side(void* workspace, size_t bytes, hipStream_t stream, int32_t* sides);
// Bytes from a workspace's start to the by-side layout: the next 16 KiB boundary (a row's two homes are the two
// 8 KiB blocks of an aligned pair, so that both lie in one region).
inline size_t side_pad(const void* workspace) { return (size_t)(-reinterpret_cast<intptr_t>(workspace)) & (2 * kSideBlock - 1); }
// The kernel is built for the by-side layout with the wave counts the dispatcher picks itself: four wavefronts per
// workgroup, eight for (padded) groups of 8 query heads. Other wave counts keep the plain layout.
constexpr bool by_side_variant(int group_pad, int waves) { return group_pad <= 8 && waves == (group_pad == 8 ? 8 : 4); }
// Waits of the fused combine that gave up since the library was loaded (device counter of the current device).
int read_poll_timeouts(unsigned long long* count);
// Fewest splits at which the fused combine hands the heads of a KV head to different workgroups.
int spread_merge_min_splits(int group_pad);
// The mask of the staggered walk (KernelArgs::stagger) for splits whose runs are `run_bytes` long (the shorter ones,
// when they differ by a tile: `ragged`).
int stagger_mask(int kv_layout, int64_t run_bytes, bool ragged);
// ... its head-major rule, for the host and for the kernels that read the position on the device: runs of 512 KiB to
// below 2 MiB at a multiple of 512 KiB, or up to 8 tiles of 4 KiB above one (the measurements are with stagger_mask).
#if defined(__HIPCC__)
#define LLMI_HOST_DEVICE __host__ __device__
#else
#define LLMI_HOST_DEVICE
#endif
LLMI_HOST_DEVICE constexpr int head_major_stagger_rule(long long run_bytes) {
    return run_bytes >= (512 << 10) && run_bytes < (2 << 20) && run_bytes % (512 << 10) < 8 * 4096 ? 31 : 0;
}
// KernelArgs::stagger of a launch whose position is read on the device: the kernel applies the rule to the length it finds.
constexpr int kStaggerByDevice = -1;
// ... and whether such a launch can reach a length the rule applies to at all (else the kernels without the walk run).
int dyn_stagger(int kv_layout, int64_t max_run_bytes);
// Polls (each followed by a short sleep) the fused combine waits for the other splits.
int poll_limit();
// Testing aid (llmi_hip_set_test_far_home): 1 = every split but the merging one, 2 = every second split stores into
// the home of the other side of the package.
int test_far_home();

// `append` non-null: the fused QK-Norm + RoPE + K/V append variant.
// `oproj` non-null (with `append`): the attention launch also computes the output projection + residual add.
int launch_mha_decode(const llmi_mha_args& args, const llmi_mha_plan& plan, const llmi_mha_append_args* append = nullptr,
                      const llmi_attn_oproj_args* oproj = nullptr);
// The multi-layer launch (llmi_hip_mha_decode_append_stack in its one-launch form); `plan` is layer 0's.
int launch_mha_stack(const llmi_mha_stack_args& st, const llmi_mha_plan& plan);
// Bytes the multi-layer launch keeps behind the fused combine's records (its "done" tags, with room to align them).
size_t stack_workspace_extra(int head_num);
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
