// C entry points into the C++ host layer for drivers that are not C++ (the
// Python benchmark and tests, through ctypes). A harness interface: the
// drop-in boundary is include/llmi_hip.h.
#ifndef LLMI_HOST_HOOKS_H
#define LLMI_HOST_HOOKS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct llmi_host_stack llmi_host_stack;

/* Last error message of a failed hook on this thread ("" if none). Hooks return 0 / non-NULL on success. */
const char* llmi_host_last_error(void);

llmi_host_stack* llmi_host_stack_create(int32_t layer_num, int32_t max_seq_len, int32_t head_num,
                                        int32_t kv_head_num, int32_t kv_layout);
void llmi_host_stack_destroy(llmi_host_stack* s);
/* which: 0 key cache base, 1 value cache base, 2 raw query of `layer`, 3 raw key, 4 raw value,
 * 5 norm weight, 6 output of `layer`, 7 sin table, 8 cos table, 9 normalised query buffer; after
 * llmi_host_stack_enable_projections: 10 packed QKV weight of `layer`, 11 output-projection weight, 12 hidden
 * input of `layer`, 13 residual stream. Device pointers. */
void* llmi_host_stack_ptr(llmi_host_stack* s, int32_t which, int32_t layer);
/* Allocates the projections either side of the attention (mode 3: QKV GEMV, attention, o_proj + residual). */
int llmi_host_stack_enable_projections(llmi_host_stack* s, int32_t hidden_dim);
int llmi_host_stack_build_sincos(llmi_host_stack* s);
/* with_qk_norm_rope: 0 attention only, 1 separate QK-Norm/RoPE/append kernel + attention, 2 both fused,
 * 3 the whole attention block (packed QKV GEMV, fused append attention, output projection + residual) */
int llmi_host_stack_run(llmi_host_stack* s, int32_t pos, int32_t with_qk_norm_rope);      /* eager + synchronise */
int llmi_host_stack_capture(llmi_host_stack* s, int32_t pos, int32_t with_qk_norm_rope);
int llmi_host_stack_replay(llmi_host_stack* s, int32_t times, float* elapsed_ms);
/* Captures the stack for every position up to max_pos: the kernels read the position from a device word
 * (llmi_mha_args.pos_device) that llmi_host_stack_set_pos writes between replays. mode 0 or 2. */
int llmi_host_stack_capture_following(llmi_host_stack* s, int32_t max_pos, int32_t mode);
int llmi_host_stack_set_pos(llmi_host_stack* s, int32_t pos);
/* Loads the attention block's weights of every layer from an engine weight file (model::WeightFile). */
int llmi_host_stack_load_weights(llmi_host_stack* s, const char* path);
/* Opens a weight file (header_ints 8, or 7 for the older header) and reports: info[0..7] the header as stored,
 * info[8] head_dim, info[9] kv_dim, info[10] |vocab_size|, info[11] payload elements (bf16). Copies up to
 * payload_bytes of the payload to payload_out. Returns the base::Status code (0 success, 2 path, 3 parse). */
int llmi_host_weight_file_info(const char* path, int32_t header_ints, int64_t info[12], void* payload_out,
                               int64_t payload_bytes);
/* Process-wide tuning overrides of the HIP attention arm (0 = automatic). */
void llmi_host_set_mha_options(int32_t force_path, int32_t num_splits, int32_t waves_per_group);

/* Runs op::MultiHeadAttention::forward through the registry on borrowed device pointers; returns the
 * base::Status code (0 = success), -1 for a fatal error. cache_dims is 3 (position-major) or 4 (head-major). */
int llmi_host_mha_forward(void* query, void* key_cache, void* value_cache, void* workspace, int64_t workspace_floats,
                          void* output, int32_t layer_num, int32_t layer_id, int32_t pos, int32_t kv_dim,
                          int32_t kv_mul, int32_t head_num, int32_t head_dim, int32_t max_seq_len,
                          int32_t cache_dims);

#ifdef __cplusplus
}
#endif
#endif
