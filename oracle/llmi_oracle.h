/*
 * CPU oracle for decode-phase grouped-query attention.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's
 * CPU attention path, used as the checker in tests, in the smoke check and as
 * the timed CPU baseline of the benchmark. Nothing in the product path may
 * link, load or call it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout). Arithmetic is fp32, summed left to right; the
 * reference delegates its sums to Armadillo (arma::sum, arma::mean, matrix
 * product), whose internal summation order is not specified, so agreement with
 * a build of the reference is to a few fp32 ulp, not bit-exact. No test of the
 * reference pins that boundary: "parity unpinned" at the Armadillo call sites
 * (softmax_kernel.cpp:15-19, scale_sum_kernel.cpp:26-34,
 * matmul_kernel.cpp:48-51, rmsnorm_kernel.cpp:28-51). The functions are pinned
 * instead by closed forms, invariants and long-double brute force.
 */
#ifndef LLMI_ORACLE_H
#define LLMI_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* bf16 <-> fp32, round to nearest even.
 * test_kernel/bench_qwen3_gemv_bf16_cublaslt.cu:52-64 */
uint16_t llmi_oracle_f32_to_bf16(float x);
float llmi_oracle_bf16_to_f32(uint16_t h);
void llmi_oracle_f32_to_bf16_n(const float* x, uint16_t* y, size_t n);
void llmi_oracle_bf16_to_f32_n(const uint16_t* x, float* y, size_t n);

/* (sum_i q[i]*k[i]) * scale, scale applied after the sum.
 * code/source/op/kernel/cpu/matmul_kernel.cpp:48-51 for a 1xd . dx1 product,
 * the call the commented line code/source/op/kernel/cpu/mha_kernel.cpp:75
 * intends. */
float llmi_oracle_dot_scaled(const float* q, const float* k, int32_t d, float scale);

/* x <- exp(x - max x) / sum.  code/source/op/kernel/cpu/softmax_kernel.cpp:11-19 */
void llmi_oracle_softmax_inplace(float* x, int32_t n);

/* out += score[t] * value[t*kv_dim .. +head_dim], t = 0..pos ascending.
 * code/source/op/kernel/cpu/scale_sum_kernel.cpp:29-35 */
void llmi_oracle_scale_sum(const float* score, const float* value, float* out,
                           int32_t pos, int32_t head_dim, int32_t kv_dim);

/* The CPU attention op, argument order of the CPU kernel
 * (query, score, key_cache, value_cache, output, ...).
 * code/source/op/kernel/cpu/mha_kernel.cpp:6-111 with line 75 restored.
 * Caches are position-major [layer][max_seq_len][kv_dim]; score is
 * [head_num][max_seq_len] scratch that holds the softmax weights on return.
 * Returns 0, or -1 on an argument the reference would CHECK-fail on. */
int llmi_oracle_mha_cpu(const float* query, float* score, const float* key_cache,
                        const float* value_cache, float* output, int32_t layer_id,
                        int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num,
                        int32_t head_dim, int32_t max_seq_len);

/* Same algorithm reading bf16 query/caches (widened exactly to fp32 on load),
 * fp32 output: what "the CPU path on the same bf16-rounded inputs" means
 * without materialising fp32 copies of a large cache. */
int llmi_oracle_mha_cpu_bf16(const uint16_t* query, float* score, const uint16_t* key_cache,
                             const uint16_t* value_cache, float* output, int32_t layer_id,
                             int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num,
                             int32_t head_dim, int32_t max_seq_len);

/* One split of the KV-split path for one query head over positions
 * [begin, end): m = max score, l = sum exp(score-m), o[d] = sum exp(score-m)*v.
 * The quantities code/source/op/kernel/cuda/mha_kernel.cu:243-386 leaves in
 * its workspace (un-normalised o, m, l), computed directly from their
 * definition. An empty range gives m=-inf, l=0, o=0. */
void llmi_oracle_split_partial(const float* q_head, const float* key_base,
                               const float* value_base, int32_t begin, int32_t end,
                               int32_t head_dim, int32_t kv_dim, float scale, float* o,
                               float* m, float* l);

/* Log-sum-exp merge of S partials into out[d] = sum_s o_s[d] e^(m_s-M) / sum_s l_s e^(m_s-M).
 * code/source/op/kernel/cuda/mha_kernel.cu:421-437.  o is [S][head_dim]. */
void llmi_oracle_combine(const float* o, const float* m, const float* l, int32_t num_splits,
                         int32_t head_dim, float* out);

/* sin/cos table [max_seq_len][head_dim/2], theta 1e6.
 * code/source/op/kernel/cpu/rope_kernel.cpp:5-23 */
void llmi_oracle_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim,
                              int32_t max_seq_len);

/* Fused per-head RMSNorm(eps)*w then half-rotation RoPE on bf16 data, fp32
 * chain with a single final rounding, in place on x ([n_heads][head_dim]).
 * Order of operations of code/source/op/kernel/cuda/rmsnorm_kernel.cu:221-244
 * (mirrored by test_kernel/test_qwen3_bf16_ops.py:777-794); norm from
 * code/source/op/kernel/cpu/rmsnorm_kernel.cpp:43-51 with eps passed in,
 * rotation from code/source/op/kernel/cpu/rope_kernel.cpp:45-57.
 * weight is [head_dim] bf16, sin_row/cos_row are [head_dim/2] fp32. */
void llmi_oracle_qk_norm_rope(uint16_t* x, int32_t n_heads, int32_t head_dim,
                              const uint16_t* weight, const float* sin_row,
                              const float* cos_row, float eps);

/* bf16 GEMV of the layer's projections: out[r] = sum_k x[k] * w[r][k], fp32
 * accumulate, in the order of the reference's 256-thread block
 * (code/source/op/kernel/cuda/matmul_kernel.cu:38-63 with the block reduction
 * :6-36): thread t adds the 8-element chunks t, t+256, ... left to right (the
 * compiler's fused multiply-add), the 32 lanes of a warp fold by halving,
 * then the 8 warp sums do. Result in fp32 (the lm_head variant, :65-98);
 * llmi_oracle_f32_to_bf16 of it is the bf16 variant (:62), and
 * f32_to_bf16(bf16_to_f32(residual[r]) + out[r]) the fused residual add
 * (:143-172). The packed QKV GEMV (:211-246) is this routine on the weight
 * [dim + 2*kv_dim][k] with the rows dealt to query, key and value.
 * k must be a multiple of 8. */
void llmi_oracle_gemv_bf16(const uint16_t* x, const uint16_t* w, int32_t n, int32_t k,
                           float* out);

#ifdef __cplusplus
}
#endif
#endif
