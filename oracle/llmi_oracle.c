/*
 * CPU oracle for decode-phase grouped-query attention: TEST INFRASTRUCTURE
 * ONLY (see llmi_oracle.h). Plain C, fp32, left-to-right sums, no threads:
 * the reference's CPU path is single-threaded
 * (code/source/op/kernel/cpu/mha_kernel.cpp:40).
 */
#include "llmi_oracle.h"

#include <math.h>
#include <string.h>

/* test_kernel/bench_qwen3_gemv_bf16_cublaslt.cu:52-58 */
uint16_t llmi_oracle_f32_to_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, sizeof(u));
    uint32_t lsb = (u >> 16) & 1u;
    uint32_t rounding_bias = 0x7FFFu + lsb;
    return (uint16_t)((u + rounding_bias) >> 16);
}

/* test_kernel/bench_qwen3_gemv_bf16_cublaslt.cu:60-65 */
float llmi_oracle_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float x;
    memcpy(&x, &u, sizeof(x));
    return x;
}

void llmi_oracle_f32_to_bf16_n(const float* x, uint16_t* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = llmi_oracle_f32_to_bf16(x[i]);
}

void llmi_oracle_bf16_to_f32_n(const uint16_t* x, float* y, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = llmi_oracle_bf16_to_f32(x[i]);
}

/* code/source/op/kernel/cpu/matmul_kernel.cpp:51: out = (in * wei) * scale */
float llmi_oracle_dot_scaled(const float* q, const float* k, int32_t d, float scale) {
    float acc = 0.0f;
    for (int32_t i = 0; i < d; ++i) acc += q[i] * k[i];
    return acc * scale;
}

/* code/source/op/kernel/cpu/softmax_kernel.cpp:13-19 */
void llmi_oracle_softmax_inplace(float* x, int32_t n) {
    float max_val = x[0];
    for (int32_t i = 1; i < n; ++i)
        if (x[i] > max_val) max_val = x[i];
    float sum_exp = 0.0f;
    for (int32_t i = 0; i < n; ++i) {
        x[i] = expf(x[i] - max_val);
        sum_exp += x[i];
    }
    for (int32_t i = 0; i < n; ++i) x[i] /= sum_exp;
}

/* code/source/op/kernel/cpu/scale_sum_kernel.cpp:29-35 */
void llmi_oracle_scale_sum(const float* score, const float* value, float* out, int32_t pos,
                           int32_t head_dim, int32_t kv_dim) {
    for (int32_t t = 0; t <= pos; ++t) {
        const float* val = value + (size_t)t * (size_t)kv_dim;
        const float s = score[t];
        for (int32_t i = 0; i < head_dim; ++i) out[i] += s * val[i];
    }
}

static int mha_args_ok(int32_t layer_id, int32_t pos, int32_t kv_dim, int32_t kv_mul,
                       int32_t head_num, int32_t head_dim, int32_t max_seq_len) {
    return layer_id >= 0 && pos >= 0 && pos < max_seq_len && kv_dim > 0 && kv_mul > 0 &&
           head_num > 0 && head_dim > 0;
}

/* code/source/op/kernel/cpu/mha_kernel.cpp:34-110 */
int llmi_oracle_mha_cpu(const float* query, float* score, const float* key_cache,
                        const float* value_cache, float* output, int32_t layer_id, int32_t pos,
                        int32_t kv_dim, int32_t kv_mul, int32_t head_num, int32_t head_dim,
                        int32_t max_seq_len) {
    if (!query || !score || !key_cache || !value_cache || !output) return -1;
    if (!mha_args_ok(layer_id, pos, kv_dim, kv_mul, head_num, head_dim, max_seq_len)) return -1;

    /* :34 (the reference computes this in int32; widened here so that large
     * caches do not overflow -- same value wherever the reference is defined) */
    const size_t layer_offset = (size_t)layer_id * (size_t)max_seq_len * (size_t)kv_dim;
    /* :37 */
    const float scale = 1.0f / sqrtf((float)head_dim);

    for (int32_t h = 0; h < head_num; ++h) {                      /* :40 */
        float* score_head = score + (size_t)h * (size_t)max_seq_len;  /* :43 */
        const float* query_head = query + (size_t)h * (size_t)head_dim; /* :46 */
        for (int32_t t = 0; t <= pos; ++t) {                      /* :53 */
            const size_t key_off = layer_offset + (size_t)t * (size_t)kv_dim +
                                   (size_t)(h / kv_mul) * (size_t)head_dim; /* :59 */
            /* :75 restored: score[t] = (q . k_t) * scale */
            score_head[t] = llmi_oracle_dot_scaled(query_head, key_cache + key_off, head_dim, scale);
        }
        llmi_oracle_softmax_inplace(score_head, pos + 1);         /* :79-84 */
        float* out_head = output + (size_t)h * (size_t)head_dim;  /* :87 */
        memset(out_head, 0, (size_t)head_dim * sizeof(float));    /* :90 */
        const size_t value_off = layer_offset + (size_t)(h / kv_mul) * (size_t)head_dim; /* :101 */
        llmi_oracle_scale_sum(score_head, value_cache + value_off, out_head, pos, head_dim,
                              kv_dim);                            /* :109 */
    }
    return 0;
}

int llmi_oracle_mha_cpu_bf16(const uint16_t* query, float* score, const uint16_t* key_cache,
                             const uint16_t* value_cache, float* output, int32_t layer_id,
                             int32_t pos, int32_t kv_dim, int32_t kv_mul, int32_t head_num,
                             int32_t head_dim, int32_t max_seq_len) {
    if (!query || !score || !key_cache || !value_cache || !output) return -1;
    if (!mha_args_ok(layer_id, pos, kv_dim, kv_mul, head_num, head_dim, max_seq_len)) return -1;
    if (head_dim > 1024) return -1;

    const size_t layer_offset = (size_t)layer_id * (size_t)max_seq_len * (size_t)kv_dim;
    const float scale = 1.0f / sqrtf((float)head_dim);
    float qf[1024];

    for (int32_t h = 0; h < head_num; ++h) {
        float* score_head = score + (size_t)h * (size_t)max_seq_len;
        for (int32_t i = 0; i < head_dim; ++i)
            qf[i] = llmi_oracle_bf16_to_f32(query[(size_t)h * (size_t)head_dim + i]);
        const size_t head_off = layer_offset + (size_t)(h / kv_mul) * (size_t)head_dim;
        for (int32_t t = 0; t <= pos; ++t) {
            const uint16_t* k = key_cache + head_off + (size_t)t * (size_t)kv_dim;
            float acc = 0.0f;
            for (int32_t i = 0; i < head_dim; ++i) acc += qf[i] * llmi_oracle_bf16_to_f32(k[i]);
            score_head[t] = acc * scale;
        }
        llmi_oracle_softmax_inplace(score_head, pos + 1);
        float* out_head = output + (size_t)h * (size_t)head_dim;
        memset(out_head, 0, (size_t)head_dim * sizeof(float));
        for (int32_t t = 0; t <= pos; ++t) {
            const uint16_t* v = value_cache + head_off + (size_t)t * (size_t)kv_dim;
            const float s = score_head[t];
            for (int32_t i = 0; i < head_dim; ++i) out_head[i] += s * llmi_oracle_bf16_to_f32(v[i]);
        }
    }
    return 0;
}

/* Definition of the per-split quantities of
 * code/source/op/kernel/cuda/mha_kernel.cu:243-386. */
void llmi_oracle_split_partial(const float* q_head, const float* key_base,
                               const float* value_base, int32_t begin, int32_t end,
                               int32_t head_dim, int32_t kv_dim, float scale, float* o, float* m,
                               float* l) {
    float mx = -INFINITY;
    for (int32_t t = begin; t < end; ++t) {
        float s = llmi_oracle_dot_scaled(q_head, key_base + (size_t)t * (size_t)kv_dim, head_dim, scale);
        if (s > mx) mx = s;
    }
    float sum = 0.0f;
    for (int32_t i = 0; i < head_dim; ++i) o[i] = 0.0f;
    for (int32_t t = begin; t < end; ++t) {
        float s = llmi_oracle_dot_scaled(q_head, key_base + (size_t)t * (size_t)kv_dim, head_dim, scale);
        float p = expf(s - mx);
        sum += p;
        const float* v = value_base + (size_t)t * (size_t)kv_dim;
        for (int32_t i = 0; i < head_dim; ++i) o[i] += p * v[i];
    }
    *m = mx;
    *l = sum;
}

/* code/source/op/kernel/cuda/mha_kernel.cu:421-437 */
void llmi_oracle_combine(const float* o, const float* m, const float* l, int32_t num_splits,
                         int32_t head_dim, float* out) {
    float mx = -INFINITY;
    for (int32_t s = 0; s < num_splits; ++s)
        if (m[s] > mx) mx = m[s];
    float sum = 0.0f;
    for (int32_t s = 0; s < num_splits; ++s)
        if (l[s] > 0.0f) sum += l[s] * expf(m[s] - mx);
    for (int32_t i = 0; i < head_dim; ++i) {
        float acc = 0.0f;
        for (int32_t s = 0; s < num_splits; ++s)
            if (l[s] > 0.0f) acc += o[(size_t)s * (size_t)head_dim + i] * expf(m[s] - mx);
        out[i] = acc / sum;
    }
}

/* code/source/op/kernel/cpu/rope_kernel.cpp:7-22 */
void llmi_oracle_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim,
                              int32_t max_seq_len) {
    const int32_t half = head_dim / 2;
    const float inv_head_dim = 1.0f / (float)head_dim;      /* :9 */
    const float ln_base = logf(1000000.0f);                  /* :10 */
    for (int32_t pos = 0; pos < max_seq_len; ++pos) {
        for (int32_t i = 0; i < half; ++i) {
            /* :12 -- the product is formed in double, stored as float */
            const float freq = (float)exp(-2.0 * i * inv_head_dim * ln_base);
            const float theta = (float)pos * freq;             /* :19 */
            sin_cache[(size_t)pos * half + i] = sinf(theta);   /* :20 */
            cos_cache[(size_t)pos * half + i] = cosf(theta);
        }
    }
}

/* code/source/op/kernel/cuda/rmsnorm_kernel.cu:221-244 */
void llmi_oracle_qk_norm_rope(uint16_t* x, int32_t n_heads, int32_t head_dim,
                              const uint16_t* weight, const float* sin_row,
                              const float* cos_row, float eps) {
    const int32_t half = head_dim / 2;
    for (int32_t h = 0; h < n_heads; ++h) {
        uint16_t* xh = x + (size_t)h * (size_t)head_dim;
        float ss = 0.0f;
        for (int32_t i = 0; i < head_dim; ++i) {
            const float v = llmi_oracle_bf16_to_f32(xh[i]);
            ss += v * v;                                        /* :221-223 */
        }
        /* :227 with cpu/rmsnorm_kernel.cpp:43-46 (1/sqrtf of mean + eps) */
        const float r = 1.0f / sqrtf(ss / (float)head_dim + eps);
        for (int32_t i = 0; i < half; ++i) {
            const float a = llmi_oracle_bf16_to_f32(xh[i]) * llmi_oracle_bf16_to_f32(weight[i]) * r;             /* :237 */
            const float b = llmi_oracle_bf16_to_f32(xh[i + half]) * llmi_oracle_bf16_to_f32(weight[i + half]) * r; /* :238 */
            const float a1 = a * cos_row[i] - b * sin_row[i];  /* :240 */
            const float b1 = a * sin_row[i] + b * cos_row[i];  /* :241 */
            xh[i] = llmi_oracle_f32_to_bf16(a1);               /* :243 */
            xh[i + half] = llmi_oracle_f32_to_bf16(b1);        /* :244 */
        }
    }
}

/* code/source/op/kernel/cuda/matmul_kernel.cu:6-63 */
void llmi_oracle_gemv_bf16(const uint16_t* x, const uint16_t* w, int32_t n, int32_t k,
                           float* out) {
    enum { kThreads = 256, kWarp = 32, kWarps = kThreads / kWarp };
    const int32_t k8 = k / 8;                                   /* :46 */
    for (int32_t r = 0; r < n; ++r) {
        const uint16_t* wr = w + (size_t)r * (size_t)k;        /* :48 */
        float part[kThreads];
        for (int32_t t = 0; t < kThreads; ++t) {
            float sum = 0.0f;                                   /* :50 */
            for (int32_t i = t; i < k8; i += kThreads) {        /* :51 */
                for (int32_t j = 0; j < 8; ++j) {               /* :57-60, pairs (x, y) in order */
                    sum = fmaf(llmi_oracle_bf16_to_f32(x[i * 8 + j]), llmi_oracle_bf16_to_f32(wr[i * 8 + j]), sum);
                }
            }
            part[t] = sum;
        }
        float warp_sum[kWarps];
        for (int32_t wv = 0; wv < kWarps; ++wv) {               /* warp_reduce_sum<32>, :6-13 */
            float* v = part + wv * kWarp;
            for (int32_t delta = kWarp / 2; delta > 0; delta /= 2)
                for (int32_t lane = 0; lane < delta; ++lane) v[lane] += v[lane + delta];
            warp_sum[wv] = v[0];                                /* :21-23 */
        }
        for (int32_t delta = kWarps / 2; delta > 0; delta /= 2)  /* warp_reduce_sum<WARP_NUM>, :26-30 */
            for (int32_t lane = 0; lane < delta; ++lane) warp_sum[lane] += warp_sum[lane + delta];
        out[r] = warp_sum[0];
    }
}
