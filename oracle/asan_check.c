/* Runs every function of the CPU oracle once on exact-size heap buffers, for a
 * build with -fsanitize=address,undefined (`make -C oracle asan`): an access one
 * element past any argument, or undefined arithmetic, ends the program with a
 * report. TEST INFRASTRUCTURE, like the oracle itself. It checks memory safety
 * only; the numbers are checked by tests/test_oracle.py. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "llmi_oracle.h"

static float* f32(size_t n, unsigned seed) {
    float* p = (float*)malloc(n * sizeof(float) + (n == 0));
    for (size_t i = 0; i < n; ++i) {
        seed = seed * 1664525u + 1013904223u;
        p[i] = (float)((int)(seed >> 8) % 2001 - 1000) / 500.0f;
    }
    return p;
}
static uint16_t* bf16(size_t n, unsigned seed) {
    float* x = f32(n, seed);
    uint16_t* p = (uint16_t*)malloc(n * sizeof(uint16_t) + (n == 0));
    llmi_oracle_f32_to_bf16_n(x, p, n);
    free(x);
    return p;
}

static int mha_case(int head_num, int kv_mul, int head_dim, int max_seq_len, int layers, int layer_id, int pos) {
    const int kv_dim = head_num / kv_mul * head_dim;
    const size_t cache = (size_t)layers * max_seq_len * kv_dim;
    float *q = f32((size_t)head_num * head_dim, 1), *k = f32(cache, 2), *v = f32(cache, 3);
    float* score = f32((size_t)head_num * max_seq_len, 4);
    float* out = f32((size_t)head_num * head_dim, 5);
    int rc = llmi_oracle_mha_cpu(q, score, k, v, out, layer_id, pos, kv_dim, kv_mul, head_num, head_dim, max_seq_len);
    uint16_t *qb = bf16((size_t)head_num * head_dim, 1), *kb = bf16(cache, 2), *vb = bf16(cache, 3);
    rc |= llmi_oracle_mha_cpu_bf16(qb, score, kb, vb, out, layer_id, pos, kv_dim, kv_mul, head_num, head_dim, max_seq_len);
    for (int i = 0; i < head_num * head_dim; ++i)
        if (!isfinite(out[i])) rc |= 2;
    free(q); free(k); free(v); free(score); free(out); free(qb); free(kb); free(vb);
    return rc;
}

int main(void) {
    int bad = 0;
    /* last layer, last position: the highest addresses the op touches */
    bad |= mha_case(16, 2, 128, 257, 1, 0, 256);
    bad |= mha_case(32, 4, 128, 64, 3, 2, 63);
    bad |= mha_case(8, 8, 128, 5, 2, 1, 0);
    bad |= mha_case(4, 1, 64, 33, 1, 0, 32);

    {
        float* x = f32(7, 6);
        llmi_oracle_softmax_inplace(x, 7);
        llmi_oracle_softmax_inplace(x, 1);
        float *qv = f32(128, 7), *kv = f32(128, 8);
        if (!isfinite(llmi_oracle_dot_scaled(qv, kv, 128, 0.088f))) bad |= 4;
        free(x); free(qv); free(kv);
    }
    {
        const int pos = 9, head_dim = 128, kv_dim = 256;
        float* score = f32(pos + 1, 9);
        float* value = f32((size_t)pos * kv_dim + head_dim, 10); /* exactly up to the last row's head */
        float* out = f32(head_dim, 11);
        llmi_oracle_scale_sum(score, value, out, pos, head_dim, kv_dim);
        free(score); free(value); free(out);
    }
    {
        const int head_dim = 128, kv_dim = 256, begin = 3, end = 11, S = 4;
        float* q = f32(head_dim, 12);
        float* kbuf = f32((size_t)(end - 1) * kv_dim + head_dim, 13);
        float* vbuf = f32((size_t)(end - 1) * kv_dim + head_dim, 14);
        float *o = f32((size_t)S * head_dim, 15), *m = f32(S, 16), *l = f32(S, 17), *out = f32(head_dim, 18);
        for (int s = 0; s < S; ++s)
            llmi_oracle_split_partial(q, kbuf, vbuf, begin + 2 * s, s == 3 ? begin + 2 * s : begin + 2 * s + 2, head_dim,
                                      kv_dim, 0.088f, o + (size_t)s * head_dim, m + s, l + s);
        llmi_oracle_combine(o, m, l, S, head_dim, out);
        free(q); free(kbuf); free(vbuf); free(o); free(m); free(l); free(out);
    }
    {
        const int head_dim = 128, msl = 37, heads = 5;
        float *sn = f32((size_t)msl * head_dim / 2, 19), *cs = f32((size_t)msl * head_dim / 2, 20);
        llmi_oracle_sincos_table(sn, cs, head_dim, msl);
        uint16_t *x = bf16((size_t)heads * head_dim, 21), *w = bf16(head_dim, 22);
        llmi_oracle_qk_norm_rope(x, heads, head_dim, w, sn + (size_t)(msl - 1) * head_dim / 2, cs + (size_t)(msl - 1) * head_dim / 2, 1e-6f);
        free(sn); free(cs); free(x); free(w);
    }
    {
        const int n = 19, k = 2056; /* k a multiple of 8, not of 256 * 8 */
        uint16_t *x = bf16(k, 23), *w = bf16((size_t)n * k, 24);
        float* out = f32(n, 25);
        llmi_oracle_gemv_bf16(x, w, n, k, out);
        free(x); free(w); free(out);
    }
    {
        float x[3] = {1.0f, -0.0f, 3.14159f};
        uint16_t y[3];
        float z[3];
        llmi_oracle_f32_to_bf16_n(x, y, 3);
        llmi_oracle_bf16_to_f32_n(y, z, 3);
        if (llmi_oracle_bf16_to_f32(llmi_oracle_f32_to_bf16(NAN)) == 0.0f) bad |= 8;
    }
    printf("oracle asan check: %s\n", bad ? "FAILED" : "ok");
    return bad;
}
