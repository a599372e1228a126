/*
 * vt_oracle.c - CPU restatement of the voxtral-tts.c backbone / acoustic hot path.
 *
 * TEST INFRASTRUCTURE ONLY (see vt_oracle.h).  Sequential IEEE fp32, products
 * rounded before they are added (build with -ffp-contract=off, no -ffast-math),
 * summation orders exactly those of the reference CPU kernels so that results
 * are bit-identical to the compiled reference.  Citations are into the
 * reference tree (voxtral_tts_*.c).
 */
#include "vt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int  orc_get_threads(void) { return g_threads; }

/* ---- elementwise (voxtral_tts_kernels.c:25-31, 361-366) ------------------ */

void orc_add_inplace(float *a, const float *b, int n) {
    for (int i = 0; i < n; i++) a[i] = a[i] + b[i];
}

void orc_mul_inplace(float *a, const float *b, int n) {
    for (int i = 0; i < n; i++) a[i] = a[i] * b[i];
}

void orc_silu(float *x, int n) {
    for (int i = 0; i < n; i++) {
        float v = x[i];
        x[i] = v / (1.0f + expf(-v));
    }
}

/* ---- bf16 (voxtral_tts_kernels.h:159-164, voxtral_tts_kernels.c:49-59) --- */

static inline float widen(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

void orc_bf16_to_f32_buf(float *dst, const uint16_t *src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = widen(src[i]);
}

void orc_embed_token_bf16(float *out, const uint16_t *emb, int token_id, int dim) {
    orc_bf16_to_f32_buf(out, emb + (size_t)token_id * dim, (size_t)dim);
}

/* ---- linear (voxtral_tts_kernels.c:152-185 for one row of x,
 *              :187-211 + :127-138 for several) -----------------------------
 * Both reference paths start the accumulator at the bias (or 0) and add
 * w*x for k ascending; widening bf16 is exact, so one loop restates both.
 *
 * Every output element is its own sequential chain (product rounded, then added, k
 * ascending); the chains of different outputs are independent, so several of them are
 * advanced side by side - eight output rows for a single row of x, and for several rows of x
 * the rows of x as the lanes of a vector (x transposed into blocks of LANES columns) - which
 * changes no bit of any result and takes the dependent-add latency off the critical path.
 * tests/test_oracle_golden.py holds this against the compiled reference bit for bit. */
typedef float v8f __attribute__((vector_size(32)));

static void linear_one_row(float *y, const float *x, const uint16_t *W, const float *bias,
                           int in_dim, int out_dim) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (int o0 = 0; o0 < out_dim; o0 += 8) {
        const int nb = out_dim - o0 < 8 ? out_dim - o0 : 8;
        if (nb == 8) {
            const uint16_t *w = W + (size_t)o0 * in_dim;
            float a0 = bias ? bias[o0] : 0.0f, a1 = bias ? bias[o0 + 1] : 0.0f;
            float a2 = bias ? bias[o0 + 2] : 0.0f, a3 = bias ? bias[o0 + 3] : 0.0f;
            float a4 = bias ? bias[o0 + 4] : 0.0f, a5 = bias ? bias[o0 + 5] : 0.0f;
            float a6 = bias ? bias[o0 + 6] : 0.0f, a7 = bias ? bias[o0 + 7] : 0.0f;
            const size_t n = (size_t)in_dim;
            for (int k = 0; k < in_dim; k++) {
                const float xv = x[k];
                float p0 = widen(w[k]) * xv, p1 = widen(w[n + k]) * xv;
                float p2 = widen(w[2 * n + k]) * xv, p3 = widen(w[3 * n + k]) * xv;
                float p4 = widen(w[4 * n + k]) * xv, p5 = widen(w[5 * n + k]) * xv;
                float p6 = widen(w[6 * n + k]) * xv, p7 = widen(w[7 * n + k]) * xv;
                a0 = a0 + p0; a1 = a1 + p1; a2 = a2 + p2; a3 = a3 + p3;
                a4 = a4 + p4; a5 = a5 + p5; a6 = a6 + p6; a7 = a7 + p7;
            }
            y[o0] = a0; y[o0 + 1] = a1; y[o0 + 2] = a2; y[o0 + 3] = a3;
            y[o0 + 4] = a4; y[o0 + 5] = a5; y[o0 + 6] = a6; y[o0 + 7] = a7;
        } else {
            for (int o = o0; o < o0 + nb; o++) {
                const uint16_t *wr = W + (size_t)o * in_dim;
                float acc = bias ? bias[o] : 0.0f;
                for (int k = 0; k < in_dim; k++) {
                    float p = widen(wr[k]) * x[k];
                    acc = acc + p;
                }
                y[o] = acc;
            }
        }
    }
}

/* rows s0 .. s0 + ns - 1 of x (ns <= 8 * NV) against every row of W; xt is x transposed,
 * [in_dim][8 * NV] with zero padding */
#define LINEAR_BLOCK(NV)                                                                        \
static void linear_block_##NV(float *y, const v8f *xt, const uint16_t *W, const float *bias,    \
                              int s0, int ns, int in_dim, int out_dim) {                        \
    _Pragma("omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)")      \
    for (int o0 = 0; o0 < out_dim; o0 += 2) {                                                    \
        const int two = o0 + 1 < out_dim;                                                        \
        const uint16_t *w0 = W + (size_t)o0 * in_dim, *w1 = two ? w0 + in_dim : w0;             \
        const float b0 = bias ? bias[o0] : 0.0f, b1 = bias ? bias[o0 + two] : 0.0f;             \
        v8f a0[NV], a1[NV];                                                                      \
        for (int v = 0; v < NV; v++)                                                             \
            for (int l = 0; l < 8; l++) { a0[v][l] = b0; a1[v][l] = b1; }                        \
        for (int k = 0; k < in_dim; k++) {                                                       \
            const float f0 = widen(w0[k]), f1 = widen(w1[k]);                                    \
            const v8f *xk = xt + (size_t)k * NV;                                                 \
            for (int v = 0; v < NV; v++) {                                                       \
                const v8f p0 = xk[v] * f0, p1 = xk[v] * f1;                                      \
                a0[v] = a0[v] + p0;                                                              \
                a1[v] = a1[v] + p1;                                                              \
            }                                                                                    \
        }                                                                                        \
        for (int s = 0; s < ns; s++) {                                                           \
            y[(size_t)(s0 + s) * out_dim + o0] = a0[s >> 3][s & 7];                              \
            if (two) y[(size_t)(s0 + s) * out_dim + o0 + 1] = a1[s >> 3][s & 7];                 \
        }                                                                                        \
    }                                                                                            \
}
LINEAR_BLOCK(1)
LINEAR_BLOCK(4)

void orc_linear_bf16(float *y, const float *x, const uint16_t *W_bf16,
                     const float *bias, int seq_len, int in_dim, int out_dim) {
    if (seq_len == 1) {
        linear_one_row(y, x, W_bf16, bias, in_dim, out_dim);
        return;
    }
    const int nv = seq_len <= 8 ? 1 : 4, lanes = 8 * nv;
    v8f *xt = aligned_alloc(32, sizeof(v8f) * (size_t)in_dim * nv);
    if (!xt) abort();
    for (int s0 = 0; s0 < seq_len; s0 += lanes) {
        const int ns = seq_len - s0 < lanes ? seq_len - s0 : lanes;
        float *t = (float *)xt;
        for (int k = 0; k < in_dim; k++)
            for (int l = 0; l < lanes; l++)
                t[(size_t)k * lanes + l] = l < ns ? x[(size_t)(s0 + l) * in_dim + k] : 0.0f;
        if (nv == 1) linear_block_1(y, xt, W_bf16, bias, s0, ns, in_dim, out_dim);
        else linear_block_4(y, xt, W_bf16, bias, s0, ns, in_dim, out_dim);
    }
    free(xt);
}

/* ---- RMSNorm (voxtral_tts_kernels.c:333-349) ------------------------------ */

void orc_rms_norm(float *out, const float *x, const float *weight,
                  int seq_len, int hidden, float eps) {
    for (int s = 0; s < seq_len; s++) {
        const float *xr = x + (size_t)s * hidden;
        float *or_ = out + (size_t)s * hidden;
        float ss = 0.0f;
        for (int i = 0; i < hidden; i++) {
            float sq = xr[i] * xr[i];
            ss = ss + sq;
        }
        float inv = 1.0f / sqrtf(ss / hidden + eps);
        for (int i = 0; i < hidden; i++) {
            float t = xr[i] * inv;
            or_[i] = t * weight[i];
        }
    }
}

/* ---- RoPE (voxtral_tts_kernels.c:602-634) --------------------------------- */

void orc_compute_rope_freqs(float *freqs, const int *pos, int seq, int dim, float theta) {
    int half = dim / 2;
    for (int s = 0; s < seq; s++) {
        float p = (float)pos[s];
        float *row = freqs + (size_t)s * half * 2;
        for (int d = 0; d < half; d++) {
            float f = 1.0f / powf(theta, (float)(2 * d) / (float)dim);
            float ang = p * f;
            row[2 * d] = cosf(ang);
            row[2 * d + 1] = sinf(ang);
        }
    }
}

void orc_apply_rope(float *x, const float *freqs, int seq, int heads, int head_dim) {
    int half = head_dim / 2;
    size_t hidden = (size_t)heads * head_dim;
    for (int s = 0; s < seq; s++) {
        const float *cs = freqs + (size_t)s * half * 2;
        for (int h = 0; h < heads; h++) {
            float *v = x + s * hidden + (size_t)h * head_dim;
            for (int d = 0; d < half; d++) {
                float c = cs[2 * d], sn = cs[2 * d + 1];
                float a = v[2 * d], b = v[2 * d + 1];
                float ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
                v[2 * d] = ac - bs;
                v[2 * d + 1] = as + bc;
            }
        }
    }
}

/* ---- attention (voxtral_tts_kernels.c:403-465 causal, :467-525 bidirectional)
 * Online softmax in key order: a strictly larger score rescales the running
 * sum and output by expf(old_max - score) and adds the value row with weight 1;
 * otherwise the value row is added with weight expf(score - max). */
static void attend_row(float *o, const float *q, const float *K, const float *V,
                       int j0, int j1, int kv_hidden, int kv_off, int head_dim,
                       float scale) {
    float mx = -1e30f;
    float se = 0.0f;
    for (int d = 0; d < head_dim; d++) o[d] = 0.0f;
    for (int j = j0; j < j1; j++) {
        const float *kr = K + (size_t)j * kv_hidden + kv_off;
        const float *vr = V + (size_t)j * kv_hidden + kv_off;
        float sc = 0.0f;
        for (int d = 0; d < head_dim; d++) {
            float p = q[d] * kr[d];
            sc = sc + p;
        }
        sc = sc * scale;
        if (sc > mx) {
            float corr = expf(mx - sc);
            se = se * corr + 1.0f;
            for (int d = 0; d < head_dim; d++) {
                float t = o[d] * corr;
                o[d] = t + vr[d];
            }
            mx = sc;
        } else {
            float w = expf(sc - mx);
            se = se + w;
            for (int d = 0; d < head_dim; d++) {
                float t = w * vr[d];
                o[d] = o[d] + t;
            }
        }
    }
    if (se > 0.0f) {
        float inv = 1.0f / se;
        for (int d = 0; d < head_dim; d++) o[d] = o[d] * inv;
    }
}

void orc_causal_attention(float *out, const float *Q, const float *K, const float *V,
                          int seq_q, int seq_k, int n_heads, int n_kv_heads,
                          int head_dim, float scale, int window_size, int q_offset) {
    int group = n_heads / n_kv_heads;
    int q_hidden = n_heads * head_dim;
    int kv_hidden = n_kv_heads * head_dim;
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
    for (int h = 0; h < n_heads; h++) {
        int kv_off = (h / group) * head_dim;
        for (int i = 0; i < seq_q; i++) {
            int gp = q_offset + i;
            int j0 = 0;
            if (window_size > 0 && gp - window_size + 1 > 0) j0 = gp - window_size + 1;
            int j1 = gp + 1;
            if (j1 > seq_k) j1 = seq_k;
            attend_row(out + (size_t)i * q_hidden + (size_t)h * head_dim,
                       Q + (size_t)i * q_hidden + (size_t)h * head_dim,
                       K, V, j0, j1, kv_hidden, kv_off, head_dim, scale);
        }
    }
}

void orc_bidirectional_attention(float *out, const float *Q, const float *K, const float *V,
                                 int seq_len, int n_heads, int n_kv_heads,
                                 int head_dim, float scale) {
    int group = n_heads / n_kv_heads;
    int q_hidden = n_heads * head_dim;
    int kv_hidden = n_kv_heads * head_dim;
    for (int h = 0; h < n_heads; h++) {
        int kv_off = (h / group) * head_dim;
        for (int i = 0; i < seq_len; i++) {
            attend_row(out + (size_t)i * q_hidden + (size_t)h * head_dim,
                       Q + (size_t)i * q_hidden + (size_t)h * head_dim,
                       K, V, 0, seq_len, kv_hidden, kv_off, head_dim, scale);
        }
    }
}

/* ---- RNG (voxtral_tts_kernels.c:640-669) ---------------------------------- */

void orc_rng_seed(uint64_t *state, uint64_t seed) {
    *state = seed ? seed : 0x12345678ABCDEF01ULL;
}

static uint64_t next_u64(uint64_t *state) {
    uint64_t s = *state;
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    *state = s;
    return s;
}

static float next_unit(uint64_t *state) {
    return (float)(next_u64(state) >> 11) * (1.0f / 9007199254740992.0f);
}

float orc_randn(uint64_t *state) {
    float u1;
    do { u1 = next_unit(state); } while (u1 < 1e-30f);
    float u2 = next_unit(state);
    float r = sqrtf(-2.0f * logf(u1));
    return r * cosf(6.2831853071795864f * u2);
}

void orc_randn_fill(uint64_t *state, float *buf, int n) {
    for (int i = 0; i < n; i++) buf[i] = orc_randn(state);
}

/* ---- backbone decode step (voxtral_tts_llm.c:171-271; cache rows :105-113) */

static float *kv_row(float *cache, int layer, int kv_max, int pos) {
    return cache + ((size_t)layer * kv_max + pos) * ORC_KV_DIM;
}

void orc_llm_forward(const orc_layer_t *layers, int n_layers, const float *final_norm,
                     float *kv_k, float *kv_v, int kv_max, int pos,
                     const float *input_embed, float *out_hidden) {
    float *x = malloc(sizeof(float) * ORC_DIM);
    float *xn = malloc(sizeof(float) * ORC_DIM);
    float *q = malloc(sizeof(float) * ORC_Q_DIM);
    float *k = malloc(sizeof(float) * ORC_KV_DIM);
    float *v = malloc(sizeof(float) * ORC_KV_DIM);
    float *att = malloc(sizeof(float) * ORC_Q_DIM);
    float *proj = malloc(sizeof(float) * ORC_DIM);
    float *gate = malloc(sizeof(float) * ORC_FFN);
    float *up = malloc(sizeof(float) * ORC_FFN);
    float rope[ORC_HEAD_DIM];
    float scale = 1.0f / sqrtf((float)ORC_HEAD_DIM);

    orc_compute_rope_freqs(rope, &pos, 1, ORC_HEAD_DIM, ORC_ROPE_THETA);
    memcpy(x, input_embed, sizeof(float) * ORC_DIM);

    for (int l = 0; l < n_layers; l++) {
        const orc_layer_t *w = &layers[l];
        orc_rms_norm(xn, x, w->attention_norm, 1, ORC_DIM, ORC_EPS);
        orc_linear_bf16(q, xn, w->wq, NULL, 1, ORC_DIM, ORC_Q_DIM);
        orc_linear_bf16(k, xn, w->wk, NULL, 1, ORC_DIM, ORC_KV_DIM);
        orc_linear_bf16(v, xn, w->wv, NULL, 1, ORC_DIM, ORC_KV_DIM);
        orc_apply_rope(q, rope, 1, ORC_HEADS, ORC_HEAD_DIM);
        orc_apply_rope(k, rope, 1, ORC_KV_HEADS, ORC_HEAD_DIM);
        memcpy(kv_row(kv_k, l, kv_max, pos), k, sizeof(float) * ORC_KV_DIM);
        memcpy(kv_row(kv_v, l, kv_max, pos), v, sizeof(float) * ORC_KV_DIM);
        orc_causal_attention(att, q, kv_row(kv_k, l, kv_max, 0), kv_row(kv_v, l, kv_max, 0),
                             1, pos + 1, ORC_HEADS, ORC_KV_HEADS, ORC_HEAD_DIM,
                             scale, 0, pos);
        orc_linear_bf16(proj, att, w->wo, NULL, 1, ORC_Q_DIM, ORC_DIM);
        orc_add_inplace(x, proj, ORC_DIM);

        orc_rms_norm(xn, x, w->ffn_norm, 1, ORC_DIM, ORC_EPS);
        orc_linear_bf16(gate, xn, w->w1, NULL, 1, ORC_DIM, ORC_FFN);
        orc_linear_bf16(up, xn, w->w3, NULL, 1, ORC_DIM, ORC_FFN);
        orc_silu(gate, ORC_FFN);
        orc_mul_inplace(gate, up, ORC_FFN);
        orc_linear_bf16(proj, gate, w->w2, NULL, 1, ORC_FFN, ORC_DIM);
        orc_add_inplace(x, proj, ORC_DIM);
    }
    orc_rms_norm(out_hidden, x, final_norm, 1, ORC_DIM, ORC_EPS);

    free(x); free(xn); free(q); free(k); free(v); free(att); free(proj);
    free(gate); free(up);
}

/* ---- backbone prefill (voxtral_tts_llm.c:277-373) ------------------------- */

void orc_llm_prefill(const orc_layer_t *layers, int n_layers,
                     float *kv_k, float *kv_v, int kv_max, int start_pos,
                     const float *embeds, int seq_len, float *out_x) {
    size_t S = (size_t)seq_len;
    float *x = malloc(sizeof(float) * S * ORC_DIM);
    float *xn = malloc(sizeof(float) * S * ORC_DIM);
    float *q = malloc(sizeof(float) * S * ORC_Q_DIM);
    float *k = malloc(sizeof(float) * S * ORC_KV_DIM);
    float *v = malloc(sizeof(float) * S * ORC_KV_DIM);
    float *att = malloc(sizeof(float) * S * ORC_Q_DIM);
    float *proj = malloc(sizeof(float) * S * ORC_DIM);
    float *gate = malloc(sizeof(float) * S * ORC_FFN);
    float *up = malloc(sizeof(float) * S * ORC_FFN);
    int *posv = malloc(sizeof(int) * S);
    float *rope = malloc(sizeof(float) * S * ORC_HEAD_DIM);
    float scale = 1.0f / sqrtf((float)ORC_HEAD_DIM);

    for (int i = 0; i < seq_len; i++) posv[i] = start_pos + i;
    orc_compute_rope_freqs(rope, posv, seq_len, ORC_HEAD_DIM, ORC_ROPE_THETA);
    memcpy(x, embeds, sizeof(float) * S * ORC_DIM);

    for (int l = 0; l < n_layers; l++) {
        const orc_layer_t *w = &layers[l];
        orc_rms_norm(xn, x, w->attention_norm, seq_len, ORC_DIM, ORC_EPS);
        orc_linear_bf16(q, xn, w->wq, NULL, seq_len, ORC_DIM, ORC_Q_DIM);
        orc_linear_bf16(k, xn, w->wk, NULL, seq_len, ORC_DIM, ORC_KV_DIM);
        orc_linear_bf16(v, xn, w->wv, NULL, seq_len, ORC_DIM, ORC_KV_DIM);
        orc_apply_rope(q, rope, seq_len, ORC_HEADS, ORC_HEAD_DIM);
        orc_apply_rope(k, rope, seq_len, ORC_KV_HEADS, ORC_HEAD_DIM);
        memcpy(kv_row(kv_k, l, kv_max, start_pos), k, sizeof(float) * S * ORC_KV_DIM);
        memcpy(kv_row(kv_v, l, kv_max, start_pos), v, sizeof(float) * S * ORC_KV_DIM);
        orc_causal_attention(att, q, kv_row(kv_k, l, kv_max, 0), kv_row(kv_v, l, kv_max, 0),
                             seq_len, start_pos + seq_len, ORC_HEADS, ORC_KV_HEADS,
                             ORC_HEAD_DIM, scale, 0, start_pos);
        orc_linear_bf16(proj, att, w->wo, NULL, seq_len, ORC_Q_DIM, ORC_DIM);
        orc_add_inplace(x, proj, seq_len * ORC_DIM);

        orc_rms_norm(xn, x, w->ffn_norm, seq_len, ORC_DIM, ORC_EPS);
        orc_linear_bf16(gate, xn, w->w1, NULL, seq_len, ORC_DIM, ORC_FFN);
        orc_linear_bf16(up, xn, w->w3, NULL, seq_len, ORC_DIM, ORC_FFN);
        orc_silu(gate, seq_len * ORC_FFN);
        orc_mul_inplace(gate, up, seq_len * ORC_FFN);
        orc_linear_bf16(proj, gate, w->w2, NULL, seq_len, ORC_FFN, ORC_DIM);
        orc_add_inplace(x, proj, seq_len * ORC_DIM);
    }
    if (out_x) memcpy(out_x, x, sizeof(float) * S * ORC_DIM);

    free(x); free(xn); free(q); free(k); free(v); free(att); free(proj);
    free(gate); free(up); free(posv); free(rope);
}

/* ---- acoustic transformer -------------------------------------------------- */

/* voxtral_tts_acoustic.c:166-176 */
void orc_time_embedding(const float *inv_freq, float t_val, float *out, int dim) {
    int half = dim / 2;
    for (int i = 0; i < half; i++) {
        float ang = t_val * inv_freq[i];
        out[i] = cosf(ang);
        out[half + i] = sinf(ang);
    }
}

/* voxtral_tts_acoustic.c:48-60 (used when the checkpoint carries no table) */
void orc_default_time_inv_freq(float *inv_freq, int half_dim) {
    float theta = 10000.0f;
    for (int i = 0; i < half_dim; i++)
        inv_freq[i] = expf(-logf(theta) * (float)i / (float)half_dim);
}

/* voxtral_tts_acoustic.c:182-262 (CPU branch) */
void orc_predict_velocity(const orc_acoustic_t *ac, const float *x_t,
                          const float *llm_hidden, float t_val, float *out_velocity) {
    enum { SEQ = 3 };
    float *tok = malloc(sizeof(float) * SEQ * ORC_DIM);
    float *tn = malloc(sizeof(float) * SEQ * ORC_DIM);
    float *q = malloc(sizeof(float) * SEQ * ORC_Q_DIM);
    float *k = malloc(sizeof(float) * SEQ * ORC_KV_DIM);
    float *v = malloc(sizeof(float) * SEQ * ORC_KV_DIM);
    float *att = malloc(sizeof(float) * SEQ * ORC_Q_DIM);
    float *proj = malloc(sizeof(float) * SEQ * ORC_DIM);
    float *gate = malloc(sizeof(float) * SEQ * ORC_FFN);
    float *up = malloc(sizeof(float) * SEQ * ORC_FFN);
    float *temb = malloc(sizeof(float) * ORC_DIM);
    float scale = 1.0f / sqrtf((float)ORC_HEAD_DIM);

    orc_linear_bf16(tok, x_t, ac->input_proj, NULL, 1, ORC_ACOUSTIC_DIM, ORC_DIM);
    orc_time_embedding(ac->time_inv_freq, t_val, temb, ORC_DIM);
    orc_linear_bf16(tok + ORC_DIM, temb, ac->time_proj, NULL, 1, ORC_DIM, ORC_DIM);
    orc_linear_bf16(tok + 2 * ORC_DIM, llm_hidden, ac->llm_proj, NULL, 1, ORC_DIM, ORC_DIM);

    for (int l = 0; l < ac->n_layers; l++) {
        const orc_layer_t *w = &ac->layers[l];
        orc_rms_norm(tn, tok, w->attention_norm, SEQ, ORC_DIM, ORC_EPS);
        orc_linear_bf16(q, tn, w->wq, NULL, SEQ, ORC_DIM, ORC_Q_DIM);
        orc_linear_bf16(k, tn, w->wk, NULL, SEQ, ORC_DIM, ORC_KV_DIM);
        orc_linear_bf16(v, tn, w->wv, NULL, SEQ, ORC_DIM, ORC_KV_DIM);
        orc_bidirectional_attention(att, q, k, v, SEQ, ORC_HEADS, ORC_KV_HEADS,
                                    ORC_HEAD_DIM, scale);
        orc_linear_bf16(proj, att, w->wo, NULL, SEQ, ORC_Q_DIM, ORC_DIM);
        orc_add_inplace(tok, proj, SEQ * ORC_DIM);

        orc_rms_norm(tn, tok, w->ffn_norm, SEQ, ORC_DIM, ORC_EPS);
        orc_linear_bf16(gate, tn, w->w1, NULL, SEQ, ORC_DIM, ORC_FFN);
        orc_linear_bf16(up, tn, w->w3, NULL, SEQ, ORC_DIM, ORC_FFN);
        orc_silu(gate, SEQ * ORC_FFN);
        orc_mul_inplace(gate, up, SEQ * ORC_FFN);
        orc_linear_bf16(proj, gate, w->w2, NULL, SEQ, ORC_FFN, ORC_DIM);
        orc_add_inplace(tok, proj, SEQ * ORC_DIM);
    }
    orc_rms_norm(tn, tok, ac->norm, 1, ORC_DIM, ORC_EPS);
    orc_linear_bf16(out_velocity, tn, ac->acoustic_out, NULL, 1, ORC_DIM, ORC_ACOUSTIC_DIM);

    free(tok); free(tn); free(q); free(k); free(v); free(att); free(proj);
    free(gate); free(up); free(temb);
}

/* voxtral_tts_acoustic.c:268-373 */
void orc_acoustic_forward(const orc_acoustic_t *ac, const float *llm_hidden,
                          uint64_t *rng_state, int *out_codes, float *out_x) {
    float *logits = malloc(sizeof(float) * ORC_SEM_PADDED);
    orc_linear_bf16(logits, llm_hidden, ac->semantic_out, ac->semantic_out_bias,
                    1, ORC_DIM, ORC_SEM_PADDED);
    logits[0] = -1e30f;
    for (int i = 2 + ORC_SEM_SIZE; i < ORC_SEM_PADDED; i++) logits[i] = -1e30f;
    int best_i = 0;
    float best = logits[0];
    for (int i = 1; i < ORC_SEM_PADDED; i++) {
        if (logits[i] > best) { best = logits[i]; best_i = i; }
    }
    free(logits);
    out_codes[0] = best_i;

    if (best_i == 1) {                       /* END_AUDIO: no flow matching, no RNG draw */
        for (int i = 1; i < ORC_CODES_PER_FRAME; i++) out_codes[i] = 2;
        if (out_x) memset(out_x, 0, sizeof(float) * ORC_ACOUSTIC_DIM);
        return;
    }

    float x[ORC_ACOUSTIC_DIM], vc[ORC_ACOUSTIC_DIM], vu[ORC_ACOUSTIC_DIM];
    float *zero = calloc(ORC_DIM, sizeof(float));
    orc_randn_fill(rng_state, x, ORC_ACOUSTIC_DIM);
    for (int i = 0; i < ORC_ACOUSTIC_DIM; i++) x[i] = x[i] * 1.0f;

    float ts[ORC_FLOW_STEPS];
    for (int i = 0; i < ORC_FLOW_STEPS; i++) ts[i] = (float)i / (float)(ORC_FLOW_STEPS - 1);

    for (int s = 0; s < ORC_FLOW_STEPS - 1; s++) {
        float t = ts[s];
        float dt = ts[s + 1] - ts[s];
        orc_predict_velocity(ac, x, llm_hidden, t, vc);
        orc_predict_velocity(ac, x, zero, t, vu);
        for (int i = 0; i < ORC_ACOUSTIC_DIM; i++) {
            float a = ORC_CFG_ALPHA * vc[i];
            float b = (1.0f - ORC_CFG_ALPHA) * vu[i];
            float vv = a + b;
            float step = vv * dt;
            x[i] = x[i] + step;
        }
    }
    free(zero);
    if (out_x) memcpy(out_x, x, sizeof x);

    for (int i = 0; i < ORC_ACOUSTIC_DIM; i++) {
        float val = x[i];
        if (val > 1.0f) val = 1.0f;
        if (val < -1.0f) val = -1.0f;
        float scaled = ((val + 1.0f) / 2.0f) * (float)(ORC_FSQ_LEVELS - 1);
        int code = (int)(scaled + 0.5f);
        if (code < 0) code = 0;
        if (code >= ORC_FSQ_LEVELS) code = ORC_FSQ_LEVELS - 1;
        out_codes[i + 1] = code + 2;
    }
}

/* voxtral_tts_voice.c:292-315 */
void orc_audio_embed_forward(const uint16_t *emb_bf16, const int *offsets,
                             const int *codes, float *out_embed, int dim) {
    for (int i = 0; i < dim; i++) out_embed[i] = 0.0f;
    for (int cb = 0; cb < ORC_CODES_PER_FRAME; cb++) {
        const uint16_t *row = emb_bf16 + (size_t)(offsets[cb] + codes[cb]) * dim;
        for (int i = 0; i < dim; i++) out_embed[i] = out_embed[i] + widen(row[i]);
    }
}
