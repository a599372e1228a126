/*
 * vt_oracle_codec.c - CPU restatement of the audio codec decoder (codes -> waveform).
 *
 * TEST INFRASTRUCTURE ONLY: the checker the HIP codec path is compared against.  Nothing in
 * the product library links, loads or calls it.
 *
 * Plain sequential IEEE fp32, no FMA contraction; each function cites the reference lines it
 * follows.  Loops over independent outputs run on orc_get_threads() workers; every single sum
 * keeps the reference's order, so results do not depend on the worker count.
 *
 * Pin status: every function here is compared bit for bit with the compiled reference sources
 * (oracle/_ref) in tests/golden/make_golden.py and tests/test_oracle_codec.py, frozen in
 * tests/golden/codec.npz; closed-form cases (delta-tap convolutions, a window of one, geometric
 * ALiBi weights) and a float64 numpy model of the whole decoder are in tests/test_oracle_codec.py.
 */
#include "vt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define NT orc_get_threads()

/* ---- weight norm (voxtral_tts_codec.c:38-57) ------------------------------------------- */
void orc_weight_norm(float *weight, const float *weight_v, const float *weight_g, int out_ch, int fan_in) {
    for (int o = 0; o < out_ch; o++) {
        const float *v = weight_v + (size_t)o * fan_in;
        float nsq = 0.0f;
        for (int i = 0; i < fan_in; i++) {
            float sq = v[i] * v[i];
            nsq = nsq + sq;
        }
        float scale = weight_g[o] / sqrtf(nsq + 1e-12f);
        for (int i = 0; i < fan_in; i++) weight[(size_t)o * fan_in + i] = v[i] * scale;
    }
}

/* ---- semantic codebook (voxtral_tts_codec.c:196-205) and ALiBi slopes (:209-210) -------- */
void orc_codec_semantic_embedding(float *emb, const float *emb_sum, const float *cluster_usage) {
    for (int i = 0; i < ORC_SEM_SIZE; i++) {
        float usage = cluster_usage[i] < 1e-5f ? 1e-5f : cluster_usage[i];
        for (int j = 0; j < ORC_CODEC_SEM_DIM; j++)
            emb[i * ORC_CODEC_SEM_DIM + j] = emb_sum[i * ORC_CODEC_SEM_DIM + j] / usage;
    }
}

void orc_codec_alibi_slopes(float *slopes) {
    for (int h = 0; h < ORC_CODEC_HEADS; h++)
        slopes[h] = powf(2.0f, -8.0f / (float)ORC_CODEC_HEADS * (float)(h + 1));
}

/* ---- f32 linear without bias (voxtral_tts_kernels.c:127-145, no-BLAS loop) -------------- */
void orc_linear_f32(float *y, const float *x, const float *W, int seq_len, int in_dim, int out_dim) {
#pragma omp parallel for collapse(2) schedule(static) num_threads(NT) if (NT > 1)
    for (int s = 0; s < seq_len; s++)
        for (int o = 0; o < out_dim; o++) {
            const float *xr = x + (size_t)s * in_dim, *wr = W + (size_t)o * in_dim;
            float acc = 0.0f;
            for (int k = 0; k < in_dim; k++) {
                float p = xr[k] * wr[k];
                acc = acc + p;
            }
            y[(size_t)s * out_dim + o] = acc;
        }
}

/* ---- causal conv1d, channel-first (voxtral_tts_kernels.c:217-272) ----------------------- */
int orc_causal_conv1d(float *out, const float *in, const float *weight, const float *bias,
                      int ch_in, int ch_out, int length, int kernel, int stride) {
    int pad = kernel - stride;
    float nf = ((float)(length - kernel + pad)) / (float)stride + 1.0f;
    int out_len = (int)ceilf(nf);
    if (out_len <= 0) return 0;
#pragma omp parallel for collapse(2) schedule(static) num_threads(NT) if (NT > 1)
    for (int oc = 0; oc < ch_out; oc++)
        for (int ol = 0; ol < out_len; ol++) {
            float sum = bias ? bias[oc] : 0.0f;
            for (int ic = 0; ic < ch_in; ic++)
                for (int k = 0; k < kernel; k++) {
                    int il = ol * stride + k - pad;
                    float val = 0.0f;
                    if (il >= 0 && il < length) {
                        val = in[(size_t)ic * length + il];
                    } else if (il < 0) {            /* reflected on the left */
                        if (-il < length) val = in[(size_t)ic * length - il];
                    } else {                        /* reflected on the right */
                        int r = 2 * length - 2 - il;
                        if (r >= 0 && r < length) val = in[(size_t)ic * length + r];
                    }
                    float p = val * weight[((size_t)oc * ch_in + ic) * kernel + k];
                    sum = sum + p;
                }
            out[(size_t)oc * out_len + ol] = sum;
        }
    return out_len;
}

/* ---- causal transposed conv1d, channel-first, weight [ch_in, ch_out, kernel]
 *      (voxtral_tts_kernels.c:274-327).  The reference scatters over (ic, il) into a zeroed
 *      buffer; an output element therefore receives its terms for ic ascending and, within
 *      one ic, for il ascending, which the gather below keeps. ------------------------------ */
int orc_causal_conv_transpose_1d(float *out, const float *in, const float *weight, const float *bias,
                                 int ch_in, int ch_out, int length, int kernel, int stride) {
    int raw_len = (length - 1) * stride + kernel;
    int total = kernel - stride;
    int right = (int)ceilf((float)total * 1.0f);
    int left = total - right;
    int final_len = raw_len - left - right;
    if (final_len <= 0) return 0;
#pragma omp parallel for collapse(2) schedule(static) num_threads(NT) if (NT > 1)
    for (int oc = 0; oc < ch_out; oc++)
        for (int ol = 0; ol < final_len; ol++) {
            int pos = ol + left;                     /* index into the untrimmed output */
            float acc = 0.0f;
            for (int ic = 0; ic < ch_in; ic++)
                for (int il = 0; il < length; il++) {
                    int k = pos - il * stride;
                    if (k < 0 || k >= kernel) continue;
                    float p = in[(size_t)ic * length + il] * weight[((size_t)ic * ch_out + oc) * kernel + k];
                    acc = acc + p;
                }
            out[(size_t)oc * final_len + ol] = acc + (bias ? bias[oc] : 0.0f);
        }
    return final_len;
}

/* ---- ALiBi causal sliding-window attention (voxtral_tts_kernels.c:527-596) -------------- */
void orc_alibi_attention(float *out, const float *Q, const float *K, const float *V, int seq_len,
                         int n_heads, int n_kv_heads, int head_dim, float scale, int window,
                         const float *slopes) {
    int per_kv = n_heads / n_kv_heads, qh = n_heads * head_dim, kvh = n_kv_heads * head_dim;
#pragma omp parallel for collapse(2) schedule(static) num_threads(NT) if (NT > 1)
    for (int h = 0; h < n_heads; h++)
        for (int i = 0; i < seq_len; i++) {
            int kv_h = h / per_kv;
            float slope = slopes[h];
            const float *q = Q + (size_t)i * qh + h * head_dim;
            float *o = out + (size_t)i * qh + h * head_dim;
            int j0 = (window > 0 && i - window + 1 > 0) ? i - window + 1 : 0;
            float mx = -1e30f, se = 0.0f;
            for (int d = 0; d < head_dim; d++) o[d] = 0.0f;
            for (int j = j0; j <= i; j++) {
                const float *k = K + (size_t)j * kvh + kv_h * head_dim;
                const float *v = V + (size_t)j * kvh + kv_h * head_dim;
                float sc = 0.0f;
                for (int d = 0; d < head_dim; d++) {
                    float p = q[d] * k[d];
                    sc = sc + p;
                }
                sc = sc * scale;
                float b = slope * (float)(j - i);
                sc = sc + b;
                if (sc > mx) {
                    float c = expf(mx - sc);
                    se = se * c + 1.0f;
                    for (int d = 0; d < head_dim; d++) {
                        float t = o[d] * c;
                        o[d] = t + v[d];
                    }
                    mx = sc;
                } else {
                    float w = expf(sc - mx);
                    se = se + w;
                    for (int d = 0; d < head_dim; d++) {
                        float t = w * v[d];
                        o[d] = o[d] + t;
                    }
                }
            }
            if (se > 0.0f) {
                float inv = 1.0f / se;
                for (int d = 0; d < head_dim; d++) o[d] = o[d] * inv;
            }
        }
}

/* ---- code embedding, channel-first [292, n_frames] (voxtral_tts_codec.c:276-300) --------- */
void orc_codec_embed_codes(const float *semantic_embedding, const int *codes, int n_frames, float *out) {
    for (int t = 0; t < n_frames; t++) {
        const int *fc = codes + t * ORC_CODES_PER_FRAME;
        int sem = fc[0] - 2;
        if (sem < 0) sem = 0;
        if (sem >= ORC_SEM_SIZE) sem = ORC_SEM_SIZE - 1;
        for (int d = 0; d < ORC_CODEC_SEM_DIM; d++)
            out[(size_t)d * n_frames + t] = semantic_embedding[sem * ORC_CODEC_SEM_DIM + d];
        for (int i = 0; i < ORC_ACOUSTIC_DIM; i++) {
            int ac = fc[i + 1] - 2;
            if (ac < 0) ac = 0;
            if (ac >= ORC_FSQ_LEVELS) ac = ORC_FSQ_LEVELS - 1;
            float val = (float)ac * 2.0f / (float)(ORC_FSQ_LEVELS - 1) - 1.0f;
            out[(size_t)(ORC_CODEC_SEM_DIM + i) * n_frames + t] = val;
        }
    }
}

/* ---- one codec transformer layer, x [seq, 1024] in place (voxtral_tts_codec.c:306-383) --- */
void orc_codec_layer(const orc_codec_layer_t *l, const float *slopes, float *x, int seq) {
    const int dim = ORC_CODEC_DIM, hid = ORC_CODEC_HIDDEN;
    const float scale = 1.0f / sqrtf((float)ORC_CODEC_HEAD_DIM);
    float *xn = malloc(sizeof(float) * (size_t)seq * dim), *q = malloc(sizeof(float) * (size_t)seq * dim);
    float *k = malloc(sizeof(float) * (size_t)seq * dim), *v = malloc(sizeof(float) * (size_t)seq * dim);
    float *att = malloc(sizeof(float) * (size_t)seq * dim), *proj = malloc(sizeof(float) * (size_t)seq * dim);
    float *gate = malloc(sizeof(float) * (size_t)seq * hid), *up = malloc(sizeof(float) * (size_t)seq * hid);

    orc_rms_norm(xn, x, l->attention_norm, seq, dim, ORC_CODEC_EPS);
    orc_linear_f32(q, xn, l->wq, seq, dim, dim);
    orc_linear_f32(k, xn, l->wk, seq, dim, dim);
    orc_linear_f32(v, xn, l->wv, seq, dim, dim);
    if (l->q_norm) orc_rms_norm(q, q, l->q_norm, seq, dim, 1e-6f);
    if (l->k_norm) orc_rms_norm(k, k, l->k_norm, seq, dim, 1e-6f);
    orc_alibi_attention(att, q, k, v, seq, ORC_CODEC_HEADS, ORC_CODEC_HEADS, ORC_CODEC_HEAD_DIM, scale,
                        l->window_size, slopes);
    orc_linear_f32(proj, att, l->wo, seq, dim, dim);
    for (size_t i = 0; i < (size_t)seq * dim; i++) {
        float t = l->attn_scale ? proj[i] * l->attn_scale[i % dim] : proj[i];
        x[i] = x[i] + t;
    }
    orc_rms_norm(xn, x, l->ffn_norm, seq, dim, ORC_CODEC_EPS);
    orc_linear_f32(gate, xn, l->w1, seq, dim, hid);
    orc_linear_f32(up, xn, l->w3, seq, dim, hid);
    orc_silu(gate, seq * hid);
    orc_mul_inplace(gate, up, seq * hid);
    orc_linear_f32(proj, gate, l->w2, seq, hid, dim);
    for (size_t i = 0; i < (size_t)seq * dim; i++) {
        float t = l->ffn_scale ? proj[i] * l->ffn_scale[i % dim] : proj[i];
        x[i] = x[i] + t;
    }
    free(xn); free(q); free(k); free(v); free(att); free(proj); free(gate); free(up);
}

static void transpose(float *dst, const float *src, int rows, int cols) {   /* src [rows, cols] */
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) dst[(size_t)c * rows + r] = src[(size_t)r * cols + c];
}

/* ---- codes [n_frames, 37] -> waveform [n_frames * 8 * 240] (voxtral_tts_codec.c:389-503).
 *      Returns the number of samples written to out (capacity n_frames * 1920). ------------ */
int orc_codec_decode(const orc_codec_t *c, const int *codes, int n_frames, float *out) {
    const int dim = ORC_CODEC_DIM;
    int len = n_frames;
    float *emb = calloc((size_t)ORC_CODEC_EMBED * len, sizeof(float));
    float *cf = calloc((size_t)dim * (len + 16), sizeof(float));
    orc_codec_embed_codes(c->semantic_embedding, codes, len, emb);
    orc_causal_conv1d(cf, emb, c->input_conv.weight, c->input_conv.bias, ORC_CODEC_EMBED, dim, len,
                      c->input_conv.kernel, c->input_conv.stride);
    free(emb);
    float *x = malloc(sizeof(float) * (size_t)len * dim);
    transpose(x, cf, dim, len);
    free(cf);
    int li = 0;
    for (int stage = 0; stage < ORC_CODEC_STAGES; stage++) {
        for (int l = 0; l < 2; l++) orc_codec_layer(&c->layers[li++], c->alibi_slopes, x, len);
        if (stage < ORC_CODEC_STAGES - 1) {
            const orc_conv_t *u = &c->stage_convs[stage];
            float *in_cf = malloc(sizeof(float) * (size_t)dim * len);
            transpose(in_cf, x, len, dim);
            float *up = calloc((size_t)dim * (len * u->stride + u->kernel + 8), sizeof(float));
            int nl = orc_causal_conv_transpose_1d(up, in_cf, u->weight, u->bias, u->in_ch, u->out_ch, len,
                                                  u->kernel, u->stride);
            free(in_cf);
            free(x);
            x = malloc(sizeof(float) * (size_t)nl * dim);
            transpose(x, up, dim, nl);
            free(up);
            len = nl;
        }
    }
    float *fin = malloc(sizeof(float) * (size_t)dim * len);
    transpose(fin, x, len, dim);
    free(x);
    float *proj = calloc((size_t)ORC_CODEC_PATCH * (len + 16), sizeof(float));
    orc_causal_conv1d(proj, fin, c->output_proj.weight, c->output_proj.bias, dim, ORC_CODEC_PATCH, len,
                      c->output_proj.kernel, c->output_proj.stride);
    free(fin);
    transpose(out, proj, ORC_CODEC_PATCH, len);
    free(proj);
    return len * ORC_CODEC_PATCH;
}
