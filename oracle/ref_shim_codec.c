/*
 * ref_shim_codec.c - driver around the UNMODIFIED reference codec decoder.
 *
 * TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile (target `ref`) into
 * oracle/_ref/libvoxtral_ref.so.  The reference's codec translation unit is pulled in by
 * name from $(REF) so that its file-static functions (weight-norm reconstruction, code
 * embedding, one transformer layer) can be called; no reference source text is kept here.
 * The wrappers fill the reference's own structs with caller-provided buffers.
 */
#include "voxtral_tts_codec.c"

#include <stdlib.h>
#include <string.h>

void ref_codec_set_conv(tts_ctx_t *ctx, int which, float *weight, float *bias, int in_ch, int out_ch,
                        int kernel, int stride, int is_transpose) {
    tts_codec_t *c = &ctx->codec;
    tts_conv_t *cv = which == 0 ? &c->input_conv : which == 4 ? &c->output_proj : &c->stage_convs[which - 1];
    cv->weight = weight; cv->bias = bias; cv->in_ch = in_ch; cv->out_ch = out_ch;
    cv->kernel = kernel; cv->stride = stride; cv->is_transpose = is_transpose;
}

void ref_codec_set_layer(tts_ctx_t *ctx, int i, float *wq, float *wk, float *wv, float *wo,
                         float *q_norm, float *k_norm, float *attention_norm, float *w1, float *w2,
                         float *w3, float *ffn_norm, float *attn_scale, float *ffn_scale, int window) {
    tts_codec_layer_t *l = &ctx->codec.transformers[i];
    l->wq = wq; l->wk = wk; l->wv = wv; l->wo = wo; l->q_norm = q_norm; l->k_norm = k_norm;
    l->attention_norm = attention_norm; l->w1 = w1; l->w2 = w2; l->w3 = w3; l->ffn_norm = ffn_norm;
    l->attn_scale = attn_scale; l->ffn_scale = ffn_scale; l->window_size = window;
}

void ref_codec_set_tables(tts_ctx_t *ctx, float *semantic_embedding, const float *slopes) {
    ctx->codec.semantic_embedding = semantic_embedding;
    for (int h = 0; h < TTS_CODEC_HEADS; h++) ctx->codec.alibi_slopes[h] = slopes[h];
}

/* waveform into out (capacity n_frames * 1920); returns the sample count */
int ref_codec_decode(tts_ctx_t *ctx, const int *codes, int n_frames, float *out) {
    float *samples = NULL;
    int n = 0;
    tts_codec_decode(ctx, codes, n_frames, &samples, &n);
    if (samples) { memcpy(out, samples, sizeof(float) * (size_t)n); free(samples); }
    return n;
}

void ref_codec_layer(tts_ctx_t *ctx, int i, float *x, int seq_len) {
    codec_transformer_forward(&ctx->codec.transformers[i], ctx->codec.alibi_slopes, x, seq_len);
}

void ref_codec_embed_codes(tts_ctx_t *ctx, const int *codes, int n_frames, float *out) {
    embed_codes(&ctx->codec, codes, n_frames, out);
}

void ref_weight_norm(float *weight, const float *weight_v, const float *weight_g, int out_ch, int fan_in) {
    float *w = reconstruct_weight_norm(weight_v, weight_g, out_ch, fan_in);
    if (w) { memcpy(weight, w, sizeof(float) * (size_t)out_ch * fan_in); free(w); }
}

void *ref_codec_ptr(tts_ctx_t *ctx) { return &ctx->codec; }
