/*
 * ref_shim.c - thin driver around the UNMODIFIED reference sources.
 *
 * TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile (target `ref`)
 * together with the reference's own C files, taken where they lie under
 * $(REF) (default /root/reference), into oracle/_ref/libvoxtral_ref.so.
 * No reference source text is kept in this repository: this file only
 * includes the reference headers / one reference translation unit by name
 * and fills the reference's own structs with caller-provided buffers, so
 * that tests can run tts_llm_forward / tts_llm_prefill /
 * tts_acoustic_forward / predict_velocity on synthetic weights without a
 * checkpoint on disk.
 */
#include "voxtral_tts.h"
#include "voxtral_tts_kernels.h"

/* predict_velocity is file-static in the reference; pulling the translation
 * unit in by name makes it callable from the wrapper below. */
#include "voxtral_tts_acoustic.c"

#include <stdlib.h>
#include <string.h>

tts_ctx_t *ref_ctx_new(int kv_max) {
    tts_ctx_t *ctx = (tts_ctx_t *)calloc(1, sizeof(tts_ctx_t));
    if (!ctx) return NULL;
    if (kv_max > 0 && tts_llm_kv_cache_alloc(ctx, kv_max) != 0) { free(ctx); return NULL; }
    tts_rng_seed(&ctx->rng_state, 0);
    return ctx;
}

/* Frees only what the shim or the reference's lazy allocators made; weight
 * buffers belong to the caller. */
void ref_ctx_free(tts_ctx_t *ctx) {
    if (!ctx) return;
    free(ctx->kv_cache_k); free(ctx->kv_cache_v);
    free(ctx->dec_x); free(ctx->dec_x_norm); free(ctx->dec_q); free(ctx->dec_k);
    free(ctx->dec_v); free(ctx->dec_attn_out); free(ctx->dec_proj_out);
    free(ctx->dec_gate); free(ctx->dec_up); free(ctx->dec_ffn_out);
    free(ctx->ac_tokens); free(ctx->ac_tokens_norm); free(ctx->ac_q); free(ctx->ac_k);
    free(ctx->ac_v); free(ctx->ac_attn_out); free(ctx->ac_proj_out); free(ctx->ac_gate);
    free(ctx->ac_up); free(ctx->ac_ffn_out); free(ctx->ac_time_emb);
    free(ctx->ac_velocity); free(ctx->ac_noise);
    free(ctx);
}

int ref_dec_layers(void) { return TTS_DEC_LAYERS; }
int ref_ac_layers(void) { return TTS_AC_LAYERS; }

void ref_set_dec_layer(tts_ctx_t *ctx, int i, uint16_t *wq, uint16_t *wk, uint16_t *wv,
                       uint16_t *wo, float *attention_norm, uint16_t *w1, uint16_t *w2,
                       uint16_t *w3, float *ffn_norm) {
    tts_dec_layer_t *l = &ctx->decoder.layers[i];
    l->wq_bf16 = wq; l->wk_bf16 = wk; l->wv_bf16 = wv; l->wo_bf16 = wo;
    l->attention_norm = attention_norm;
    l->w1_bf16 = w1; l->w2_bf16 = w2; l->w3_bf16 = w3;
    l->ffn_norm = ffn_norm;
}

void ref_set_dec_norm(tts_ctx_t *ctx, float *norm) { ctx->decoder.norm = norm; }

void ref_set_ac_layer(tts_ctx_t *ctx, int i, uint16_t *wq, uint16_t *wk, uint16_t *wv,
                      uint16_t *wo, float *attention_norm, uint16_t *w1, uint16_t *w2,
                      uint16_t *w3, float *ffn_norm) {
    tts_ac_layer_t *l = &ctx->acoustic.layers[i];
    l->wq_bf16 = wq; l->wk_bf16 = wk; l->wv_bf16 = wv; l->wo_bf16 = wo;
    l->attention_norm = attention_norm;
    l->w1_bf16 = w1; l->w2_bf16 = w2; l->w3_bf16 = w3;
    l->ffn_norm = ffn_norm;
}

void ref_set_acoustic(tts_ctx_t *ctx, float *time_inv_freq, uint16_t *input_proj,
                      uint16_t *time_proj, uint16_t *llm_proj, uint16_t *semantic_out,
                      float *semantic_out_bias, uint16_t *acoustic_out, float *norm) {
    tts_acoustic_t *ac = &ctx->acoustic;
    ac->time_inv_freq = time_inv_freq;
    ac->input_proj_bf16 = input_proj;
    ac->time_proj_bf16 = time_proj;
    ac->llm_proj_bf16 = llm_proj;
    ac->semantic_out_bf16 = semantic_out;
    ac->semantic_out_bias = semantic_out_bias;
    ac->acoustic_out_bf16 = acoustic_out;
    ac->norm = norm;
}

float *ref_kv_k(tts_ctx_t *ctx) { return ctx->kv_cache_k; }
float *ref_kv_v(tts_ctx_t *ctx) { return ctx->kv_cache_v; }
int ref_get_kv_len(tts_ctx_t *ctx) { return ctx->kv_cache_len; }
void ref_set_kv_len(tts_ctx_t *ctx, int n) { ctx->kv_cache_len = n; }
void ref_seed(tts_ctx_t *ctx, uint64_t seed) { tts_rng_seed(&ctx->rng_state, seed); }
uint64_t ref_rng_state(tts_ctx_t *ctx) { return ctx->rng_state; }

void ref_llm_forward(tts_ctx_t *ctx, const float *embed, float *out_hidden) {
    tts_llm_forward(ctx, embed, out_hidden);
}

void ref_llm_prefill(tts_ctx_t *ctx, const float *embeds, int seq_len) {
    tts_llm_prefill(ctx, embeds, seq_len);
}

void ref_acoustic_forward(tts_ctx_t *ctx, const float *llm_hidden, int *codes) {
    tts_acoustic_forward(ctx, llm_hidden, codes);
}

void ref_predict_velocity(tts_ctx_t *ctx, const float *x_t, const float *llm_hidden,
                          float t_val, float *out_velocity) {
    if (!ctx->ac_tokens) alloc_acoustic_buffers(ctx);
    predict_velocity(ctx, x_t, llm_hidden, t_val, out_velocity);
}

void ref_time_embedding(tts_ctx_t *ctx, float t_val, float *out) {
    compute_time_embedding(&ctx->acoustic, t_val, out, TTS_AC_DIM);
}

void ref_audio_embed_set(tts_ctx_t *ctx, uint16_t *emb) {
    tts_audio_embed_t *ae = &ctx->audio_embed;
    ae->embeddings_bf16 = emb;
    ae->embed_dim = TTS_DEC_DIM;
    ae->offsets[0] = 0;
    ae->offsets[1] = TTS_SEMANTIC_CB_SIZE + TTS_AUDIO_SPECIAL_COUNT;
    for (int i = 2; i <= TTS_NUM_CODEBOOKS; i++)
        ae->offsets[i] = ae->offsets[i - 1] + TTS_FSQ_LEVELS + TTS_AUDIO_SPECIAL_COUNT;
    ae->total_size = ae->offsets[TTS_NUM_CODEBOOKS];
}

void ref_audio_embed_forward(tts_ctx_t *ctx, const int *codes, float *out) {
    tts_audio_embed_forward(ctx, codes, out);
}

/* Addresses of the weight structs inside the context: what the reference's
 * tts_load passes to the upload entry points (voxtral_tts.c:96-99). */
void *ref_decoder_ptr(tts_ctx_t *ctx) { return &ctx->decoder; }
void *ref_acoustic_ptr(tts_ctx_t *ctx) { return &ctx->acoustic; }
int ref_kv_max(tts_ctx_t *ctx) { return ctx->kv_cache_max; }
