/*
 * voxtral_tts_hip.h - C ABI of the MI355X (gfx950) backend for the
 * voxtral-tts.c LLM-backbone / acoustic-transformer hot path.
 *
 * The entry points mirror, one for one, the GPU backend interface of the
 * reference (voxtral_tts_cuda.h:89-185): same argument order and meaning,
 * same host-pointer / device-pointer conventions, same `int` 0 / -1 results
 * for init and uploads and `void` compute entry points.  The reference
 * declaration each one replaces is cited at its prototype.  Entry points with
 * no counterpart in the reference are grouped at the end and say so.
 *
 * Plain C, no HIP or torch types in any signature: device memory is passed as
 * `void *` / `float *` addresses obtained from tts_hip_alloc (or from any
 * other allocator of the same HIP device).
 *
 * One global context, not thread-safe, one internal stream; every entry
 * point that takes host pointers is synchronous, every entry point that
 * takes device pointers is asynchronous on the internal stream (call
 * tts_hip_sync) - the conventions of the reference backend.
 */
#ifndef VOXTRAL_TTS_HIP_H
#define VOXTRAL_TTS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTS_HIP_DEC_LAYERS 26
#define TTS_HIP_AC_LAYERS  3

/* ---- host-side weight structs consumed through `void *` -------------------
 * Field order and types are the upload ABI: they equal tts_dec_layer_t /
 * tts_decoder_t (voxtral_tts.h:101-125) and tts_ac_layer_t / tts_acoustic_t
 * (voxtral_tts.h:131-165), so a pointer to the reference's structs can be
 * passed unchanged. */
typedef struct {
    uint16_t *wq_bf16;        /* [4096, 3072] */
    uint16_t *wk_bf16;        /* [1024, 3072] */
    uint16_t *wv_bf16;        /* [1024, 3072] */
    uint16_t *wo_bf16;        /* [3072, 4096] */
    float *attention_norm;    /* [3072] */
    uint16_t *w1_bf16;        /* [9216, 3072] gate */
    uint16_t *w2_bf16;        /* [3072, 9216] down */
    uint16_t *w3_bf16;        /* [9216, 3072] up */
    float *ffn_norm;          /* [3072] */
} tts_hip_host_layer_t;

typedef struct {
    uint16_t *tok_embeddings_bf16;                    /* [131072, 3072] or NULL */
    tts_hip_host_layer_t layers[TTS_HIP_DEC_LAYERS];
    float *norm;                                      /* [3072] */
} tts_hip_host_decoder_t;

typedef struct {
    float *time_inv_freq;              /* [1536] */
    uint16_t *input_proj_bf16;         /* [3072, 36] */
    uint16_t *time_proj_bf16;          /* [3072, 3072] */
    uint16_t *llm_proj_bf16;           /* [3072, 3072] */
    uint16_t *semantic_out_bf16;       /* [8320, 3072] */
    float *semantic_out_bias;          /* [8320] or NULL */
    uint16_t *acoustic_out_bf16;       /* [36, 3072] */
    float *norm;                       /* [3072] */
    tts_hip_host_layer_t layers[TTS_HIP_AC_LAYERS];
} tts_hip_host_acoustic_t;

/* Audio codec decoder weights: field order and types equal tts_conv_t / tts_codec_layer_t /
 * tts_codec_t (voxtral_tts.h:172-225), so a pointer to the reference's struct can be passed
 * unchanged.  All tensors fp32 (weight norm already folded, voxtral_tts_codec.c:38-57). */
typedef struct {
    float *weight;            /* conv1d [out_ch, in_ch, kernel]; transposed [in_ch, out_ch, kernel] */
    float *bias;              /* [out_ch] or NULL */
    int in_ch, out_ch, kernel, stride, is_transpose;
} tts_hip_host_conv_t;

typedef struct {
    float *wq, *wk, *wv, *wo; /* [1024, 1024] */
    float *q_norm, *k_norm;   /* [1024] or NULL */
    float *attention_norm;    /* [1024] */
    float *w1, *w2, *w3;      /* [4096, 1024] [1024, 4096] [4096, 1024] */
    float *ffn_norm;          /* [1024] */
    float *attn_scale, *ffn_scale;   /* [1024] layer scale, or NULL */
    int window_size;
} tts_hip_host_codec_layer_t;

typedef struct {
    float *semantic_embedding;                 /* [8192, 256] */
    tts_hip_host_conv_t input_conv;            /* 292 -> 1024, k 3, s 1 */
    tts_hip_host_codec_layer_t transformers[8];
    tts_hip_host_conv_t stage_convs[4];        /* 3 used: transposed 1024 -> 1024, k 4, s 2 */
    tts_hip_host_conv_t output_proj;           /* 1024 -> 240, k 7, s 1 */
    float alibi_slopes[8];
} tts_hip_host_codec_t;

/* ---- exported context (replaces the fields of `g_cuda` that code outside the
 * backend touches: voxtral_tts_cuda.h:51-54,78 read at voxtral_tts_llm.c:380-381) */
typedef struct {
    float *kv_cache_k_gpu;    /* f32 [26, kv_cache_max, 1024] */
    float *kv_cache_v_gpu;
    int kv_cache_max;
    int initialized;
    int n_cu;                 /* compute units of the device */
    int dec_layers_uploaded;
    int ac_layers_uploaded;
} tts_hip_ctx_t;

extern tts_hip_ctx_t g_hip;

/* ---- init / upload / teardown -------------------------------------------- */

/* replaces tts_cuda_init (voxtral_tts_cuda.h:89). Idempotent. 0 / -1. */
int tts_hip_init(int kv_cache_max);
/* replaces tts_cuda_upload_llm_weights (voxtral_tts_cuda.h:92); decoder_ptr is a
 * tts_decoder_t * / tts_hip_host_decoder_t *.  Copies; the host keeps ownership. */
int tts_hip_upload_llm_weights(void *decoder_ptr);
/* replaces tts_cuda_upload_acoustic_weights (voxtral_tts_cuda.h:93). */
int tts_hip_upload_acoustic_weights(void *acoustic_ptr);
/* replaces tts_cuda_free (voxtral_tts_cuda.h:96). */
void tts_hip_free(void);
/* replaces tts_cuda_available (voxtral_tts_cuda.h:99). */
int tts_hip_available(void);

/* ---- linear ---------------------------------------------------------------- */

/* replaces tts_cuda_linear_bf16 (voxtral_tts_cuda.h:109-111): y = x W^T, x and y
 * each host or device, W_gpu device bf16 [out_dim, in_dim]; W_gpu == NULL
 * uploads W_bf16 from the host for the call. */
void tts_hip_linear_bf16(float *y, const float *x, const uint16_t *W_bf16,
                         int seq_len, int in_dim, int out_dim, const void *W_gpu);

/* ---- kernel-level operators on device pointers ---------------------------- */

/* replaces tts_cuda_rms_norm (voxtral_tts_cuda.h:118-119) */
void tts_hip_rms_norm(float *d_out, const float *d_x, const float *d_weight,
                      int seq_len, int dim, float eps);
/* replaces tts_cuda_apply_rope (voxtral_tts_cuda.h:122-123); d_freqs is
 * f32 [seq, head_dim/2, 2] (cos, sin) and IS honoured (the reference ignores it). */
void tts_hip_apply_rope(float *d_x, const float *d_freqs, int seq, int heads, int head_dim);
/* replaces tts_cuda_compute_rope_freqs (voxtral_tts_cuda.h:126-127), a stub in
 * the reference; here it fills d_freqs for positions start_pos..start_pos+seq-1. */
void tts_hip_compute_rope_freqs(float *d_freqs, int start_pos, int seq, int dim, float theta);
/* replaces tts_cuda_silu_mul (voxtral_tts_cuda.h:130) */
void tts_hip_silu_mul(float *d_gate, const float *d_up, int n);
/* replaces tts_cuda_add_inplace (voxtral_tts_cuda.h:133) */
void tts_hip_add_inplace(float *d_a, const float *d_b, int n);
/* replaces tts_cuda_causal_attention_decode (voxtral_tts_cuda.h:136-139);
 * kv_cache_stride is the row stride in floats (0 = n_kv_heads*head_dim). */
void tts_hip_causal_attention_decode(float *d_out, const float *d_Q, const float *d_K_cache,
                                     const float *d_V_cache, int seq_k, int n_heads,
                                     int n_kv_heads, int head_dim, float scale,
                                     int kv_cache_stride);
/* replaces tts_cuda_causal_attention_prefill (voxtral_tts_cuda.h:142-145).  With the model's head
 * counts and 8 or more queries it runs on the matrix cores, from tile images of K and V that a first
 * kernel writes into a buffer of the library's own (8 x ceil((start_pos + seq_len) / 32) x 37 KB,
 * allocated when a call needs more than any before it). */
void tts_hip_causal_attention_prefill(float *d_out, const float *d_Q, const float *d_K,
                                      const float *d_V, int seq_len, int start_pos,
                                      int n_heads, int n_kv_heads, int head_dim, float scale);
/* replaces tts_cuda_bidirectional_attention (voxtral_tts_cuda.h:148-150) */
void tts_hip_bidirectional_attention(float *d_out, const float *d_Q, const float *d_K,
                                     const float *d_V, int seq_len, int n_heads,
                                     int n_kv_heads, int head_dim, float scale);
/* replaces tts_cuda_embed_token (voxtral_tts_cuda.h:153-154) */
void tts_hip_embed_token(float *d_out, const void *d_embeddings_bf16, int token_id, int dim);

/* ---- backbone --------------------------------------------------------------- */

/* replaces tts_cuda_llm_forward (voxtral_tts_cuda.h:161-162): one decode step
 * at cache position pos; host pointers; synchronous. */
void tts_hip_llm_forward(float *out_hidden, const float *input_embed, int pos);
/* replaces tts_cuda_llm_prefill (voxtral_tts_cuda.h:165): fills cache rows
 * start_pos..start_pos+seq_len-1 on the device; host pointer; synchronous. */
void tts_hip_llm_prefill(const float *embeds, int seq_len, int start_pos);

/* ---- acoustic transformer -------------------------------------------------- */

/* replaces tts_cuda_predict_velocity (voxtral_tts_cuda.h:172-174) */
void tts_hip_predict_velocity(float *out_velocity, const float *x_t,
                              const float *llm_hidden, float t_val);

/* ---- transfers --------------------------------------------------------------- */

/* replace tts_cuda_to_device / to_host / memset / alloc / free_ptr / sync
 * (voxtral_tts_cuda.h:180-185) */
void tts_hip_to_device(void *d_dst, const void *h_src, size_t bytes);
void tts_hip_to_host(void *h_dst, const void *d_src, size_t bytes);
void tts_hip_memset(void *d_ptr, int value, size_t bytes);
void *tts_hip_alloc(size_t bytes);
void tts_hip_free_ptr(void *d_ptr);
void tts_hip_sync(void);

/* ==== entry points with no counterpart in the reference ===================== */

/* Upload only the first n_layers decoder layers (1..26); used for one-layer
 * and few-layer configurations.  Sources may be host or device pointers. */
int tts_hip_upload_llm_weights_n(void *decoder_ptr, int n_layers);
/* Upload one decoder layer (index 0..25) from host or device pointers. */
int tts_hip_upload_llm_layer(int layer, const tts_hip_host_layer_t *src);
/* Final-norm weights f32 [3072], host or device pointer. */
int tts_hip_upload_llm_norm(const float *norm);

/* One decode step on device-resident buffers, asynchronous on the internal
 * stream: d_input_embed f32 [3072] -> d_out_hidden f32 [3072]. */
void tts_hip_llm_forward_device(float *d_out_hidden, const float *d_input_embed, int pos);
/* One decoder layer at batch 1 on a device-resident hidden state (in place),
 * appending row pos of that layer's cache.  Asynchronous. */
void tts_hip_layer_decode(int layer, float *d_hidden, int pos);
/* Prefill that also returns the residual stream after the last layer
 * ([seq_len, 3072], host pointer, may be NULL). */
void tts_hip_llm_prefill_out(const float *embeds, int seq_len, int start_pos, float *out_x);

/* Conditional + unconditional velocity in one batch-2 pass (classifier-free
 * guidance): equals predict_velocity(x_t, llm_hidden, t) and
 * predict_velocity(x_t, 0, t) (voxtral_tts_acoustic.c:345-348). */
void tts_hip_predict_velocity_cfg(float *out_v_cond, float *out_v_uncond, const float *x_t,
                                  const float *llm_hidden, float t_val);
/* One audio frame on the device: semantic head + argmax, 7 Euler steps with
 * CFG from the caller's noise x0[36], FSQ quantisation -> codes[37]
 * (voxtral_tts_acoustic.c:268-373).  Host pointers; synchronous.  out_x
 * (optional) receives the final latent. */
void tts_hip_acoustic_frame(int *out_codes, const float *llm_hidden, const float *x0,
                            float *out_x);

/* Audio-code embedding table bf16 [total_rows, 3072] and the first row of each of the 37
 * codebooks (tts_audio_embed_t, voxtral_tts.h:226-236; tts_audio_embed_load,
 * voxtral_tts_voice.c:251-290).  Host or device pointers; copies.  0 / -1. */
int tts_hip_upload_audio_embeddings(const uint16_t *emb_bf16, int total_rows, const int *offsets);
/* replaces tts_audio_embed_forward (voxtral_tts_voice.c:292-315): host codes [37] -> host
 * embedding [3072], the 37 rows summed in codebook order; synchronous. */
void tts_hip_audio_embed(float *out_embed, const int *codes);
/* One turn of the generation loop of voxtral_tts.c:301-321 on the device: backbone step at
 * cache position pos on d_embed (device, f32 [3072]) -> frame of 37 codes from the noise x0
 * (host, f32 [36]) -> embedding of the codes written back to d_embed.  Synchronous; returns
 * the codes (END_AUDIO: codes[0] == 1, the rest 2). */
void tts_hip_generate_frame(int *out_codes, float *d_embed, const float *x0, int pos);

/* Audio codec decoder on the device (the reference runs it on the CPU only).  Upload: codec_ptr
 * is a tts_codec_t * / tts_hip_host_codec_t * (tts_codec_load fills it, voxtral_tts_codec.c:
 * 177-270); tensors may be host or device memory; copies.  0 / -1. */
int tts_hip_upload_codec_weights(void *codec_ptr);
/* replaces tts_codec_decode (voxtral_tts_codec.c:389-503): host codes [n_frames, 37] ->
 * *out_samples, a malloc'ed waveform of *out_n_samples = n_frames * 1920 floats that the caller
 * frees (NULL / 0 on failure); synchronous.  At most 4096 frames per call. */
void tts_hip_codec_decode(const int *codes, int n_frames, float **out_samples, int *out_n_samples);
/* The same with device buffers (d_codes [n_frames, 37], d_samples [n_frames * 1920]), queued
 * on the library's stream without synchronising; 0 / -1. */
int tts_hip_codec_decode_device(const int *d_codes, int n_frames, float *d_samples);

/* Checkpoint file -> device in one call, in place of the host-side loading that precedes
 * the uploads in the reference (safetensors_open / safetensors_find / safetensors_data,
 * voxtral_tts_safetensors.c:204-405; tts_decoder_load, voxtral_tts_llm.c:45-100;
 * tts_acoustic_load, voxtral_tts_acoustic.c:40-130; tts_audio_embed_load,
 * voxtral_tts_voice.c:251-290).  Maps the .safetensors file and uploads what it holds under
 * the reference's tensor names: backbone layers 0..n-1 (as many consecutive ones as are
 * present) with norm.weight and the token embeddings, the acoustic transformer, the
 * audio-code embedding table, the codec decoder (tts_codec_load, voxtral_tts_codec.c:177-270,
 * weight norm folded).  Returns a bit mask (1 backbone, 2 acoustic, 4 audio-code embeddings,
 * 8 codec decoder) or -1; tts_hip_init first. */
int tts_hip_load_safetensors(const char *path);
/* Looks one tensor of a .safetensors file up without touching the GPU (safetensors_find,
 * voxtral_tts_safetensors.c:330-345): 0 and dtype (8 chars), rank, shape (4 entries) and
 * byte size; 1 if the file has no such tensor; -1 if the file cannot be read. */
int tts_hip_safetensors_probe(const char *path, const char *name, char *dtype8, int *rank,
                              long long *shape4, long long *nbytes);

/* y[seq_len, out_dim] = x[seq_len, in_dim] W[out_dim, in_dim]^T on device pointers, like
 * tts_hip_linear_bf16 with device buffers and the same kernels, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that forbid it).  No
 * counterpart in the reference.  The work area of the matrix-core path (two bf16 planes of x and
 * the partial planes of a K cut) is a fixed array of 16 MiB that every GPU the library runs on
 * holds until the process ends; a product that needs more is refused with an error (use
 * tts_hip_linear_bf16).  Calls no hipMalloc / hipFree.  All calls on one GPU share the array:
 * calls that overlap on one GPU race.  Asynchronous on the library's stream; 0 / -1. */
int tts_hip_linear_bf16_noalloc(float *d_y, const float *d_x, int seq_len, int in_dim, int out_dim,
                                const void *d_W);

/* The table the loader uses when a checkpoint has no `time_embedding.inv_freq`: out[i] =
 * expf(-logf(10000) * i / half_dim) for i < half_dim (the fallback of tts_acoustic_load,
 * voxtral_tts_acoustic.c:48-60).  Host pointer; touches no GPU state. */
void tts_hip_default_time_inv_freq(float *out, int half_dim);

/* Decode schedule: 0 = persistent whole-step kernel (default; a device on which its grid cannot be
 * resident at once runs schedule 1 instead), 1 = one kernel per phase.  Other values are an error
 * and leave the schedule as it is. */
void tts_hip_set_decode_mode(int mode);
/* Prefill schedule: 0 (default) = one launch per product and row pass; 1 = per layer, everything behind the
 * attention (output projection, residual + RMSNorm, gate|up with SiLU*up, down projection, residual + next
 * RMSNorm, next layer's q|k|v) is one persistent launch whose work items wait for each other per block of 128
 * rows.  The results are the same, bit for bit; schedule 1 measures 3-9 % slower (its dependency waits cost
 * more than the launch boundaries they replace) and is kept as a cross-check.  A context without the
 * fragment-order weight copies, or a device on which the persistent grid cannot be resident, runs schedule 0.
 * Other values are an error.  No counterpart in the reference. */
void tts_hip_set_prefill_mode(int mode);
/* Spin budget of one grid barrier of the whole-step kernel, in ticks of the 100 MHz wall clock
 * (0 = the default of 0.2 s).  When it runs out every workgroup leaves the kernel and the result is
 * invalid.  Entry points with host pointers (tts_hip_llm_forward, tts_hip_generate_frame) report
 * that themselves; after the asynchronous ones (tts_hip_llm_forward_device, tts_hip_layer_decode)
 * it is reported, once, by the next call that waits for the stream: tts_hip_sync, tts_hip_to_host,
 * tts_hip_to_device, tts_hip_memset.
 * The report resets the barrier; the next step starts clean. */
void tts_hip_set_barrier_timeout(unsigned long long ticks);
/* Workgroups of the backbone's whole-step decode kernel: 0 (the default) = the CU count rounded down to
 * a multiple of 8, else a multiple of 8 from 72 up to that.  Waits for the library's stream.  Results
 * agree to rounding, not bit for bit (the attention's key chunks follow the grid).  No counterpart in
 * the reference. */
void tts_hip_set_decode_grid(int workgroups);
/* Workgroups of the acoustic transformer's product kernels: 0 (the default) = one per CU, else
 * 1 .. the CU count.  The results do not depend on it, bit for bit (a unit of 12 weight rows is summed the
 * same way whichever workgroup takes it); a smaller grid leaves CUs to other work and makes a workgroup
 * walk more units.  No counterpart in the reference. */
void tts_hip_set_acoustic_grid(int workgroups);
/* Number of failed calls since init, and the text of the last failure. */
int tts_hip_error_count(void);
const char *tts_hip_last_error(void);

/* The activation format of the sequence-level products: n fp32 values (n even, device pointers,
 * 8-byte aligned) -> two bf16 planes, hi = bf16(x) rounded to nearest even and lo = bf16(x - hi),
 * so that hi + lo carries x to about 2^-17 relative (tts_hip_linear_bf16 with seq_len >= 8 and
 * tts_hip_llm_prefill multiply every weight tile with both planes).  No counterpart in the
 * reference, whose CPU products read the fp32 activations directly (voxtral_tts_kernels.c:127-138);
 * exported so that the format can be checked bit for bit.  Returns 0, or -1 on error. */
int tts_hip_split_planes(uint16_t *d_hi, uint16_t *d_lo, const float *d_x, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* VOXTRAL_TTS_HIP_H */
