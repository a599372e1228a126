/*
 * voxtral_tts_cuda.h (drop-in) - lets the reference's UNMODIFIED host files
 * (voxtral_tts.c, voxtral_tts_llm.c, voxtral_tts_acoustic.c, test_kernels.c)
 * compile with -DUSE_CUDA against the gfx950 backend: every `tts_cuda_*` name
 * and the global `g_cuda` they use is aliased to its `tts_hip_*` / `g_hip`
 * counterpart declared in ../voxtral_tts_hip.h.  Names only; no CUDA runtime
 * call is emulated.
 *
 * Use it in place of the reference's header of the same name, or force it in
 * front with `-include include/compat/voxtral_tts_cuda.h` (it defines the same
 * include guard, so the reference's own header then expands to nothing).
 * Interface replaced: voxtral_tts_cuda.h:14-194 of the reference.
 */
#ifndef VOXTRAL_TTS_CUDA_H
#define VOXTRAL_TTS_CUDA_H

#include "../voxtral_tts_hip.h"

#ifdef USE_CUDA

/* the context type of the exported global; only kv_cache_k_gpu / kv_cache_v_gpu / kv_cache_max /
 * initialized are read from outside the backend (voxtral_tts_llm.c:380-381); the per-layer
 * device pointers of tts_cuda_layer_weights_t are private to the backend and have no alias */
#define tts_cuda_ctx_t                      tts_hip_ctx_t
#define g_cuda                              g_hip
#define tts_cuda_init                       tts_hip_init
#define tts_cuda_upload_llm_weights         tts_hip_upload_llm_weights
#define tts_cuda_upload_acoustic_weights    tts_hip_upload_acoustic_weights
#define tts_cuda_free                       tts_hip_free
#define tts_cuda_available                  tts_hip_available
#define tts_cuda_linear_bf16                tts_hip_linear_bf16
#define tts_cuda_rms_norm                   tts_hip_rms_norm
#define tts_cuda_apply_rope                 tts_hip_apply_rope
#define tts_cuda_compute_rope_freqs         tts_hip_compute_rope_freqs
#define tts_cuda_silu_mul                   tts_hip_silu_mul
#define tts_cuda_add_inplace                tts_hip_add_inplace
#define tts_cuda_causal_attention_decode    tts_hip_causal_attention_decode
#define tts_cuda_causal_attention_prefill   tts_hip_causal_attention_prefill
#define tts_cuda_bidirectional_attention    tts_hip_bidirectional_attention
#define tts_cuda_embed_token                tts_hip_embed_token
#define tts_cuda_llm_forward                tts_hip_llm_forward
#define tts_cuda_llm_prefill                tts_hip_llm_prefill
#define tts_cuda_predict_velocity           tts_hip_predict_velocity
#define tts_cuda_to_device                  tts_hip_to_device
#define tts_cuda_to_host                    tts_hip_to_host
#define tts_cuda_memset                     tts_hip_memset
#define tts_cuda_alloc                      tts_hip_alloc
#define tts_cuda_free_ptr                   tts_hip_free_ptr
#define tts_cuda_sync                       tts_hip_sync

#else /* !USE_CUDA: same stubs as the reference (voxtral_tts_cuda.h:187-194) */

static inline int tts_cuda_available(void) { return 0; }
static inline int tts_cuda_init(int kv_cache_max) { (void)kv_cache_max; return -1; }
static inline void tts_cuda_free(void) {}

#endif
#endif /* VOXTRAL_TTS_CUDA_H */
