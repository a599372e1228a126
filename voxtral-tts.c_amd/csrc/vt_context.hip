/*
 * vt_context.hip - context, device memory, weight upload and transfers of the
 * gfx950 backend.  Replaces the context half of the reference backend
 * (voxtral_tts_cuda.cu:56-310): one global context, weights copied at upload
 * (the host keeps ownership), KV cache f32 [26, kv_max, 1024] x 2 on the device.
 *
 * Upload lays the weights out for the decode kernels: wq, wk, wv are stored
 * back to back as one [6144, 3072] matrix and w1 / w3 rows are interleaved
 * into one [18432, 3072] matrix so that a (gate, up) pair is adjacent.
 */
#include "vt_state.h"
#include "vt_gemm.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

extern "C" {
tts_hip_ctx_t g_hip = {0, 0, 0, 0, 0, 0, 0};
}
vt_state g_vt = {};

void vt_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_vt.last_error, sizeof g_vt.last_error, fmt, ap);
    va_end(ap);
    g_vt.error_count++;
    fprintf(stderr, "tts_hip: %s\n", g_vt.last_error);
}

int vt_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    vt_set_error("%s failed: %s", what, hipGetErrorString(e));
    return -1;
}

void *vt_dev_alloc(size_t bytes) {
    void *p = NULL;
    if (vt_check(hipMalloc(&p, bytes), "hipMalloc")) return NULL;
    return p;
}

void *vt_scratch(size_t bytes) {
    if (bytes > g_vt.scratch_bytes) {
        if (g_vt.d_scratch) {
            (void)hipStreamSynchronize(g_vt.stream);
            (void)hipFree(g_vt.d_scratch);
        }
        g_vt.d_scratch = vt_dev_alloc(bytes);
        g_vt.scratch_bytes = g_vt.d_scratch ? bytes : 0;
    }
    return g_vt.d_scratch;
}

/* RoPE table for every cache position, built on the host with the same libm
 * calls and operation order as voxtral_tts_kernels.c:602-614 so that its
 * entries are bit-equal to the CPU path's. */
static int build_rope_table(int kv_max) {
    const int half = VT_HEAD_DIM / 2;
    float *t = (float *)malloc(sizeof(float) * (size_t)kv_max * VT_HEAD_DIM);
    if (!t) { vt_set_error("out of host memory for the RoPE table"); return -1; }
    float freq[VT_HEAD_DIM / 2];
    for (int d = 0; d < half; d++)
        freq[d] = 1.0f / powf(1000000.0f, (float)(2 * d) / (float)VT_HEAD_DIM);
    for (int p = 0; p < kv_max; p++) {
        for (int d = 0; d < half; d++) {
            volatile float ang = (float)p * freq[d];
            t[((size_t)p * half + d) * 2] = cosf(ang);
            t[((size_t)p * half + d) * 2 + 1] = sinf(ang);
        }
    }
    hipError_t e = hipMemcpy(g_vt.d_rope, t, sizeof(float) * (size_t)kv_max * VT_HEAD_DIM,
                             hipMemcpyHostToDevice);
    free(t);
    return vt_check(e, "rope table upload");
}

static void teardown(void);

static int init_context(int kv_cache_max) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
        vt_set_error("no HIP device found");
        return -1;
    }
    VT_TRY(hipGetDevice(&g_vt.device));
    hipDeviceProp_t prop;
    VT_TRY(hipGetDeviceProperties(&prop, g_vt.device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        fprintf(stderr, "tts_hip: warning: built for gfx950, device reports %s\n", prop.gcnArchName);
    g_vt.n_cu = prop.multiProcessorCount;
    g_vt.grid = g_vt.n_cu / VT_KV_HEADS * VT_KV_HEADS;
    if (g_vt.grid < VT_KV_HEADS) { vt_set_error("device has too few compute units"); return -1; }
    if (getenv("TTS_HIP_VERBOSE"))
        fprintf(stderr, "  HIP: %s, %d CUs, %.1f GB, LDS %zu/%zu KB, grid %d\n", prop.gcnArchName,
                g_vt.n_cu, (double)prop.totalGlobalMem / (1 << 30), (size_t)prop.sharedMemPerBlock >> 10,
                (size_t)prop.maxSharedMemoryPerMultiProcessor >> 10, g_vt.grid);

    VT_TRY(hipStreamCreateWithFlags(&g_vt.stream, hipStreamNonBlocking));
    VT_TRY(hipEventCreate(&g_vt.ev0));
    VT_TRY(hipEventCreate(&g_vt.ev1));

    const size_t kv_bytes = (size_t)TTS_HIP_DEC_LAYERS * kv_cache_max * VT_KV_DIM * sizeof(float);
    if (!(g_hip.kv_cache_k_gpu = (float *)vt_dev_alloc(kv_bytes))) return -1;
    if (!(g_hip.kv_cache_v_gpu = (float *)vt_dev_alloc(kv_bytes))) return -1;
    VT_TRY(hipMemset(g_hip.kv_cache_k_gpu, 0, kv_bytes));
    VT_TRY(hipMemset(g_hip.kv_cache_v_gpu, 0, kv_bytes));
    g_hip.kv_cache_max = g_vt.kv_max = kv_cache_max;

    if (!(g_vt.d_rope = (float *)vt_dev_alloc(sizeof(float) * (size_t)kv_cache_max * VT_HEAD_DIM))) return -1;
    if (build_rope_table(kv_cache_max)) return -1;

    const int max_chunks = g_vt.grid / VT_KV_HEADS;
    struct { void **p; size_t bytes; } bufs[] = {
        {(void **)&g_vt.d_layers, sizeof(vt_layer_dev) * TTS_HIP_DEC_LAYERS},
        {(void **)&g_vt.d_dec_norm, sizeof(float) * VT_DIM},
        {(void **)&g_vt.d_x, sizeof(float) * VT_DIM},
        {(void **)&g_vt.d_q, sizeof(float) * VT_Q_DIM},
        {(void **)&g_vt.d_attn, sizeof(float) * VT_Q_DIM},
        {(void **)&g_vt.d_h, sizeof(float) * VT_FFN},
        {(void **)&g_vt.d_att_part, sizeof(float) * VT_HEADS * max_chunks * VT_ATT_STRIDE},
        {(void **)&g_vt.d_att_cnt, sizeof(unsigned) * TTS_HIP_DEC_LAYERS * VT_KV_HEADS},
        {(void **)&g_vt.d_embed, sizeof(float) * VT_DIM},
        {(void **)&g_vt.d_hidden, sizeof(float) * (VT_DIM + 64)},
        {(void **)&g_vt.d_bar_flags, sizeof(unsigned) * (size_t)VT_FLAG_COPIES * VT_FLAG_STRIDE},
        {(void **)&g_vt.d_abort, 256},
        {(void **)&g_vt.d_dummy, 4096},
    };
    for (size_t i = 0; i < sizeof bufs / sizeof bufs[0]; i++) {
        if (!(*bufs[i].p = vt_dev_alloc(bufs[i].bytes))) return -1;
        VT_TRY(hipMemset(*bufs[i].p, 0, bufs[i].bytes));
    }
    g_vt.bar_epoch = 0;
    VT_TRY(hipHostMalloc((void **)&g_vt.h_pin, sizeof(float) * (2 * VT_DIM + 64), hipHostMallocDefault));
    VT_TRY(hipDeviceSynchronize());

    g_hip.n_cu = g_vt.n_cu;
    g_hip.initialized = g_vt.initialized = 1;
    return 0;
}

extern "C" int tts_hip_init(int kv_cache_max) {
    if (g_vt.initialized) return 0;
    if (kv_cache_max <= 0) { vt_set_error("tts_hip_init: kv_cache_max must be positive"); return -1; }
    if (init_context(kv_cache_max)) {
        teardown();                 /* a failed init leaves nothing allocated behind */
        return -1;
    }
    return 0;
}

static void free_frag(vt_layer_frag *g) {
    (void)hipFree(g->wqkv); (void)hipFree(g->wo); (void)hipFree(g->w13); (void)hipFree(g->w2);
    memset(g, 0, sizeof *g);
}

/* The fragment-order copies of a complete backbone layer (6.05 GB for 26 layers, next to the 6.05 GB of
 * the row-major ones).  A failure leaves the layer without them: the prefill then multiplies from the
 * row-major matrices with the 128 x 128 tile kernel, whose K cuts differ, so its results differ in the
 * last bits from those of a context that has the copies; build_frag_or_say reports that. */
static int build_frag(vt_layer_frag *g, const vt_layer_dev *l) {
    free_frag(g);
    struct { uint16_t **dst; const uint16_t *src; int n, k; } m[4] = {
        {&g->wqkv, l->wqkv, VT_QKV_DIM, VT_DIM}, {&g->wo, l->wo, VT_DIM, VT_Q_DIM},
        {&g->w13, l->w13, 2 * VT_FFN, VT_DIM}, {&g->w2, l->w2, VT_DIM, VT_FFN}};
    for (int i = 0; i < 4; i++) {
        if (!(*m[i].dst = (uint16_t *)vt_dev_alloc((size_t)m[i].n * m[i].k * 2))) { free_frag(g); return -1; }
        vt_launch_frag_layout(*m[i].dst, m[i].src, m[i].n, m[i].k, i == 2);      /* gate|up: paired */
    }
    if (vt_check(hipGetLastError(), "fragment layout launch") || vt_check(hipStreamSynchronize(g_vt.stream), "fragment layout")) {
        free_frag(g);
        return -1;
    }
    return 0;
}

static void build_frag_or_say(int layer) {
    if (build_frag(&g_vt.h_frag[layer], &g_vt.h_layers[layer]) == 0) return;
    /* the failed allocation is already on record as an error (vt_set_error); say what follows from it */
    fprintf(stderr, "tts_hip: layer %d has no fragment-order copy of its weights: its prefill products run from the "
                    "row-major matrices (128 x 128 tiles, other K cuts: results differ in the last bits)\n", layer);
}

static void free_layer(vt_layer_dev *l) {
    (void)hipFree((void *)l->wqkv); (void)hipFree((void *)l->wo);
    (void)hipFree((void *)l->w13); (void)hipFree((void *)l->w2);
    (void)hipFree((void *)l->attn_norm); (void)hipFree((void *)l->ffn_norm);
    memset(l, 0, sizeof *l);
}

/* Releases whatever the context holds, complete or not; keeps the error count and message. */
static void teardown(void) {
    (void)hipDeviceSynchronize();
    vt_codec_free();
    for (int i = 0; i < TTS_HIP_DEC_LAYERS; i++) { free_layer(&g_vt.h_layers[i]); free_frag(&g_vt.h_frag[i]); }
    for (int i = 0; i < TTS_HIP_AC_LAYERS; i++) free_layer(&g_vt.ac.layers[i]);
    void *ptrs[] = {g_vt.d_layers, g_vt.d_dec_norm, g_vt.d_tok_emb, g_vt.ac.input_proj,
                    g_vt.ac.time_proj, g_vt.ac.llm_proj, g_vt.ac.semantic_out,
                    g_vt.ac.acoustic_out, g_vt.ac.semantic_bias, g_vt.ac.norm,
                    g_vt.ac.time_inv_freq, g_vt.ac.time_tok, g_vt.ac.audio_emb, g_vt.ac.audio_offsets,
                    g_hip.kv_cache_k_gpu, g_hip.kv_cache_v_gpu,
                    g_vt.d_rope, g_vt.d_x, g_vt.d_q, g_vt.d_attn, g_vt.d_h, g_vt.d_att_part,
                    g_vt.d_att_cnt, g_vt.d_embed, g_vt.d_hidden, g_vt.d_bar_flags,
                    g_vt.d_abort, g_vt.d_dummy, g_vt.d_scratch, g_vt.d_kv_img};
    for (size_t i = 0; i < sizeof ptrs / sizeof ptrs[0]; i++)
        if (ptrs[i]) (void)hipFree(ptrs[i]);
    if (g_vt.h_pin) (void)hipHostFree(g_vt.h_pin);
    if (g_vt.ev0) (void)hipEventDestroy(g_vt.ev0);
    if (g_vt.ev1) (void)hipEventDestroy(g_vt.ev1);
    if (g_vt.stream) (void)hipStreamDestroy(g_vt.stream);
    const int errs = g_vt.error_count;
    char msg[sizeof g_vt.last_error];
    memcpy(msg, g_vt.last_error, sizeof msg);
    memset(&g_vt, 0, sizeof g_vt);
    g_vt.error_count = errs;
    memcpy(g_vt.last_error, msg, sizeof msg);
    memset(&g_hip, 0, sizeof g_hip);
}

extern "C" void tts_hip_free(void) {
    if (!g_vt.initialized) return;
    teardown();
}

extern "C" int tts_hip_available(void) { return g_vt.initialized; }

/* ---- weight upload ----------------------------------------------------------- */

static void *upload(const void *src, size_t bytes) {
    if (!src) { vt_set_error("upload: NULL source tensor"); return NULL; }
    void *d = vt_dev_alloc(bytes);
    if (d && vt_check(hipMemcpy(d, src, bytes, hipMemcpyDefault), "weight copy")) {
        (void)hipFree(d);
        return NULL;
    }
    return d;
}

/* Sources may be host or device memory (hipMemcpyDefault resolves the kind). */
static int upload_layer(vt_layer_dev *dst, const tts_hip_host_layer_t *s) {
    if (!s->wq_bf16 || !s->wk_bf16 || !s->wv_bf16 || !s->wo_bf16 || !s->w1_bf16 ||
        !s->w2_bf16 || !s->w3_bf16 || !s->attention_norm || !s->ffn_norm) {
        vt_set_error("upload: layer has a NULL tensor");
        return -1;
    }
    free_layer(dst);
    const size_t row = (size_t)VT_DIM * 2;
    /* every allocation lands in `dst` at once, so that a failure half way leaks nothing: the next
     * upload of this layer, or the teardown, frees it */
    uint16_t *wqkv = (uint16_t *)vt_dev_alloc((size_t)VT_QKV_DIM * row);
    dst->wqkv = wqkv;
    uint16_t *w13 = (uint16_t *)vt_dev_alloc((size_t)2 * VT_FFN * row);
    dst->w13 = w13;
    if (!wqkv || !w13) return -1;
    VT_TRY(hipMemcpy(wqkv, s->wq_bf16, (size_t)VT_Q_DIM * row, hipMemcpyDefault));
    VT_TRY(hipMemcpy(wqkv + (size_t)VT_Q_DIM * VT_DIM, s->wk_bf16, (size_t)VT_KV_DIM * row, hipMemcpyDefault));
    VT_TRY(hipMemcpy(wqkv + (size_t)(VT_Q_DIM + VT_KV_DIM) * VT_DIM, s->wv_bf16, (size_t)VT_KV_DIM * row,
                     hipMemcpyDefault));
    VT_TRY(hipMemcpy2D(w13, 2 * row, s->w1_bf16, row, row, VT_FFN, hipMemcpyDefault));
    VT_TRY(hipMemcpy2D(w13 + VT_DIM, 2 * row, s->w3_bf16, row, row, VT_FFN, hipMemcpyDefault));
    if (!(dst->wo = (uint16_t *)upload(s->wo_bf16, (size_t)VT_DIM * VT_Q_DIM * 2))) return -1;
    if (!(dst->w2 = (uint16_t *)upload(s->w2_bf16, (size_t)VT_DIM * VT_FFN * 2))) return -1;
    if (!(dst->attn_norm = (float *)upload(s->attention_norm, sizeof(float) * VT_DIM))) return -1;
    if (!(dst->ffn_norm = (float *)upload(s->ffn_norm, sizeof(float) * VT_DIM))) return -1;
    return 0;
}

static int layer_complete(const vt_layer_dev *l) {
    return l->wqkv && l->wo && l->w13 && l->w2 && l->attn_norm && l->ffn_norm;
}

/* The backbone runs over the leading layers that are completely uploaded; the device's copy of
 * the layer table follows the host's after every change, so that it never names freed memory. */
static int publish_dec_layers(void) {
    int n = 0;
    while (n < TTS_HIP_DEC_LAYERS && layer_complete(&g_vt.h_layers[n])) n++;
    g_vt.n_dec_layers = n;
    g_hip.dec_layers_uploaded = n;
    return vt_check(hipMemcpy(g_vt.d_layers, g_vt.h_layers, sizeof g_vt.h_layers, hipMemcpyHostToDevice),
                    "layer table upload");
}

static int need_init(const char *who) {
    if (g_vt.initialized) return 0;
    vt_set_error("%s: tts_hip_init has not succeeded", who);
    return -1;
}

extern "C" int tts_hip_upload_llm_layer(int layer, const tts_hip_host_layer_t *src) {
    if (need_init("tts_hip_upload_llm_layer")) return -1;
    if (layer < 0 || layer >= TTS_HIP_DEC_LAYERS || !src) {
        vt_set_error("tts_hip_upload_llm_layer: bad layer index %d", layer);
        return -1;
    }
    (void)hipStreamSynchronize(g_vt.stream);
    const int bad = upload_layer(&g_vt.h_layers[layer], src);
    if (bad) { free_layer(&g_vt.h_layers[layer]); free_frag(&g_vt.h_frag[layer]); }   /* incomplete: the backbone ends in front of it */
    else build_frag_or_say(layer);
    if (publish_dec_layers()) return -1;
    return bad ? -1 : 0;
}

extern "C" int tts_hip_upload_llm_norm(const float *norm) {
    if (need_init("tts_hip_upload_llm_norm")) return -1;
    if (!norm) { vt_set_error("tts_hip_upload_llm_norm: NULL"); return -1; }
    VT_TRY(hipMemcpy(g_vt.d_dec_norm, norm, sizeof(float) * VT_DIM, hipMemcpyDefault));
    return 0;
}

extern "C" int tts_hip_upload_llm_weights_n(void *decoder_ptr, int n_layers) {
    if (need_init("tts_hip_upload_llm_weights")) return -1;
    tts_hip_host_decoder_t *dec = (tts_hip_host_decoder_t *)decoder_ptr;
    if (!dec || n_layers < 1 || n_layers > TTS_HIP_DEC_LAYERS) {
        vt_set_error("tts_hip_upload_llm_weights: bad arguments");
        return -1;
    }
    if (dec->tok_embeddings_bf16) {
        if (g_vt.d_tok_emb) (void)hipFree(g_vt.d_tok_emb);
        g_vt.d_tok_emb = (uint16_t *)upload(dec->tok_embeddings_bf16, (size_t)131072 * VT_DIM * 2);
        if (!g_vt.d_tok_emb) return -1;
    }
    if (!dec->norm) { vt_set_error("tts_hip_upload_llm_weights: NULL final norm"); return -1; }
    if (tts_hip_upload_llm_norm(dec->norm)) return -1;
    (void)hipStreamSynchronize(g_vt.stream);
    g_vt.n_dec_layers = 0;
    for (int i = 0; i < TTS_HIP_DEC_LAYERS; i++) {
        if (i < n_layers && upload_layer(&g_vt.h_layers[i], &dec->layers[i])) {
            fprintf(stderr, "tts_hip: failed to upload LLM layer %d\n", i);
            free_layer(&g_vt.h_layers[i]);
            free_frag(&g_vt.h_frag[i]);
            (void)publish_dec_layers();
            return -1;
        }
        if (i < n_layers) build_frag_or_say(i);
        if (i >= n_layers) { free_layer(&g_vt.h_layers[i]); free_frag(&g_vt.h_frag[i]); }   /* a shorter backbone than before */
    }
    if (publish_dec_layers()) return -1;
    if (g_vt.n_dec_layers != n_layers) { vt_set_error("tts_hip_upload_llm_weights: internal layer count"); return -1; }
    return 0;
}

extern "C" int tts_hip_upload_llm_weights(void *decoder_ptr) {
    return tts_hip_upload_llm_weights_n(decoder_ptr, TTS_HIP_DEC_LAYERS);
}

extern "C" int tts_hip_upload_acoustic_weights(void *acoustic_ptr) {
    if (need_init("tts_hip_upload_acoustic_weights")) return -1;
    tts_hip_host_acoustic_t *ac = (tts_hip_host_acoustic_t *)acoustic_ptr;
    if (!ac) { vt_set_error("tts_hip_upload_acoustic_weights: NULL"); return -1; }
    vt_acoustic_dev *d = &g_vt.ac;
    (void)hipStreamSynchronize(g_vt.stream);
    void **old[] = {(void **)&d->input_proj, (void **)&d->time_proj, (void **)&d->llm_proj,
                    (void **)&d->semantic_out, (void **)&d->acoustic_out, (void **)&d->semantic_bias,
                    (void **)&d->norm, (void **)&d->time_inv_freq, (void **)&d->time_tok};
    for (size_t i = 0; i < sizeof old / sizeof old[0]; i++) {
        if (*old[i]) (void)hipFree(*old[i]);
        *old[i] = NULL;              /* a failure below must not leave a freed pointer for the teardown */
    }
    g_vt.ac_uploaded = 0;
    g_hip.ac_layers_uploaded = 0;
    d->time_tok_ready = 0;
    if (!(d->time_tok = (float *)vt_dev_alloc(sizeof(float) * 8 * VT_DIM))) return -1;
    if (!(d->input_proj = (uint16_t *)upload(ac->input_proj_bf16, (size_t)VT_DIM * VT_AC_DIM_IN * 2))) return -1;
    if (!(d->time_proj = (uint16_t *)upload(ac->time_proj_bf16, (size_t)VT_DIM * VT_DIM * 2))) return -1;
    if (!(d->llm_proj = (uint16_t *)upload(ac->llm_proj_bf16, (size_t)VT_DIM * VT_DIM * 2))) return -1;
    if (!(d->semantic_out = (uint16_t *)upload(ac->semantic_out_bf16, (size_t)VT_SEM_PADDED * VT_DIM * 2))) return -1;
    if (!(d->acoustic_out = (uint16_t *)upload(ac->acoustic_out_bf16, (size_t)VT_AC_DIM_IN * VT_DIM * 2))) return -1;
    if (ac->semantic_out_bias &&
        !(d->semantic_bias = (float *)upload(ac->semantic_out_bias, sizeof(float) * VT_SEM_PADDED))) return -1;
    if (!(d->norm = (float *)upload(ac->norm, sizeof(float) * VT_DIM))) return -1;
    if (!(d->time_inv_freq = (float *)upload(ac->time_inv_freq, sizeof(float) * VT_DIM / 2))) return -1;
    VT_TRY(hipMemcpy(d->h_time_inv_freq, ac->time_inv_freq, sizeof d->h_time_inv_freq, hipMemcpyDefault));
    for (int i = 0; i < TTS_HIP_AC_LAYERS; i++)
        if (upload_layer(&d->layers[i], &ac->layers[i])) return -1;
    g_vt.ac_uploaded = 1;
    g_hip.ac_layers_uploaded = TTS_HIP_AC_LAYERS;
    return 0;
}

/* ---- transfers (voxtral_tts_cuda.cu:62-86) ----------------------------------- */

extern "C" void tts_hip_to_device(void *d_dst, const void *h_src, size_t bytes) {
    (void)hipStreamSynchronize(g_vt.stream);
    (void)vt_step_poll_abort();
    (void)vt_check(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice), "tts_hip_to_device");
}

extern "C" void tts_hip_to_host(void *h_dst, const void *d_src, size_t bytes) {
    (void)hipStreamSynchronize(g_vt.stream);
    (void)vt_step_poll_abort();
    (void)vt_check(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost), "tts_hip_to_host");
}

extern "C" void tts_hip_memset(void *d_ptr, int value, size_t bytes) {
    (void)hipStreamSynchronize(g_vt.stream);
    (void)vt_step_poll_abort();
    (void)vt_check(hipMemset(d_ptr, value, bytes), "tts_hip_memset");
}

extern "C" void *tts_hip_alloc(size_t bytes) { return vt_dev_alloc(bytes); }

extern "C" void tts_hip_free_ptr(void *d_ptr) {
    if (d_ptr) (void)hipFree(d_ptr);
}

extern "C" void tts_hip_sync(void) {
    if (vt_check(hipDeviceSynchronize(), "tts_hip_sync")) return;
    (void)vt_step_poll_abort();
}

extern "C" void tts_hip_set_decode_mode(int mode) {
    if (mode != 0 && mode != 1) { vt_set_error("tts_hip_set_decode_mode: unknown schedule %d", mode); return; }
    g_vt.decode_mode = mode;
}
extern "C" void tts_hip_set_prefill_mode(int mode) {
    if (mode != 0 && mode != 1) { vt_set_error("tts_hip_set_prefill_mode: unknown schedule %d", mode); return; }
    g_vt.prefill_mode = mode;
}
extern "C" void tts_hip_set_barrier_timeout(unsigned long long ticks) { g_vt.bar_timeout = ticks; }
extern "C" void tts_hip_set_acoustic_grid(int workgroups) {
    if (workgroups < 0 || (g_vt.initialized && workgroups > g_vt.n_cu)) {
        vt_set_error("tts_hip_set_acoustic_grid: %d workgroups (0 or 1..%d)", workgroups, g_vt.n_cu);
        return;
    }
    g_vt.ac_grid = workgroups;
}
extern "C" int tts_hip_error_count(void) { return g_vt.error_count; }
extern "C" const char *tts_hip_last_error(void) { return g_vt.last_error; }
