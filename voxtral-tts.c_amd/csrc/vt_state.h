/*
 * vt_state.h - host-side state of the backend (one global context, as in the
 * reference backend: voxtral_tts_cuda.cu:56) and the helpers shared by the
 * translation units of the library.
 */
#ifndef VT_STATE_H
#define VT_STATE_H

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/voxtral_tts_hip.h"
#include "vt_decode_phases.h"

#define VT_MAX_WAVES 8
#define VT_STEP_THREADS 512
#define VT_AC_SEQ 3
#define VT_AC_DIM_IN 36
#define VT_SEM_PADDED 8320
#define VT_SEM_VALID_END 8194     /* 2 special + 8192 codes */

/* Second copy of a backbone layer's four matrices, in the order the 128 x 256 tile product reads them
 * (vt_launch_frag_layout); the decode step streams the row-major copy. */
struct vt_layer_frag { uint16_t *wqkv, *wo, *w13, *w2; };

struct vt_acoustic_dev {
    vt_layer_dev layers[TTS_HIP_AC_LAYERS];
    uint16_t *input_proj, *time_proj, *llm_proj, *semantic_out, *acoustic_out;
    float *semantic_bias;         /* NULL when the checkpoint has none */
    float *norm;
    float *time_inv_freq;
    float h_time_inv_freq[VT_DIM / 2];
    float *time_tok;              /* [8, 3072]: projected time tokens of the Euler grid, then the last LLM token */
    int time_tok_ready;
    uint16_t *audio_emb;          /* [audio_rows, 3072] audio-code embedding table */
    int *audio_offsets;           /* [37] first row of every codebook, then 37 ints of staging for codes */
    int audio_rows;
};

struct vt_state {
    int initialized;
    int device;
    int n_cu;
    int ac_grid;                  /* workgroups of the acoustic product kernels; 0 = n_cu */
    int grid;                     /* workgroups of the persistent kernels */
    size_t step_dyn_lds;          /* dynamic LDS that pins one workgroup per CU */
    int step_checked, step_fits;  /* residency of the whole-step kernel's grid, asked once per context */
    int step_pending;             /* a whole-step kernel was launched and its abort flag not yet looked at */
    hipStream_t stream;
    hipEvent_t ev0, ev1;
    int decode_mode;
    int prefill_mode;             /* 0 = one launch per product and row pass, 1 = one persistent launch per layer behind the attention */

    /* backbone weights */
    vt_layer_dev h_layers[TTS_HIP_DEC_LAYERS];
    vt_layer_frag h_frag[TTS_HIP_DEC_LAYERS];   /* the same matrices in the fragment order of the prefill product */
    vt_layer_dev *d_layers;
    float *d_dec_norm;
    uint16_t *d_tok_emb;
    int n_dec_layers;

    /* acoustic weights */
    vt_acoustic_dev ac;
    int ac_uploaded;

    /* caches and tables */
    float *d_rope;                /* [kv_max, 64, 2] */
    int kv_max;

    /* decode work buffers */
    float *d_x, *d_q, *d_attn, *d_h, *d_att_part, *d_embed, *d_hidden;
    unsigned int *d_att_cnt;
    unsigned int *d_bar_flags;    /* one flag per workgroup of the persistent kernel */
    unsigned int bar_epoch;       /* last barrier epoch handed to a launch */
    unsigned long long bar_timeout; /* spin budget of a barrier in 100 MHz ticks; 0 = default */
    int *d_abort;
    uint16_t *d_dummy;            /* small resident block requested in place of a layer beyond the last */
    float *h_pin;                 /* pinned staging: [3072 in][3072 out + flag] */

    /* generic scratch (prefill / acoustic / linear) */
    void *d_scratch;
    size_t scratch_bytes;
    void *d_kv_img;               /* prefill attention: tile images of one layer's K and V */
    size_t kv_img_bytes;

    int error_count;
    char last_error[512];
};

extern vt_state g_vt;

void vt_set_error(const char *fmt, ...);
int vt_check(hipError_t e, const char *what);
void *vt_scratch(size_t bytes);      /* grows on demand; contents undefined */
void *vt_dev_alloc(size_t bytes);

#define VT_TRY(call) do { if (vt_check((call), #call)) return -1; } while (0)
#define VT_TRYV(call) do { if (vt_check((call), #call)) return; } while (0)

/* kernels launched from other translation units */
void vt_launch_linear(float *d_y, const float *d_x, const uint16_t *d_W, const float *d_bias,
                      int seq_len, int in_dim, int out_dim);
void vt_launch_rms_norm(float *d_out, const float *d_x, const float *d_w, int seq, int dim, float eps);
void vt_launch_attention(float *d_out, const float *d_Q, const float *d_K, const float *d_V,
                         int seq_q, int q_offset, int seq_k, int causal, int n_heads,
                         int n_kv_heads, int head_dim, float scale, int kv_stride, int q_stride);
void vt_launch_add(float *d_a, const float *d_b, int n);
void vt_launch_prefill_attention(float *d_out, uint16_t *d_hi, uint16_t *d_lo, const float *d_Q,
                                 int q_stride, const float *d_K, const float *d_V, int S, int start_pos,
                                 float scale);
/* the model's attention scale, 1/sqrt(head_dim), computed like the CPU path does (voxtral_tts_llm.c:189) */
#define VT_ATT_SCALE (1.0f / sqrtf((float)VT_HEAD_DIM))
void vt_codec_free(void);
/* single launches for the library's other translation units and its benchmark companion (vt_bench.hip) */
int vt_codec_probe_buffers(float **xn, float **att, float **h, int **codes);
int vt_codec_probe_launch(int which);
int vt_ac_launch_layer_phase(int layer, int phase);
float *vt_ac_work_area(size_t *n_floats);
int vt_prefill_cuts(int tiles, int most);
unsigned char *vt_pa_image(int rows);
void vt_pa_launch_image(unsigned char *d_img, const float *d_qkv, int planes, size_t plane_stride, float *d_K,
                        float *d_V, int S, int start_pos);
void vt_launch_prefill_attention_raw(float *d_out, uint16_t *d_hi, uint16_t *d_lo, const float *d_Q,
                                     int q_stride, int q_planes, size_t q_plane_stride, const float *d_rope,
                                     const unsigned char *d_img, int S, int start_pos, float scale);
#ifndef VT_W13_TAIL_CUT
#define VT_W13_TAIL_CUT 4
#endif
int vt_step_resident(void);
int vt_step_poll_abort(void);
int vt_step_poll_abort_now(void);
int vt_run_step(const vt_layer_dev *d_layers, int n_layers, int first_layer,
                const float *d_final_norm, const float *d_in, float *d_out, int pos);

#endif /* VT_STATE_H */
