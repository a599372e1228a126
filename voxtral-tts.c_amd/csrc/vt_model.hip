/*
 * vt_model.hip - backbone prefill and the flow-matching acoustic transformer
 * (replace tts_cuda_llm_prefill, voxtral_tts_cuda.cu:806-893, and
 * tts_cuda_predict_velocity, :1016-1100; the frame loop follows
 * voxtral_tts_acoustic.c:268-373).
 *
 * Both run on the fused weight layout of the decode path: one [6144,3072]
 * q|k|v matrix and one row-interleaved [18432,3072] gate/up matrix per layer,
 * with RoPE + cache append and SiLU*up applied by small split kernels.
 */
#include "vt_state.h"

#include <math.h>
#include <string.h>

/* gu [S,18432] with (gate, up) adjacent -> h [S,9216] = silu(gate)*up */
__global__ void vt_swiglu_pairs_kernel(const float *gu, float *h, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x) {
        const float g = gu[2 * i], u = gu[2 * i + 1];
        h[i] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
    }
}

static int blocks_for(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 4096 ? 4096 : b); }

/* One transformer layer over S rows held in x [S,3072] (in place).
 * Causal with RoPE and cache append when kc != NULL (backbone), otherwise
 * bidirectional attention inside groups of `group` rows (acoustic). */
struct vt_seq_bufs { float *xn, *qkv, *q, *att, *proj, *gu, *h; };

static void carve(vt_seq_bufs *b, float *base, int S) {
    size_t o = 0;
    b->xn = base + o;   o += (size_t)S * VT_DIM;
    b->qkv = base + o;  o += (size_t)S * VT_QKV_DIM;
    b->q = base + o;    o += (size_t)S * VT_Q_DIM;
    b->att = base + o;  o += (size_t)S * VT_Q_DIM;
    b->proj = base + o; o += (size_t)S * VT_DIM;
    b->gu = base + o;   o += (size_t)S * 2 * VT_FFN;
    b->h = base + o;
}
static size_t seq_floats(int S) {
    return (size_t)S * (2 * VT_DIM + VT_QKV_DIM + 2 * VT_Q_DIM + 2 * VT_FFN + VT_FFN);
}

static void seq_layer(const vt_layer_dev *L, float *x, const vt_seq_bufs *b, int S,
                      float *kc, float *vc, int start_pos, int group) {
    hipStream_t st = g_vt.stream;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);
    vt_launch_rms_norm(b->xn, x, L->attn_norm, S, VT_DIM, VT_EPS);
    vt_launch_linear(b->qkv, b->xn, L->wqkv, NULL, S, VT_DIM, VT_QKV_DIM);
    {
        for (int g0 = 0; g0 < S; g0 += group)
            vt_launch_attention(b->att + (size_t)g0 * VT_Q_DIM, b->qkv + (size_t)g0 * VT_QKV_DIM,
                                b->qkv + (size_t)g0 * VT_QKV_DIM + VT_Q_DIM,
                                b->qkv + (size_t)g0 * VT_QKV_DIM + VT_Q_DIM + VT_KV_DIM, group, 0, group, 0,
                                VT_HEADS, VT_KV_HEADS, VT_HEAD_DIM, scale, VT_QKV_DIM, VT_QKV_DIM);
    }
    vt_launch_linear(b->proj, b->att, L->wo, NULL, S, VT_Q_DIM, VT_DIM);
    vt_launch_add(x, b->proj, S * VT_DIM);
    vt_launch_rms_norm(b->xn, x, L->ffn_norm, S, VT_DIM, VT_EPS);
    vt_launch_linear(b->gu, b->xn, L->w13, NULL, S, VT_DIM, 2 * VT_FFN);
    hipLaunchKernelGGL(vt_swiglu_pairs_kernel, dim3(blocks_for((size_t)S * VT_FFN)), dim3(256), 0, st,
                       b->gu, b->h, (size_t)S * VT_FFN);
    vt_launch_linear(b->proj, b->h, L->w2, NULL, S, VT_FFN, VT_DIM);
    vt_launch_add(x, b->proj, S * VT_DIM);
}

/* ---- acoustic transformer --------------------------------------------------------- */

/* Host evaluation of the sinusoidal time embedding with libm, in the order of
 * voxtral_tts_acoustic.c:166-176 (bit-equal input to the time projection). */
static void time_embedding_host(float t_val, float *out) {
    const int half = VT_DIM / 2;
    for (int i = 0; i < half; i++) {
        volatile float ang = t_val * g_vt.ac.h_time_inv_freq[i];
        out[i] = cosf(ang);
        out[half + i] = sinf(ang);
    }
}

/* velocity for `branches` (1 or 2) copies of the 3-token sequence;
 * branch 0 is conditioned on d_hidden, branch 1 on a zero hidden state.
 * d_xt f32 [36], d_hidden f32 [3072], d_vel f32 [branches, 36]; asynchronous. */
static int velocity_device(float *d_vel, const float *d_xt, const float *d_hidden, float t_val,
                           int branches, float *work) {
    hipStream_t st = g_vt.stream;
    const int S = VT_AC_SEQ * branches;
    float *tok = work;                                  /* [S, 3072] */
    float *temb = tok + (size_t)S * VT_DIM;             /* [3072] */
    float *nrm = temb + VT_DIM;                         /* [3072] */
    vt_seq_bufs b;
    carve(&b, nrm + VT_DIM, S);
    float h_temb[VT_DIM];
    time_embedding_host(t_val, h_temb);
    /* staged through the pinned buffer: the copy is ordered on the stream */
    if (vt_check(hipStreamSynchronize(st), "velocity sync")) return -1;
    memcpy(g_vt.h_pin, h_temb, sizeof h_temb);
    if (vt_check(hipMemcpyAsync(temb, g_vt.h_pin, sizeof h_temb, hipMemcpyHostToDevice, st), "time emb")) return -1;
    const vt_acoustic_dev *ac = &g_vt.ac;
    vt_launch_linear(tok, d_xt, ac->input_proj, NULL, 1, VT_AC_DIM_IN, VT_DIM);
    vt_launch_linear(tok + VT_DIM, temb, ac->time_proj, NULL, 1, VT_DIM, VT_DIM);
    vt_launch_linear(tok + 2 * VT_DIM, d_hidden, ac->llm_proj, NULL, 1, VT_DIM, VT_DIM);
    if (branches == 2) {
        /* unconditional branch: same noise and time tokens, llm token = llm_proj(0) = 0 */
        if (vt_check(hipMemcpyAsync(tok + 3 * VT_DIM, tok, sizeof(float) * 2 * VT_DIM,
                                    hipMemcpyDeviceToDevice, st), "uncond tokens")) return -1;
        if (vt_check(hipMemsetAsync(tok + 5 * VT_DIM, 0, sizeof(float) * VT_DIM, st), "uncond zero")) return -1;
    }
    for (int l = 0; l < TTS_HIP_AC_LAYERS; l++)
        seq_layer(&ac->layers[l], tok, &b, S, NULL, NULL, 0, VT_AC_SEQ);
    for (int br = 0; br < branches; br++) {
        vt_launch_rms_norm(nrm, tok + (size_t)br * VT_AC_SEQ * VT_DIM, ac->norm, 1, VT_DIM, VT_EPS);
        vt_launch_linear(d_vel + br * VT_AC_DIM_IN, nrm, ac->acoustic_out, NULL, 1, VT_DIM, VT_AC_DIM_IN);
    }
    return vt_check(hipGetLastError(), "velocity launch");
}

static size_t velocity_work_floats(int branches) {
    const int S = VT_AC_SEQ * branches;
    return (size_t)S * VT_DIM + 2 * VT_DIM + seq_floats(S);
}

static int ac_ready(const char *who) {
    if (g_vt.initialized && g_vt.ac_uploaded) return 1;
    vt_set_error("%s: acoustic weights not uploaded", who);
    return 0;
}

static void predict(float *out_c, float *out_u, const float *x_t, const float *llm_hidden, float t_val) {
    const int branches = out_u ? 2 : 1;
    const size_t wf = velocity_work_floats(branches);
    float *base = (float *)vt_scratch(sizeof(float) * (wf + VT_DIM + 64 + 2 * VT_AC_DIM_IN));
    if (!base) return;
    float *d_h = base + wf, *d_xt = d_h + VT_DIM, *d_vel = d_xt + 64;
    VT_TRYV(hipMemcpy(d_h, llm_hidden, sizeof(float) * VT_DIM, hipMemcpyDefault));
    VT_TRYV(hipMemcpy(d_xt, x_t, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
    if (velocity_device(d_vel, d_xt, d_h, t_val, branches, base)) return;
    VT_TRYV(hipStreamSynchronize(g_vt.stream));
    VT_TRYV(hipMemcpy(out_c, d_vel, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
    if (out_u) VT_TRYV(hipMemcpy(out_u, d_vel + VT_AC_DIM_IN, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
}

extern "C" void tts_hip_predict_velocity(float *out_velocity, const float *x_t,
                                         const float *llm_hidden, float t_val) {
    if (!ac_ready("tts_hip_predict_velocity")) return;
    predict(out_velocity, NULL, x_t, llm_hidden, t_val);
}

extern "C" void tts_hip_predict_velocity_cfg(float *out_v_cond, float *out_v_uncond, const float *x_t,
                                             const float *llm_hidden, float t_val) {
    if (!ac_ready("tts_hip_predict_velocity_cfg")) return;
    predict(out_v_cond, out_v_uncond, x_t, llm_hidden, t_val);
}

/* ---- one audio frame ------------------------------------------------------------- */

/* First maximum of the masked semantic logits (voxtral_tts_acoustic.c:291-306):
 * index 0 and indices >= 8194 are forced to -1e30; ties keep the lowest index. */
__global__ void __launch_bounds__(1024) vt_semantic_argmax_kernel(const float *logits, int *out_code) {
    __shared__ float sv[1024];
    __shared__ int si[1024];
    float best = -1e30f;              /* value of the masked slot 0 */
    int bi = 0;
    for (int i = (int)threadIdx.x; i < VT_SEM_PADDED; i += (int)blockDim.x) {
        const float v = (i == 0 || i >= VT_SEM_VALID_END) ? -1e30f : logits[i];
        if (v > best) { best = v; bi = i; }          /* ascending i per thread: first max kept */
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = (int)blockDim.x / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            const float v = sv[threadIdx.x + s];
            const int j = si[threadIdx.x + s];
            if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && j < si[threadIdx.x])) {
                sv[threadIdx.x] = v;
                si[threadIdx.x] = j;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) *out_code = si[0];
}

/* x += (1.2*vc + (1-1.2)*vu) * dt, products rounded separately as on the CPU
 * (voxtral_tts_acoustic.c:350-354) */
__global__ void vt_euler_cfg_kernel(float *x, const float *vel, float dt) {
    const int i = (int)threadIdx.x;
    if (i < VT_AC_DIM_IN) {
        const float a = __fmul_rn(1.2f, vel[i]);
        const float b = __fmul_rn(1.0f - 1.2f, vel[VT_AC_DIM_IN + i]);
        x[i] = __fadd_rn(x[i], __fmul_rn(__fadd_rn(a, b), dt));
    }
}

/* FSQ quantisation (voxtral_tts_acoustic.c:358-372) */
__global__ void vt_fsq_kernel(const float *x, int *codes) {
    const int i = (int)threadIdx.x;
    if (i < VT_AC_DIM_IN) {
        float v = x[i];
        if (v > 1.0f) v = 1.0f;
        if (v < -1.0f) v = -1.0f;
        const float scaled = __fmul_rn(__fdiv_rn(__fadd_rn(v, 1.0f), 2.0f), 20.0f);
        int c = (int)__fadd_rn(scaled, 0.5f);
        if (c < 0) c = 0;
        if (c > 20) c = 20;
        codes[i + 1] = c + 2;
    }
}

extern "C" void tts_hip_acoustic_frame(int *out_codes, const float *llm_hidden, const float *x0,
                                       float *out_x) {
    if (!ac_ready("tts_hip_acoustic_frame")) return;
    hipStream_t st = g_vt.stream;
    const size_t wf = velocity_work_floats(2);
    float *base = (float *)vt_scratch(sizeof(float) * (wf + VT_DIM + 64 + 128 + VT_SEM_PADDED + 64));
    if (!base) return;
    float *d_h = base + wf, *d_x = d_h + VT_DIM, *d_vel = d_x + 64, *d_logits = d_vel + 128;
    int *d_codes = (int *)(d_logits + VT_SEM_PADDED);
    const vt_acoustic_dev *ac = &g_vt.ac;
    VT_TRYV(hipMemcpy(d_h, llm_hidden, sizeof(float) * VT_DIM, hipMemcpyDefault));
    VT_TRYV(hipMemcpy(d_x, x0, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
    vt_launch_linear(d_logits, d_h, ac->semantic_out, ac->semantic_bias, 1, VT_DIM, VT_SEM_PADDED);
    hipLaunchKernelGGL(vt_semantic_argmax_kernel, dim3(1), dim3(1024), 0, st, d_logits, d_codes);
    int code0 = -1;
    VT_TRYV(hipMemcpyAsync(&code0, d_codes, sizeof(int), hipMemcpyDeviceToHost, st));
    VT_TRYV(hipStreamSynchronize(st));
    out_codes[0] = code0;
    if (code0 == 1) {                                   /* END_AUDIO */
        for (int i = 1; i < 37; i++) out_codes[i] = 2;
        if (out_x) memset(out_x, 0, sizeof(float) * VT_AC_DIM_IN);
        return;
    }
    float ts[8];
    for (int i = 0; i < 8; i++) ts[i] = (float)i / (float)7;
    for (int s = 0; s < 7; s++) {
        volatile float dt = ts[s + 1] - ts[s];
        if (velocity_device(d_vel, d_x, d_h, ts[s], 2, base)) return;
        hipLaunchKernelGGL(vt_euler_cfg_kernel, dim3(1), dim3(64), 0, st, d_x, d_vel, (float)dt);
    }
    hipLaunchKernelGGL(vt_fsq_kernel, dim3(1), dim3(64), 0, st, d_x, d_codes);
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    VT_TRYV(hipMemcpy(out_codes + 1, d_codes + 1, sizeof(int) * VT_AC_DIM_IN, hipMemcpyDeviceToHost));
    if (out_x) VT_TRYV(hipMemcpy(out_x, d_x, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDeviceToHost));
}
