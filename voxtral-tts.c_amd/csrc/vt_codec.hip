/*
 * vt_codec.hip - audio codec decoder on the device: frames of 37 codes -> 24 kHz waveform
 * (tts_codec_decode, voxtral_tts_codec.c:389-503; one transformer layer :306-383; the
 * convolutions voxtral_tts_kernels.c:217-327; ALiBi sliding-window attention :527-596).
 *
 * Layout: activations are token-major [T, C] from the first kernel to the last, so the
 * reference's channel-first transposes around every convolution disappear and the last
 * product writes the waveform ([T, 240] row-major is the sample order).  Weights stay fp32
 * as in the reference and are re-laid once at upload:
 *   - q|k|v and gate|up are stacked into one [3072, 1024] and one [8192, 1024] matrix;
 *   - a causal conv1d (stride 1, taps K) becomes a product over the K shifted copies of the
 *     input: W'[oc][k * C_in + ic] = w[oc][ic][k], rows and K padded with zeros;
 *   - the transposed conv (taps 4, stride 2) becomes ONE product that writes both output
 *     phases: out[2j+p][oc] = sum_ic x[j][ic] w[ic][oc][p] + x[j-1][ic] w[ic][oc][p+2], i.e.
 *     W'[p * 1024 + oc][q * 1024 + ic] = w[ic][oc][p + 2q] against rows [x[j] | x[j-1]], and
 *     the [L, 2048] result IS the [2L, 1024] upsampled sequence.
 * Every product runs on the fp32 matrix cores (v_mfma_f32_32x32x2f32: fp32 operands, fp32
 * accumulation, MFMA-bound at 157 TFLOP/s); K is cut where a launch would not fill the chip
 * and the partial planes are summed in a fixed order by the row kernel that follows, which
 * also applies bias / layer scale / residual and the next RMSNorm.
 */
#include "vt_state.h"
#include "vt_gemm.h"

#include <stdlib.h>
#include <string.h>

#define CD_DIM 1024
#define CD_HID 4096
#define CD_HEADS 8
#define CD_HEAD_DIM 128
#define CD_EPS 1e-2f
#define CD_QK_EPS 1e-6f
#define CD_EMBED 292
#define CD_SEM_DIM 256
#define CD_SEM_SIZE 8192
#define CD_PATCH 240
#define CD_LAYERS 8
#define CD_IN_TAPS 3
#define CD_OUT_TAPS 7
#define CD_IN_K 896           /* 3 * 292 = 876 padded to a multiple of 32 */
#define CD_OUT_K (CD_OUT_TAPS * CD_DIM)
#define CD_OUT_N 256          /* 240 padded to a multiple of 128 */
#define CD_MAX_SPLIT 8

/* ---- fp32 product C[M, N] = A[M, K] W[N, K]^T on the matrix cores ----------------------
 * 128 x 128 tile per workgroup, 4 waves in 2 x 2, each 64 x 64 = 2 x 2 MFMA tiles of 32 x 32,
 * K in steps of 32 through LDS (row pitch 36 floats: 16-byte reads of 32 consecutive rows fall
 * on distinct banks).  A lane of the 32x32x2 instruction feeds row (lane % 32) at k = lane / 32;
 * here the four instructions of a k-group of 8 take k = 4 * (lane / 32) + j, so that a lane
 * fetches its four k values with one 16-byte LDS read (the order of k inside a sum is free as
 * long as both operands use the same one).  blockIdx.z cuts K; plane z of C is written at
 * C + z * plane_stride.  Rows of A beyond M are read from row M - 1 and never stored; W has
 * N rounded up to 128 rows; K % (32 * gridDim.z) == 0. */
#define CG_BM 128
#define CG_BN 128
#define CG_BK 32
#define CG_PITCH 36
#ifndef CG_W64
#define CG_W64 2            /* waves per SIMD the 64-row kernel is compiled for */
#endif

typedef float cd_f16v __attribute__((ext_vector_type(16)));

template <int BM>
__device__ __forceinline__ void cd_gemm_tile(float *__restrict__ C, const float *__restrict__ A, const float *__restrict__ W,
                                             int M, int N, int K, int lda, int ldc, size_t plane_stride) {
    constexpr int MI = BM / 64;              /* 32-row blocks per wave */
    constexpr int AP = BM / 32;              /* staging passes of the activation tile */
    __shared__ float As[BM * CG_PITCH];
    __shared__ float Ws[CG_BN * CG_PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * CG_BN;
    const int kper = K / gridDim.z, kbeg = blockIdx.z * kper;

    /* staging: 4 passes of 32 rows for each operand, 16 bytes per thread and pass */
    const int lr = tid >> 3, lc = (tid & 7) * 4;
    const float *ap[AP], *wp[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        if (p < AP) {
            int am = m0 + p * 32 + lr;
            am = am < M ? am : M - 1;
            ap[p] = A + (size_t)am * lda + kbeg + lc;
        }
        wp[p] = W + (size_t)(n0 + p * 32 + lr) * K + kbeg + lc;
    }
    f32x4 ra[AP], rw[4];      /* clang vectors: HIP's float4 structs in an array end up in LDS, not registers */
#pragma unroll
    for (int p = 0; p < 4; p++) { if (p < AP) ra[p] = *(const f32x4 *)ap[p]; rw[p] = *(const f32x4 *)wp[p]; }

    cd_f16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int fr = lane & 31, fk = (lane >> 5) * 4;
    for (int k0 = 0; k0 < kper; k0 += CG_BK) {
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 4; p++) {
            if (p < AP) *(f32x4 *)&As[(p * 32 + lr) * CG_PITCH + lc] = ra[p];
            *(f32x4 *)&Ws[(p * 32 + lr) * CG_PITCH + lc] = rw[p];
        }
        __syncthreads();
        {
            /* the next K step is requested without a condition (the last step asks for its own
             * tile again, out of the L2): behind a conditional request the compiler parks the
             * registers in LDS and waits for the loads before the products instead of after */
            const int kn = k0 + CG_BK < kper ? k0 + CG_BK : k0;
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (p < AP) ra[p] = *(const f32x4 *)(ap[p] + kn);
                rw[p] = *(const f32x4 *)(wp[p] + kn);
            }
            __builtin_amdgcn_sched_barrier(0);          /* requests first, products behind them */
        }
#pragma unroll
        for (int kg = 0; kg < CG_BK; kg += 8) {
            f32x4 fa[MI], fw[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                if (i < MI) fa[i] = *(const f32x4 *)&As[(wm * (BM / 2) + i * 32 + fr) * CG_PITCH + kg + fk];
                fw[i] = *(const f32x4 *)&Ws[(wn * 64 + i * 32 + fr) * CG_PITCH + kg + fk];
            }
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].x, fw[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].y, fw[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].z, fw[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].w, fw[j].w, acc[i][j], 0, 0, 0);
                }
        }
    }
    /* accumulator element v of a lane: column lane % 32, row 8 * (v / 4) + 4 * (lane / 32) + v % 4 */
    float *Cp = C + (size_t)blockIdx.z * plane_stride;
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m < M && n < N) Cp[(size_t)m * ldc + n] = acc[i][j][v];
            }
        }
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2)))
vt_codec_gemm_kernel(float *__restrict__ C, const float *__restrict__ A, const float *__restrict__ W,
                     int M, int N, int K, int lda, int ldc, size_t plane_stride) {
    cd_gemm_tile<CG_BM>(C, A, W, M, N, K, lda, ldc, plane_stride);
}

/* The same product on 64 x 128 tiles (a wave owns 32 x 64): for row counts that 128-row tiles fit badly
 * (1600 rows are 25 tiles of 64 but 12.5 of 128) and for launches whose 128-row tiles leave the last
 * round of workgroups half empty. */
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, CG_W64)))
vt_codec_gemm64_kernel(float *__restrict__ C, const float *__restrict__ A, const float *__restrict__ W,
                       int M, int N, int K, int lda, int ldc, size_t plane_stride) {
    cd_gemm_tile<64>(C, A, W, M, N, K, lda, ldc, plane_stride);
}

/* ---- row kernels ------------------------------------------------------------------------- */

/* block-wide sum over 256 threads (4 waves), the same value in every thread */
__device__ __forceinline__ float cd_block_sum(float v, float *red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

/* One row of 1024: val = sum of the planes (+ bias) (* scale) (+ residual) -> x_out; with a
 * norm weight also xn_out = val * rsqrt(mean(val^2) + eps) * norm_w (tts_rms_norm,
 * voxtral_tts_kernels.c:333-349).  planes == NULL passes x_in through (norm only). */
__global__ void __launch_bounds__(256)
vt_codec_row_kernel(float *x_out, float *__restrict__ xn_out, const float *x_in,
                    const float *__restrict__ planes, int splits, size_t plane_stride, int ldp,
                    const float *__restrict__ bias, const float *__restrict__ scale,
                    const float *__restrict__ norm_w, float eps) {
    __shared__ float red[4];
    const int row = blockIdx.x, c = threadIdx.x * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (planes) {
        for (int s = 0; s < splits; s++) {
            const float4 p = *(const float4 *)(planes + s * plane_stride + (size_t)row * ldp + c);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        if (bias) { const float4 b = *(const float4 *)(bias + c); v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w; }
        if (scale) { const float4 g = *(const float4 *)(scale + c); v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w; }
    }
    if (x_in) { const float4 r = *(const float4 *)(x_in + (size_t)row * CD_DIM + c); v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w; }
    if (x_out) *(float4 *)(x_out + (size_t)row * CD_DIM + c) = v;
    if (norm_w) {
        const float ss = cd_block_sum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w, red);
        const float inv = 1.0f / sqrtf(ss / (float)CD_DIM + eps);
        const float4 w = *(const float4 *)(norm_w + c);
        *(float4 *)(xn_out + (size_t)row * CD_DIM + c) = make_float4(v.x * inv * w.x, v.y * inv * w.y, v.z * inv * w.z, v.w * inv * w.w);
    }
}

/* q|k|v planes [T, 3072] -> summed, with the RMSNorm over the whole 1024-wide q row and k row
 * (tts_qk_norm, voxtral_tts_kernels.c:351-355, eps 1e-6) when the layer has those weights. */
__global__ void __launch_bounds__(256)
vt_codec_qkv_kernel(float *__restrict__ qkv, const float *__restrict__ planes, int splits, size_t plane_stride,
                    const float *__restrict__ q_norm, const float *__restrict__ k_norm) {
    __shared__ float red[4];
    const int row = blockIdx.x, c = threadIdx.x * 4;
    for (int part = 0; part < 3; part++) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        const size_t off = (size_t)row * (3 * CD_DIM) + part * CD_DIM + c;
        for (int s = 0; s < splits; s++) {
            const float4 p = *(const float4 *)(planes + s * plane_stride + off);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        const float *nw = part == 0 ? q_norm : part == 1 ? k_norm : nullptr;
        if (nw) {
            const float ss = cd_block_sum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w, red);
            const float inv = 1.0f / sqrtf(ss / (float)CD_DIM + CD_QK_EPS);
            const float4 w = *(const float4 *)(nw + c);
            v = make_float4(v.x * inv * w.x, v.y * inv * w.y, v.z * inv * w.z, v.w * inv * w.w);
        }
        *(float4 *)(qkv + off) = v;
    }
}

/* gate|up planes [T, 8192] -> h = silu(gate) * up [T, 4096] (tts_silu, tts_mul_inplace) */
__global__ void __launch_bounds__(256)
vt_codec_swiglu_kernel(float *__restrict__ h, const float *__restrict__ gu, int splits, size_t plane_stride, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t row = i / CD_HID, col = i % CD_HID;
        float g = 0.f, u = 0.f;
        for (int s = 0; s < splits; s++) {
            g += gu[s * plane_stride + row * (2 * CD_HID) + col];
            u += gu[s * plane_stride + row * (2 * CD_HID) + CD_HID + col];
        }
        h[i] = g / (1.0f + expf(-g)) * u;
    }
}

/* ALiBi causal sliding-window attention: one wave per (token, head), the online softmax over
 * the at most `window` keys in the reference's order (voxtral_tts_kernels.c:527-596). */
__global__ void __launch_bounds__(256)
vt_codec_attention_kernel(float *__restrict__ out, const float *__restrict__ qkv, int T, int window,
                          const float *__restrict__ slopes, float scale) {
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (unit >= T * CD_HEADS) return;
    const int i = unit / CD_HEADS, h = unit % CD_HEADS;
    const float slope = slopes[h];
    const float2 q = *(const float2 *)(qkv + (size_t)i * (3 * CD_DIM) + h * CD_HEAD_DIM + lane * 2);
    const int j0 = (window > 0 && i - window + 1 > 0) ? i - window + 1 : 0;
    float mx = -1e30f, se = 0.f;
    float2 o = make_float2(0.f, 0.f);
    for (int j = j0; j <= i; j++) {
        const float *kr = qkv + (size_t)j * (3 * CD_DIM) + CD_DIM + h * CD_HEAD_DIM + lane * 2;
        const float2 k = *(const float2 *)kr, v = *(const float2 *)(kr + CD_DIM);
        float sc = q.x * k.x + q.y * k.y;
        for (int s = 32; s > 0; s >>= 1) sc += __shfl_xor(sc, s);
        sc = sc * scale + slope * (float)(j - i);
        if (sc > mx) {
            const float c = expf(mx - sc);
            se = se * c + 1.0f;
            o.x = o.x * c + v.x; o.y = o.y * c + v.y;
            mx = sc;
        } else {
            const float w = expf(sc - mx);
            se += w;
            o.x += w * v.x; o.y += w * v.y;
        }
    }
    const float inv = se > 0.f ? 1.0f / se : 1.0f;
    *(float2 *)(out + (size_t)i * CD_DIM + h * CD_HEAD_DIM + lane * 2) = make_float2(o.x * inv, o.y * inv);
}

/* codes [T, 37] -> the three shifted copies of the 292-wide embedding that the input
 * convolution multiplies (embed_codes, voxtral_tts_codec.c:276-300; causal padding with
 * left reflection, voxtral_tts_kernels.c:217-272): a[t][k * 292 + c] = e[src(t, k)][c],
 * src = t + k - 2, reflected to -src when negative, zero when that is outside too. */
__global__ void __launch_bounds__(256)
vt_codec_embed_kernel(float *__restrict__ a, const int *__restrict__ codes, const float *__restrict__ sem, int T) {
    const int t = blockIdx.x;
    for (int idx = threadIdx.x; idx < CD_IN_K; idx += 256) {
        float val = 0.f;
        if (idx < CD_IN_TAPS * CD_EMBED) {
            const int k = idx / CD_EMBED, c = idx % CD_EMBED;
            int src = t + k - (CD_IN_TAPS - 1);
            if (src < 0) src = -src;
            if (src < T) {
                const int *fc = codes + (size_t)src * 37;
                if (c < CD_SEM_DIM) {
                    int s = fc[0] - 2;
                    s = s < 0 ? 0 : s >= CD_SEM_SIZE ? CD_SEM_SIZE - 1 : s;
                    val = sem[(size_t)s * CD_SEM_DIM + c];
                } else {
                    int q = fc[c - CD_SEM_DIM + 1] - 2;
                    q = q < 0 ? 0 : q > 20 ? 20 : q;
                    val = (float)q * 2.0f / 20.0f - 1.0f;
                }
            }
        }
        a[(size_t)t * CD_IN_K + idx] = val;
    }
}

/* x [T, 1024] -> a[t][k * 1024 + c] = x[src(t, k)][c] for `taps` causal taps (stride 1, left
 * reflection as above): the operand of the output convolution. */
__global__ void __launch_bounds__(256)
vt_codec_taps_kernel(float *__restrict__ a, const float *__restrict__ x, int T, int taps) {
    const int t = blockIdx.x, c = threadIdx.x * 4;
    for (int k = 0; k < taps; k++) {
        int src = t + k - (taps - 1);
        if (src < 0) src = -src;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (src < T) v = *(const float4 *)(x + (size_t)src * CD_DIM + c);
        *(float4 *)(a + ((size_t)t * taps + k) * CD_DIM + c) = v;
    }
}

/* x [L, 1024] -> a[j] = [x[j] | x[j-1]] (zero before the start): the operand of the
 * transposed convolution (voxtral_tts_kernels.c:274-327 with taps 4, stride 2). */
__global__ void __launch_bounds__(256)
vt_codec_pair_kernel(float *__restrict__ a, const float *__restrict__ x, int L) {
    const int j = blockIdx.x, c = threadIdx.x * 4;
    *(float4 *)(a + (size_t)j * 2 * CD_DIM + c) = *(const float4 *)(x + (size_t)j * CD_DIM + c);
    float4 p = make_float4(0.f, 0.f, 0.f, 0.f);
    if (j > 0) p = *(const float4 *)(x + (size_t)(j - 1) * CD_DIM + c);
    *(float4 *)(a + (size_t)j * 2 * CD_DIM + CD_DIM + c) = p;
}

/* waveform: planes [T, 240 of ldp] summed + bias */
__global__ void __launch_bounds__(256)
vt_codec_wave_kernel(float *__restrict__ out, const float *__restrict__ planes, int splits, size_t plane_stride,
                     int ldp, const float *__restrict__ bias, int T) {
    const int t = blockIdx.x, c = threadIdx.x;
    if (c >= CD_PATCH) return;
    float v = 0.f;
    for (int s = 0; s < splits; s++) v += planes[s * plane_stride + (size_t)t * ldp + c];
    out[(size_t)t * CD_PATCH + c] = v + (bias ? bias[c] : 0.f);
}

/* ---- device state -------------------------------------------------------------------------- */

struct cd_layer_dev {
    float *wqkv, *wo, *w13, *w2;
    float *q_norm, *k_norm, *attention_norm, *ffn_norm, *attn_scale, *ffn_scale;
    int window;
};

static struct {
    int uploaded;
    float *sem;                   /* [8192, 256] */
    float *slopes;                /* [8] */
    float *w_in, *b_in;           /* [1024, 896] */
    cd_layer_dev layers[CD_LAYERS];
    float *w_up[3], *b_up[3];     /* [2048, 2048]; bias doubled to [2048] */
    float *w_out, *b_out;         /* [256, 7168] */
    /* work buffers for up to cap_frames frames */
    int cap_frames;
    float *x, *xn, *qkv, *att, *h, *wide, *part, *wave;
    int *codes;
} g_cd;

static void cd_free_ptr(float **p) { if (*p) (void)hipFree(*p); *p = NULL; }

void vt_codec_free(void) {
    cd_free_ptr(&g_cd.sem); cd_free_ptr(&g_cd.slopes); cd_free_ptr(&g_cd.w_in); cd_free_ptr(&g_cd.b_in);
    for (int i = 0; i < CD_LAYERS; i++) {
        cd_layer_dev *l = &g_cd.layers[i];
        float **ps[] = {&l->wqkv, &l->wo, &l->w13, &l->w2, &l->q_norm, &l->k_norm, &l->attention_norm,
                        &l->ffn_norm, &l->attn_scale, &l->ffn_scale};
        for (size_t k = 0; k < sizeof ps / sizeof ps[0]; k++) cd_free_ptr(ps[k]);
    }
    for (int i = 0; i < 3; i++) { cd_free_ptr(&g_cd.w_up[i]); cd_free_ptr(&g_cd.b_up[i]); }
    cd_free_ptr(&g_cd.w_out); cd_free_ptr(&g_cd.b_out);
    float **ws[] = {&g_cd.x, &g_cd.xn, &g_cd.qkv, &g_cd.att, &g_cd.h, &g_cd.wide, &g_cd.part, &g_cd.wave};
    for (size_t k = 0; k < sizeof ws / sizeof ws[0]; k++) cd_free_ptr(ws[k]);
    if (g_cd.codes) (void)hipFree(g_cd.codes);
    memset(&g_cd, 0, sizeof g_cd);
}

static float *cd_upload(const float *src, size_t n) {
    float *d = (float *)vt_dev_alloc(n * sizeof(float));
    if (d && vt_check(hipMemcpy(d, src, n * sizeof(float), hipMemcpyDefault), "codec weight copy")) {
        (void)hipFree(d);
        return NULL;
    }
    return d;
}

/* host copy of a tensor that may live on the host or the device (caller frees) */
static float *cd_host(const float *src, size_t n) {
    float *h = (float *)malloc(n * sizeof(float));
    if (h && vt_check(hipMemcpy(h, src, n * sizeof(float), hipMemcpyDefault), "codec weight read")) { free(h); return NULL; }
    return h;
}

/* stack of row blocks [rows_i, cols] -> one device matrix */
static float *cd_upload_stack(const float *const *srcs, const int *rows, int n, int cols) {
    size_t total = 0;
    for (int i = 0; i < n; i++) total += (size_t)rows[i] * cols;
    float *d = (float *)vt_dev_alloc(total * sizeof(float));
    size_t off = 0;
    for (int i = 0; d && i < n; i++) {
        if (vt_check(hipMemcpy(d + off, srcs[i], (size_t)rows[i] * cols * sizeof(float), hipMemcpyDefault), "codec weight copy")) {
            (void)hipFree(d);
            return NULL;
        }
        off += (size_t)rows[i] * cols;
    }
    return d;
}

/* conv1d weight [out_ch, in_ch, taps] -> [n_pad, k_pad] with k = tap * in_ch + ic */
static float *cd_upload_conv(const tts_hip_host_conv_t *cv, int n_pad, int k_pad) {
    const size_t n = (size_t)cv->out_ch * cv->in_ch * cv->kernel;
    float *h = cd_host(cv->weight, n);
    float *r = (float *)calloc((size_t)n_pad * k_pad, sizeof(float));
    float *d = NULL;
    if (h && r) {
        for (int oc = 0; oc < cv->out_ch; oc++)
            for (int ic = 0; ic < cv->in_ch; ic++)
                for (int k = 0; k < cv->kernel; k++)
                    r[(size_t)oc * k_pad + (size_t)k * cv->in_ch + ic] = h[((size_t)oc * cv->in_ch + ic) * cv->kernel + k];
        d = cd_upload(r, (size_t)n_pad * k_pad);
    } else {
        vt_set_error("codec upload: out of host memory");
    }
    free(h); free(r);
    return d;
}

/* transposed conv weight [in_ch, out_ch, 4] -> [2 * 1024, 2 * 1024]: row p * 1024 + oc, column
 * q * 1024 + ic holds w[ic][oc][p + 2q] */
static float *cd_upload_convt(const tts_hip_host_conv_t *cv) {
    const size_t n = (size_t)CD_DIM * CD_DIM * 4;
    float *h = cd_host(cv->weight, n);
    float *r = (float *)malloc(n * sizeof(float));
    float *d = NULL;
    if (h && r) {
        for (int ic = 0; ic < CD_DIM; ic++)
            for (int oc = 0; oc < CD_DIM; oc++)
                for (int k = 0; k < 4; k++) {
                    const int p = k & 1, q = k >> 1;
                    r[((size_t)p * CD_DIM + oc) * (2 * CD_DIM) + (size_t)q * CD_DIM + ic] = h[((size_t)ic * CD_DIM + oc) * 4 + k];
                }
        d = cd_upload(r, n);
    } else {
        vt_set_error("codec upload: out of host memory");
    }
    free(h); free(r);
    return d;
}

static float *cd_upload_bias(const float *bias, int n, int n_pad, int repeat) {
    if (!bias) return NULL;
    float *h = cd_host(bias, n);
    float *r = (float *)calloc((size_t)n_pad * repeat, sizeof(float));
    float *d = NULL;
    if (h && r) {
        for (int k = 0; k < repeat; k++) memcpy(r + (size_t)k * n_pad, h, n * sizeof(float));
        d = cd_upload(r, (size_t)n_pad * repeat);
    }
    free(h); free(r);
    return d;
}

static int cd_conv_is(const tts_hip_host_conv_t *cv, int in_ch, int out_ch, int kernel, int stride, int tr) {
    return cv->weight && cv->in_ch == in_ch && cv->out_ch == out_ch && cv->kernel == kernel &&
           cv->stride == stride && !cv->is_transpose == !tr;
}

extern "C" int tts_hip_upload_codec_weights(void *codec_ptr) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_upload_codec_weights: backend not initialised"); return -1; }
    const tts_hip_host_codec_t *c = (const tts_hip_host_codec_t *)codec_ptr;
    if (!c || !c->semantic_embedding) { vt_set_error("tts_hip_upload_codec_weights: NULL codec"); return -1; }
    if (!cd_conv_is(&c->input_conv, CD_EMBED, CD_DIM, CD_IN_TAPS, 1, 0) ||
        !cd_conv_is(&c->output_proj, CD_DIM, CD_PATCH, CD_OUT_TAPS, 1, 0)) {
        vt_set_error("tts_hip_upload_codec_weights: input / output convolution is not 292->1024 k3 s1 / 1024->240 k7 s1");
        return -1;
    }
    for (int i = 0; i < 3; i++)
        if (!cd_conv_is(&c->stage_convs[i], CD_DIM, CD_DIM, 4, 2, 1)) {
            vt_set_error("tts_hip_upload_codec_weights: upsampling convolution %d is not transposed 1024->1024 k4 s2", i);
            return -1;
        }
    (void)hipDeviceSynchronize();
    vt_codec_free();
    int ok = 1;
    ok &= (g_cd.sem = cd_upload(c->semantic_embedding, (size_t)CD_SEM_SIZE * CD_SEM_DIM)) != NULL;
    ok &= (g_cd.slopes = cd_upload(c->alibi_slopes, CD_HEADS)) != NULL;
    ok &= (g_cd.w_in = cd_upload_conv(&c->input_conv, CD_DIM, CD_IN_K)) != NULL;
    g_cd.b_in = cd_upload_bias(c->input_conv.bias, CD_DIM, CD_DIM, 1);
    ok &= (g_cd.w_out = cd_upload_conv(&c->output_proj, CD_OUT_N, CD_OUT_K)) != NULL;
    g_cd.b_out = cd_upload_bias(c->output_proj.bias, CD_PATCH, CD_OUT_N, 1);
    for (int i = 0; ok && i < 3; i++) {
        ok &= (g_cd.w_up[i] = cd_upload_convt(&c->stage_convs[i])) != NULL;
        g_cd.b_up[i] = cd_upload_bias(c->stage_convs[i].bias, CD_DIM, CD_DIM, 1);
    }
    for (int i = 0; ok && i < CD_LAYERS; i++) {
        const tts_hip_host_codec_layer_t *s = &c->transformers[i];
        cd_layer_dev *l = &g_cd.layers[i];
        if (!s->wq || !s->wk || !s->wv || !s->wo || !s->w1 || !s->w2 || !s->w3 || !s->attention_norm || !s->ffn_norm) {
            vt_set_error("tts_hip_upload_codec_weights: layer %d has a NULL tensor", i);
            ok = 0;
            break;
        }
        const float *qkv[3] = {s->wq, s->wk, s->wv};
        const int r3[3] = {CD_DIM, CD_DIM, CD_DIM};
        const float *gu[2] = {s->w1, s->w3};
        const int r2[2] = {CD_HID, CD_HID};
        ok &= (l->wqkv = cd_upload_stack(qkv, r3, 3, CD_DIM)) != NULL;
        ok &= (l->w13 = cd_upload_stack(gu, r2, 2, CD_DIM)) != NULL;
        ok &= (l->wo = cd_upload(s->wo, (size_t)CD_DIM * CD_DIM)) != NULL;
        ok &= (l->w2 = cd_upload(s->w2, (size_t)CD_DIM * CD_HID)) != NULL;
        ok &= (l->attention_norm = cd_upload(s->attention_norm, CD_DIM)) != NULL;
        ok &= (l->ffn_norm = cd_upload(s->ffn_norm, CD_DIM)) != NULL;
        l->q_norm = s->q_norm ? cd_upload(s->q_norm, CD_DIM) : NULL;
        l->k_norm = s->k_norm ? cd_upload(s->k_norm, CD_DIM) : NULL;
        l->attn_scale = s->attn_scale ? cd_upload(s->attn_scale, CD_DIM) : NULL;
        l->ffn_scale = s->ffn_scale ? cd_upload(s->ffn_scale, CD_DIM) : NULL;
        l->window = s->window_size;
    }
    if (!ok) { vt_codec_free(); return -1; }
    g_cd.uploaded = 1;
    return 0;
}

static int cd_reserve(int n_frames) {
    if (n_frames <= g_cd.cap_frames) return 0;
    (void)hipStreamSynchronize(g_vt.stream);
    float **ws[] = {&g_cd.x, &g_cd.xn, &g_cd.qkv, &g_cd.att, &g_cd.h, &g_cd.wide, &g_cd.part, &g_cd.wave};
    for (size_t k = 0; k < sizeof ws / sizeof ws[0]; k++) cd_free_ptr(ws[k]);
    if (g_cd.codes) { (void)hipFree(g_cd.codes); g_cd.codes = NULL; }
    g_cd.cap_frames = 0;
    const size_t T = (size_t)n_frames * 8;
    const size_t f = sizeof(float);
    g_cd.x = (float *)vt_dev_alloc(T * CD_DIM * f);
    g_cd.xn = (float *)vt_dev_alloc(T * CD_DIM * f);
    g_cd.qkv = (float *)vt_dev_alloc(T * 3 * CD_DIM * f);
    g_cd.att = (float *)vt_dev_alloc(T * CD_DIM * f);
    g_cd.h = (float *)vt_dev_alloc(T * CD_HID * f);
    g_cd.wide = (float *)vt_dev_alloc(T * 2 * CD_HID * f);             /* gate|up, tap copies (<= 7168 wide) */
    /* K-cut planes: uncut at most [T, 3072]; a cut launch has at most 4 tiles per compute unit */
    size_t part = T * 3 * CD_DIM, cut = (size_t)4 * g_vt.n_cu * CG_BM * CG_BN;
    g_cd.part = (float *)vt_dev_alloc((part > cut ? part : cut) * f);
    g_cd.wave = (float *)vt_dev_alloc(T * CD_PATCH * f);
    g_cd.codes = (int *)vt_dev_alloc((size_t)n_frames * 37 * sizeof(int));
    if (!g_cd.x || !g_cd.xn || !g_cd.qkv || !g_cd.att || !g_cd.h || !g_cd.wide || !g_cd.part || !g_cd.wave || !g_cd.codes)
        return -1;
    g_cd.cap_frames = n_frames;
    return 0;
}

/* K is cut until the launch has about two workgroups per compute unit */
static int cd_splits_bm(int M, int N, int K, int bm) {
    const int tiles = ((M + bm - 1) / bm) * ((N + CG_BN - 1) / CG_BN);
    int s = 1;
    while (s < CD_MAX_SPLIT && tiles * s < 2 * g_vt.n_cu && (K / (s * 2)) % CG_BK == 0 && K / (s * 2) >= 128) s *= 2;
    return s;
}

/* Tile height and K cuts of a product: of the two tile heights the one whose busiest compute unit has
 * less to do (workgroups per CU, rounded up, times the work of one), fewer cuts on a tie (their planes
 * are written and read again), then the taller tile. */
struct cd_plan { int bm, splits; };
static cd_plan cd_plan_for(int M, int N, int K, int max_splits) {
    cd_plan best = {CG_BM, 1};
    long best_cost = -1;
    const int heights[2] = {CG_BM, 64};
    for (int h = 0; h < 2; h++) {
        const int bm = heights[h];
        int s = cd_splits_bm(M, N, K, bm);
        while (s > max_splits) s /= 2;
        const long wgs = (long)((M + bm - 1) / bm) * ((N + CG_BN - 1) / CG_BN) * s;
        const long cost = ((wgs + g_vt.n_cu - 1) / g_vt.n_cu) * bm * (K / s);
        if (best_cost < 0 || cost < best_cost || (cost == best_cost && s < best.splits)) {
            best = cd_plan{bm, s};
            best_cost = cost;
        }
    }
    return best;
}

/* C planes (returns the number of planes written at stride M * ldc) */
static int cd_gemm(float *C, const float *A, const float *W, int M, int N, int K, int lda, int ldc, int max_splits = CD_MAX_SPLIT) {
    const cd_plan pl = cd_plan_for(M, N, K, max_splits);
    dim3 grid((N + CG_BN - 1) / CG_BN, (M + pl.bm - 1) / pl.bm, pl.splits);
    if (pl.bm == CG_BM)
        hipLaunchKernelGGL(vt_codec_gemm_kernel, grid, dim3(256), 0, g_vt.stream, C, A, W, M, N, K, lda, ldc, (size_t)M * ldc);
    else
        hipLaunchKernelGGL(vt_codec_gemm64_kernel, grid, dim3(256), 0, g_vt.stream, C, A, W, M, N, K, lda, ldc, (size_t)M * ldc);
    return pl.splits;
}

static void cd_row(float *x_out, float *xn_out, const float *x_in, const float *planes, int splits, size_t plane_stride,
                   int ldp, const float *bias, const float *scale, const float *norm_w, int rows) {
    hipLaunchKernelGGL(vt_codec_row_kernel, dim3(rows), dim3(256), 0, g_vt.stream, x_out, xn_out, x_in, planes,
                       splits, plane_stride, ldp, bias, scale, norm_w, CD_EPS);
}

/* the whole decoder on the library's stream: d_codes [n_frames, 37] -> d_samples [n_frames * 1920] */
static int cd_enqueue(const int *d_codes, int n_frames, float *d_samples) {
    int T = n_frames;
    const float scale = 1.0f / sqrtf((float)CD_HEAD_DIM);
    hipLaunchKernelGGL(vt_codec_embed_kernel, dim3(T), dim3(256), 0, g_vt.stream, g_cd.wide, d_codes, g_cd.sem, T);
    int sp = cd_gemm(g_cd.part, g_cd.wide, g_cd.w_in, T, CD_DIM, CD_IN_K, CD_IN_K, CD_DIM);
    cd_row(g_cd.x, g_cd.xn, NULL, g_cd.part, sp, (size_t)T * CD_DIM, CD_DIM, g_cd.b_in, NULL,
           g_cd.layers[0].attention_norm, T);
    for (int li = 0; li < CD_LAYERS; li++) {
        const cd_layer_dev *l = &g_cd.layers[li];
        sp = cd_gemm(g_cd.part, g_cd.xn, l->wqkv, T, 3 * CD_DIM, CD_DIM, CD_DIM, 3 * CD_DIM);
        hipLaunchKernelGGL(vt_codec_qkv_kernel, dim3(T), dim3(256), 0, g_vt.stream, g_cd.qkv, g_cd.part, sp,
                           (size_t)T * 3 * CD_DIM, l->q_norm, l->k_norm);
        hipLaunchKernelGGL(vt_codec_attention_kernel, dim3((T * CD_HEADS + 3) / 4), dim3(256), 0, g_vt.stream,
                           g_cd.att, g_cd.qkv, T, l->window, g_cd.slopes, scale);
        sp = cd_gemm(g_cd.part, g_cd.att, l->wo, T, CD_DIM, CD_DIM, CD_DIM, CD_DIM);
        cd_row(g_cd.x, g_cd.xn, g_cd.x, g_cd.part, sp, (size_t)T * CD_DIM, CD_DIM, NULL, l->attn_scale, l->ffn_norm, T);
        /* gate|up: uncut while its tiles fill the chip; the short stages (2 or 4 row tiles x 64) are cut
         * in K like the other products and the SiLU x up pass sums the planes */
        const int gu_tiles = ((T + CG_BM - 1) / CG_BM) * (2 * CD_HID / CG_BN);
        int gu_cuts = gu_tiles <= g_vt.n_cu ? CD_MAX_SPLIT : 1;
        while (gu_cuts > 1 && (size_t)T * gu_cuts > (size_t)g_cd.cap_frames * 8) gu_cuts /= 2;   /* the planes share the work area of the last stage's [8 n, 8192] */
        sp = cd_gemm(g_cd.wide, g_cd.xn, l->w13, T, 2 * CD_HID, CD_DIM, CD_DIM, 2 * CD_HID, gu_cuts);
        {
            const size_t n = (size_t)T * CD_HID;
            const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
            hipLaunchKernelGGL(vt_codec_swiglu_kernel, dim3(blocks), dim3(256), 0, g_vt.stream, g_cd.h, g_cd.wide, sp,
                               (size_t)T * 2 * CD_HID, n);
        }
        sp = cd_gemm(g_cd.part, g_cd.h, l->w2, T, CD_DIM, CD_HID, CD_HID, CD_DIM);
        const int last_of_stage = (li & 1) == 1;
        const float *next_norm = (!last_of_stage) ? g_cd.layers[li + 1].attention_norm : NULL;
        cd_row(g_cd.x, g_cd.xn, g_cd.x, g_cd.part, sp, (size_t)T * CD_DIM, CD_DIM, NULL, l->ffn_scale, next_norm, T);
        if (last_of_stage && li < CD_LAYERS - 1) {
            const int st = li / 2;
            hipLaunchKernelGGL(vt_codec_pair_kernel, dim3(T), dim3(256), 0, g_vt.stream, g_cd.wide, g_cd.x, T);
            sp = cd_gemm(g_cd.part, g_cd.wide, g_cd.w_up[st], T, 2 * CD_DIM, 2 * CD_DIM, 2 * CD_DIM, 2 * CD_DIM);
            /* [T, 2048] planes are [2T, 1024] rows */
            cd_row(g_cd.x, g_cd.xn, NULL, g_cd.part, sp, (size_t)T * 2 * CD_DIM, CD_DIM, g_cd.b_up[st], NULL,
                   g_cd.layers[li + 1].attention_norm, 2 * T);
            T *= 2;
        }
    }
    hipLaunchKernelGGL(vt_codec_taps_kernel, dim3(T), dim3(256), 0, g_vt.stream, g_cd.wide, g_cd.x, T, CD_OUT_TAPS);
    sp = cd_gemm(g_cd.part, g_cd.wide, g_cd.w_out, T, CD_PATCH, CD_OUT_K, CD_OUT_K, CD_OUT_N);
    hipLaunchKernelGGL(vt_codec_wave_kernel, dim3(T), dim3(256), 0, g_vt.stream, d_samples, g_cd.part, sp,
                       (size_t)T * CD_OUT_N, CD_OUT_N, g_cd.b_out, T);
    return vt_check(hipGetLastError(), "codec launch");
}

static int cd_ready(const char *who, int n_frames) {
    if (!g_vt.initialized || !g_cd.uploaded) { vt_set_error("%s: codec weights not uploaded", who); return -1; }
    if (n_frames < 1 || n_frames > 4096) { vt_set_error("%s: n_frames %d out of range", who, n_frames); return -1; }
    if (cd_reserve(n_frames)) { vt_set_error("%s: out of device memory for %d frames", who, n_frames); return -1; }
    return 0;
}

/* device codes -> device waveform (n_frames * 1920 floats), asynchronous on the library's stream */
extern "C" int tts_hip_codec_decode_device(const int *d_codes, int n_frames, float *d_samples) {
    if (cd_ready("tts_hip_codec_decode_device", n_frames)) return -1;
    if (!d_codes || !d_samples) { vt_set_error("tts_hip_codec_decode_device: NULL buffer"); return -1; }
    return cd_enqueue(d_codes, n_frames, d_samples);
}

/* replaces tts_codec_decode (voxtral_tts_codec.c:389): host codes [n_frames, 37] -> a malloc'ed
 * waveform the caller frees; NULL / 0 on failure. */
extern "C" void tts_hip_codec_decode(const int *codes, int n_frames, float **out_samples, int *out_n_samples) {
    if (out_samples) *out_samples = NULL;
    if (out_n_samples) *out_n_samples = 0;
    if (!codes || !out_samples || !out_n_samples) { vt_set_error("tts_hip_codec_decode: NULL argument"); return; }
    if (cd_ready("tts_hip_codec_decode", n_frames)) return;
    const int n = n_frames * 8 * CD_PATCH;
    float *s = (float *)malloc((size_t)n * sizeof(float));
    if (!s) { vt_set_error("tts_hip_codec_decode: out of host memory"); return; }
    if (vt_check(hipMemcpyAsync(g_cd.codes, codes, (size_t)n_frames * 37 * sizeof(int), hipMemcpyHostToDevice, g_vt.stream), "codes copy") ||
        cd_enqueue(g_cd.codes, n_frames, g_cd.wave) ||
        vt_check(hipMemcpyAsync(s, g_cd.wave, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, g_vt.stream), "waveform copy") ||
        vt_check(hipStreamSynchronize(g_vt.stream), "codec decode")) {
        free(s);
        return;
    }
    *out_samples = s;
    *out_n_samples = n;
}

/* For other translation units of the library: one launch of the decoder's product kernel at the last
 * stage's 1600 rows with the q|k|v, output, gate|up or down matrix of layer 7 (which 0..3; K cut as in
 * the decoder), or of the whole decoder on 200 frames of resident codes (which 4), on the decoder's own
 * work buffers.  vt_codec_probe_buffers hands out those buffers (activations xn, att [1600, 1024] and
 * h [1600, 4096], the codes) so that a caller can fill them. */
int vt_codec_probe_buffers(float **xn, float **att, float **h, int **codes) {
    if (!g_cd.uploaded) { vt_set_error("codec weights not uploaded"); return -1; }
    if (cd_reserve(200)) { vt_set_error("codec: out of device memory"); return -1; }
    *xn = g_cd.xn; *att = g_cd.att; *h = g_cd.h; *codes = g_cd.codes;
    return 0;
}

int vt_codec_probe_launch(int which) {
    const int frames = 200, T = frames * 8;
    const cd_layer_dev *l = &g_cd.layers[CD_LAYERS - 1];
    const float *W[4] = {l->wqkv, l->wo, l->w13, l->w2};
    const float *A[4] = {g_cd.xn, g_cd.att, g_cd.xn, g_cd.h};
    float *Cc[4] = {g_cd.part, g_cd.part, g_cd.wide, g_cd.part};
    static const int NN[4] = {3 * CD_DIM, CD_DIM, 2 * CD_HID, CD_DIM}, KK[4] = {CD_DIM, CD_DIM, CD_DIM, CD_HID};
    if (which == 4) return cd_enqueue(g_cd.codes, frames, g_cd.wave);
    if (which < 0 || which > 3) return -1;
    cd_gemm(Cc[which], A[which], W[which], T, NN[which], KK[which], KK[which], NN[which], which == 2 ? 1 : CD_MAX_SPLIT);
    return 0;
}
