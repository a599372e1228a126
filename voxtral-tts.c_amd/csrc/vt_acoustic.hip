/*
 * vt_acoustic.hip - the flow-matching acoustic transformer (replaces
 * tts_cuda_predict_velocity, voxtral_tts_cuda.cu:1016-1100; the frame loop
 * follows tts_acoustic_forward, voxtral_tts_acoustic.c:268-373, and the
 * velocity network predict_velocity, :182-262).
 *
 * The conditional and the unconditional branch of classifier-free guidance
 * run as one batch of 6 rows (2 branches x 3 tokens), so every weight is
 * streamed once per Euler step instead of twice.  Work that does not depend
 * on the step is hoisted: the projected LLM token is computed once per frame
 * and the 7 projected time tokens once per weight upload.
 *
 * A layer is four kernels, each a skinny product on the matrix cores
 * (v_mfma_f32_16x16x32_bf16, the 6 activation rows as (hi, lo) bf16 planes in
 * LDS, 16 weight rows per workgroup streamed straight from HBM into the B
 * operand, the 8 waves of a workgroup splitting K):
 *   RMSNorm + q|k|v            -> qkv [6, 6144]
 *   attention (3x3 per head and branch) + output projection + residual
 *   RMSNorm + gate/up + SiLU*up -> h [6, 9216]
 *   down projection + residual
 * A one-workgroup kernel closes a step (final norm, 36-wide output
 * projection of both branches, guided Euler update) and opens the next one
 * (input projection of the new latent, token assembly).
 */
#include "vt_state.h"

#include <math.h>
#include <string.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define AC_ROWS    6
#define AC_THREADS 512
#define AC_WAVES   8
#define AC_STEPS   7              /* Euler intervals (8 time points) */

enum { AC_QKV = 0, AC_WO = 1, AC_W13 = 2, AC_W2 = 3 };

struct ac_phase_args {
    const uint16_t *W;            /* [N, K] bf16 */
    const float *in;              /* QKV/W13: tok [6,3072]; WO: qkv [6,6144]; W2: h [6,9216] */
    const float *gain;            /* RMSNorm gains (QKV, W13) */
    float *out;                   /* QKV: qkv; WO/W2: tok (residual, in place); W13: h */
};

template <int PH> struct ac_shape {
    static constexpr int KP = PH == AC_WO ? VT_Q_DIM : VT_DIM;      /* K per pass */
    static constexpr int NPASS = PH == AC_W2 ? 3 : 1;
    static constexpr int KTOT = KP * NPASS;
    static constexpr int KW = KP / AC_WAVES;                         /* K per wave and pass */
    static constexpr int NL = KW / 32;                               /* 16-byte loads per lane and pass */
    static constexpr int PITCH = KP * 2 + 16;                        /* bytes per plane row */
    static constexpr int PLANE = AC_ROWS * PITCH;
    static constexpr int LDS_BYTES = 2 * PLANE + 4 * (AC_WAVES * AC_ROWS * 16 + AC_WAVES * 8);
};

/* rows of 3072 -> planes, optionally through RMSNorm.  Thread t owns the column
 * pairs 2t + 1024 j. */
template <bool NORM>
__device__ __forceinline__ void ac_rows_to_planes(unsigned char *hi, unsigned char *lo, int pitch,
                                                  const float *src, int src_stride, const float *gain,
                                                  float *red) {
    const int t = (int)threadIdx.x;
    f32x2 v[AC_ROWS][3];
#pragma unroll
    for (int m = 0; m < AC_ROWS; m++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            v[m][j] = *reinterpret_cast<const f32x2 *>(src + (size_t)m * src_stride + 2 * t + 1024 * j);
    float inv[AC_ROWS];
    if (NORM) {
#pragma unroll
        for (int m = 0; m < AC_ROWS; m++) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 3; j++) ss = fmaf(v[m][j].x, v[m][j].x, fmaf(v[m][j].y, v[m][j].y, ss));
            ss = vt_wave_sum(ss);
            if (vt_lane() == 0) red[vt_wave() * 8 + m] = ss;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < AC_ROWS; m++) {
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < AC_WAVES; w++) tot += red[w * 8 + m];
            inv[m] = 1.0f / sqrtf(tot / (float)VT_DIM + VT_EPS);
        }
    }
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int c = 2 * t + 1024 * j;
        f32x2 g = {1.f, 1.f};
        if (NORM) g = *reinterpret_cast<const f32x2 *>(gain + c);
#pragma unroll
        for (int m = 0; m < AC_ROWS; m++) {
            float a = v[m][j].x, b = v[m][j].y;
            if (NORM) {
                a = __fmul_rn(__fmul_rn(a, inv[m]), g.x);
                b = __fmul_rn(__fmul_rn(b, inv[m]), g.y);
            }
            unsigned h0, l0, h1, l1;
            vt_split_planes(a, h0, l0);
            vt_split_planes(b, h1, l1);
            *reinterpret_cast<unsigned *>(hi + m * pitch + 2 * c) = h0 | (h1 << 16);
            *reinterpret_cast<unsigned *>(lo + m * pitch + 2 * c) = l0 | (l1 << 16);
        }
    }
}

/* Bidirectional attention over the 3 tokens of each branch, straight into the
 * planes that feed the output projection (tts_bidirectional_attention,
 * voxtral_tts_kernels.c:467-525).  8 lanes per (branch, head), 16 dims each. */
__device__ __forceinline__ void ac_attention_to_planes(unsigned char *hi, unsigned char *lo, int pitch,
                                                       const float *qkv) {
    const int lane = vt_lane(), pair = vt_wave() * 8 + (lane >> 3), sub = lane & 7;
    const int br = pair >> 5, h = pair & 31, d0 = sub * 16;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);
    float q[3][16], k[3][16], v[3][16];
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const float *row = qkv + (size_t)(br * 3 + i) * VT_QKV_DIM;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const f32x4 a = *reinterpret_cast<const f32x4 *>(row + h * VT_HEAD_DIM + d0 + 4 * e);
            const f32x4 b = *reinterpret_cast<const f32x4 *>(row + VT_Q_DIM + (h >> 2) * VT_HEAD_DIM + d0 + 4 * e);
            const f32x4 c = *reinterpret_cast<const f32x4 *>(row + VT_Q_DIM + VT_KV_DIM + (h >> 2) * VT_HEAD_DIM + d0 + 4 * e);
            q[i][4 * e] = a.x; q[i][4 * e + 1] = a.y; q[i][4 * e + 2] = a.z; q[i][4 * e + 3] = a.w;
            k[i][4 * e] = b.x; k[i][4 * e + 1] = b.y; k[i][4 * e + 2] = b.z; k[i][4 * e + 3] = b.w;
            v[i][4 * e] = c.x; v[i][4 * e + 1] = c.y; v[i][4 * e + 2] = c.z; v[i][4 * e + 3] = c.w;
        }
    }
#pragma unroll
    for (int i = 0; i < 3; i++) {
        float s[3];
#pragma unroll
        for (int j = 0; j < 3; j++) {
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < 16; e++) p = fmaf(q[i][e], k[j][e], p);
            p += vt_dpp<0xB1>(p);                 /* lanes ^1 */
            p += vt_dpp<0x4E>(p);                 /* lanes ^2 */
            p += vt_dpp<0x141>(p);                /* the other half of the 8-lane group (row_half_mirror) */
            s[j] = __fmul_rn(p, scale);
        }
        const float mx = fmaxf(s[0], fmaxf(s[1], s[2]));
        const float p0 = expf(s[0] - mx), p1 = expf(s[1] - mx), p2 = expf(s[2] - mx);
        const float inv = __fdiv_rn(1.0f, (p0 + p1) + p2);
        unsigned char *ph = hi + (br * 3 + i) * pitch + 2 * (h * VT_HEAD_DIM + d0);
        unsigned char *pl = lo + (br * 3 + i) * pitch + 2 * (h * VT_HEAD_DIM + d0);
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const float o0 = __fmul_rn(fmaf(p2, v[2][e], fmaf(p1, v[1][e], p0 * v[0][e])), inv);
            const float o1 = __fmul_rn(fmaf(p2, v[2][e + 1], fmaf(p1, v[1][e + 1], p0 * v[0][e + 1])), inv);
            unsigned h0, l0, h1, l1;
            vt_split_planes(o0, h0, l0);
            vt_split_planes(o1, h1, l1);
            *reinterpret_cast<unsigned *>(ph + 2 * e) = h0 | (h1 << 16);
            *reinterpret_cast<unsigned *>(pl + 2 * e) = l0 | (l1 << 16);
        }
    }
}

template <int PH>
__global__ void __launch_bounds__(AC_THREADS)
vt_ac_phase_kernel(ac_phase_args a) {
    typedef ac_shape<PH> SH;
    extern __shared__ __attribute__((aligned(16))) unsigned char ac_lds[];
    unsigned char *hi = ac_lds, *lo = ac_lds + SH::PLANE;
    float *red = reinterpret_cast<float *>(ac_lds + 2 * SH::PLANE);          /* [8 waves][6][16] */
    float *red_ss = red + AC_WAVES * AC_ROWS * 16;                           /* [8 waves][8] */
    const int lane = vt_lane(), wave = vt_wave();
    const int col = lane & 15, kg = lane >> 4;
    const int n0 = (int)blockIdx.x * 16;
    const uint16_t *wrow = a.W + (size_t)(n0 + col) * SH::KTOT + wave * SH::KW + 8 * kg;

    u32x4 wreg[2][SH::NL];
#pragma unroll
    for (int i = 0; i < SH::NL; i++) wreg[0][i] = vt_ldw(wrow + 32 * i);

    f32x4 acc_hi = {0.f, 0.f, 0.f, 0.f}, acc_lo = {0.f, 0.f, 0.f, 0.f};
    const int arow = col < AC_ROWS ? col : 0;          /* rows 6..15 of the A operand are don't-care */
    const unsigned char *fa = hi + arow * SH::PITCH + 2 * (wave * SH::KW + 8 * kg);
    const unsigned char *fl = lo + arow * SH::PITCH + 2 * (wave * SH::KW + 8 * kg);

#pragma unroll
    for (int pass = 0; pass < SH::NPASS; pass++) {
        if (pass > 0) __syncthreads();                 /* every wave is done with the previous planes */
        if (PH == AC_QKV || PH == AC_W13) ac_rows_to_planes<true>(hi, lo, SH::PITCH, a.in, VT_DIM, a.gain, red_ss);
        if (PH == AC_W2) ac_rows_to_planes<false>(hi, lo, SH::PITCH, a.in + pass * SH::KP, VT_FFN, NULL, red_ss);
        if (PH == AC_WO) ac_attention_to_planes(hi, lo, SH::PITCH, a.in);
        __syncthreads();
        if (pass + 1 < SH::NPASS) {
#pragma unroll
            for (int i = 0; i < SH::NL; i++) wreg[(pass + 1) & 1][i] = vt_ldw(wrow + (pass + 1) * SH::KP + 32 * i);
        }
#pragma unroll
        for (int i = 0; i < SH::NL; i++) {
            const bf16x8 b = __builtin_bit_cast(bf16x8, wreg[pass & 1][i]);
            const bf16x8 xh = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(fa + 64 * i));
            const bf16x8 xl = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(fl + 64 * i));
            acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xl, b, acc_lo, 0, 0, 0);
            acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xh, b, acc_hi, 0, 0, 0);
        }
    }

    /* accumulator element v of lane l: activation row 4*(l/16) + v, weight row l%16 */
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = 4 * kg + v;
        if (m < AC_ROWS) red[(wave * AC_ROWS + m) * 16 + col] = acc_hi[v] + acc_lo[v];
    }
    __syncthreads();
    const int t = (int)threadIdx.x;
    if (PH == AC_W13) {
        if (t < AC_ROWS * 8) {
            const int m = t >> 3, j = t & 7;
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < AC_WAVES; w++) {
                g += red[(w * AC_ROWS + m) * 16 + 2 * j];
                u += red[(w * AC_ROWS + m) * 16 + 2 * j + 1];
            }
            a.out[(size_t)m * VT_FFN + (n0 >> 1) + j] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
        }
    } else if (t < AC_ROWS * 16) {
        const int m = t >> 4, n = t & 15;
        float y = 0.f;
#pragma unroll
        for (int w = 0; w < AC_WAVES; w++) y += red[(w * AC_ROWS + m) * 16 + n];
        if (PH == AC_QKV) {
            a.out[(size_t)m * VT_QKV_DIM + n0 + n] = y;
        } else {
            float *p = a.out + (size_t)m * VT_DIM + n0 + n;
            *p = __fadd_rn(*p, y);
        }
    }
}

/* ---- step boundary: one workgroup ---------------------------------------------- */

struct ac_edge_args {
    const float *tok_in;          /* [6,3072] after the last layer (back part) */
    float *tok_out;               /* [6,3072] for the next step (front part) */
    const float *norm;            /* final norm gains */
    const uint16_t *acoustic_out; /* [36,3072] */
    const uint16_t *input_proj;   /* [3072,36] */
    const float *time_tok;        /* [3072] projected time token of the next step */
    const float *llm_tok;         /* [3072] projected LLM token */
    float *x;                     /* [36] latent, updated in place */
    float *vel;                   /* [72] cond | uncond velocities (written when do_back) */
    int *codes;                   /* [37] (FSQ codes at 1..36 when do_fsq) */
    float dt;
    int do_back, do_euler, do_front, do_fsq;
};

__global__ void __launch_bounds__(1024)
vt_ac_edge_kernel(ac_edge_args a) {
    __shared__ float red[2][16];
    __shared__ float s_inv[2];
    __shared__ float s_vel[2 * VT_AC_DIM_IN];
    __shared__ float s_x[VT_AC_DIM_IN];
    const int t = (int)threadIdx.x, lane = vt_lane(), wave = vt_wave();
    if (t < VT_AC_DIM_IN) s_x[t] = a.x[t];
    if (a.do_back) {
        /* final RMSNorm of token 0 of each branch (rows 0 and 3), then the 36-wide projection
         * (voxtral_tts_acoustic.c:255-261) */
        float ss[2] = {0.f, 0.f};
#pragma unroll
        for (int b = 0; b < 2; b++) {
            for (int c = t; c < VT_DIM; c += 1024) {
                const float v = a.tok_in[(size_t)(3 * b) * VT_DIM + c];
                ss[b] = fmaf(v, v, ss[b]);
            }
            ss[b] = vt_wave_sum(ss[b]);
            if (lane == 0) red[b][wave] = ss[b];
        }
        __syncthreads();
        if (t < 2) {
            float tot = 0.f;
            for (int w = 0; w < 16; w++) tot += red[t][w];
            s_inv[t] = 1.0f / sqrtf(tot / (float)VT_DIM + VT_EPS);
        }
        __syncthreads();
        for (int o = wave; o < 2 * VT_AC_DIM_IN; o += 16) {
            const int b = o / VT_AC_DIM_IN, r = o % VT_AC_DIM_IN;
            const float inv = s_inv[b];
            float acc = 0.f;
            for (int c = lane; c < VT_DIM; c += 64) {
                const float xn = __fmul_rn(__fmul_rn(a.tok_in[(size_t)(3 * b) * VT_DIM + c], inv), a.norm[c]);
                acc = fmaf(__uint_as_float((unsigned)a.acoustic_out[(size_t)r * VT_DIM + c] << 16), xn, acc);
            }
            acc = vt_wave_sum(acc);
            if (lane == 0) { s_vel[o] = acc; a.vel[o] = acc; }
        }
        __syncthreads();
    }
    if (a.do_euler && t < VT_AC_DIM_IN) {
        /* x += (1.2*vc + (1-1.2)*vu) * dt, each product rounded (voxtral_tts_acoustic.c:350-354) */
        const float p = __fmul_rn(1.2f, s_vel[t]);
        const float q = __fmul_rn(1.0f - 1.2f, s_vel[VT_AC_DIM_IN + t]);
        const float xn = __fadd_rn(s_x[t], __fmul_rn(__fadd_rn(p, q), a.dt));
        s_x[t] = xn;
        a.x[t] = xn;
    }
    __syncthreads();
    if (a.do_fsq && t < VT_AC_DIM_IN) {
        /* voxtral_tts_acoustic.c:358-372 */
        float v = s_x[t];
        if (v > 1.0f) v = 1.0f;
        if (v < -1.0f) v = -1.0f;
        const float scaled = __fmul_rn(__fdiv_rn(__fadd_rn(v, 1.0f), 2.0f), 20.0f);
        int c = (int)__fadd_rn(scaled, 0.5f);
        if (c < 0) c = 0;
        if (c > 20) c = 20;
        a.codes[t + 1] = c + 2;
    }
    if (a.do_front) {
        /* tokens of both branches: [noise, time, llm] and [noise, time, 0]; the noise token is
         * the 36-term input projection in the CPU order (voxtral_tts_kernels.c:152-185) */
        for (int c = t; c < VT_DIM; c += 1024) {
            float acc = 0.f;
            for (int k = 0; k < VT_AC_DIM_IN; k++)
                acc = __fadd_rn(acc, __fmul_rn(__uint_as_float((unsigned)a.input_proj[(size_t)c * VT_AC_DIM_IN + k] << 16), s_x[k]));
            const float tm = a.time_tok[c];
            a.tok_out[c] = acc;
            a.tok_out[VT_DIM + c] = tm;
            a.tok_out[2 * VT_DIM + c] = a.llm_tok[c];
            a.tok_out[3 * VT_DIM + c] = acc;
            a.tok_out[4 * VT_DIM + c] = tm;
            a.tok_out[5 * VT_DIM + c] = 0.f;
        }
    }
}

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

/* ---- host side ---------------------------------------------------------------------- */

/* device work area of the acoustic path, in floats */
struct ac_work {
    float *tok, *qkv, *h, *llm_tok, *hidden, *x, *vel, *temb, *time_tok1, *logits;
    int *codes;
};
#define AC_WORK_FLOATS (AC_ROWS * (VT_DIM + VT_QKV_DIM + VT_FFN) + 4 * VT_DIM + 64 + 128 + VT_SEM_PADDED + 64)

static void carve(ac_work *w, float *base) {
    w->tok = base;
    w->qkv = w->tok + AC_ROWS * VT_DIM;
    w->h = w->qkv + AC_ROWS * VT_QKV_DIM;
    w->llm_tok = w->h + AC_ROWS * VT_FFN;
    w->hidden = w->llm_tok + VT_DIM;
    w->temb = w->hidden + VT_DIM;
    w->time_tok1 = w->temb + VT_DIM;
    w->x = w->time_tok1 + VT_DIM;
    w->vel = w->x + 64;
    w->logits = w->vel + 128;
    w->codes = (int *)(w->logits + VT_SEM_PADDED);
}

template <int PH>
static int launch_phase(const uint16_t *W, const float *in, const float *gain, float *out, int n_rows) {
    static int attr_set = 0;
    const int lds = ac_shape<PH>::LDS_BYTES;
    if (!attr_set) {
        if (vt_check(hipFuncSetAttribute((const void *)vt_ac_phase_kernel<PH>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds), "acoustic LDS size"))
            return -1;
        attr_set = 1;
    }
    ac_phase_args a = {W, in, gain, out};
    hipLaunchKernelGGL(vt_ac_phase_kernel<PH>, dim3(n_rows / 16), dim3(AC_THREADS), lds, g_vt.stream, a);
    return 0;
}

/* the three layers on tok [6,3072] (in place) */
static int run_layers(const ac_work *w) {
    const vt_acoustic_dev *ac = &g_vt.ac;
    for (int l = 0; l < TTS_HIP_AC_LAYERS; l++) {
        const vt_layer_dev *L = &ac->layers[l];
        if (launch_phase<AC_QKV>(L->wqkv, w->tok, L->attn_norm, w->qkv, VT_QKV_DIM)) return -1;
        if (launch_phase<AC_WO>(L->wo, w->qkv, NULL, w->tok, VT_DIM)) return -1;
        if (launch_phase<AC_W13>(L->w13, w->tok, L->ffn_norm, w->h, 2 * VT_FFN)) return -1;
        if (launch_phase<AC_W2>(L->w2, w->h, NULL, w->tok, VT_DIM)) return -1;
    }
    return 0;
}

static void launch_edge(const ac_work *w, const float *time_tok, float dt, int back, int euler, int front, int fsq) {
    const vt_acoustic_dev *ac = &g_vt.ac;
    ac_edge_args a;
    a.tok_in = w->tok; a.tok_out = w->tok; a.norm = ac->norm; a.acoustic_out = ac->acoustic_out;
    a.input_proj = ac->input_proj; a.time_tok = time_tok; a.llm_tok = w->llm_tok; a.x = w->x; a.vel = w->vel;
    a.codes = w->codes; a.dt = dt; a.do_back = back; a.do_euler = euler; a.do_front = front; a.do_fsq = fsq;
    hipLaunchKernelGGL(vt_ac_edge_kernel, dim3(1), dim3(1024), 0, g_vt.stream, a);
}

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

/* time_tok[n] = time_proj(embedding(ts[i])) for n rows, through the pinned staging buffer */
static int project_times(float *d_out, float *d_temb, const float *ts, int n) {
    hipStream_t st = g_vt.stream;
    for (int i = 0; i < n; i++) {
        if (vt_check(hipStreamSynchronize(st), "time token sync")) return -1;
        time_embedding_host(ts[i], g_vt.h_pin);
        if (vt_check(hipMemcpyAsync(d_temb, g_vt.h_pin, sizeof(float) * VT_DIM, hipMemcpyHostToDevice, st), "time emb"))
            return -1;
        vt_launch_linear(d_out + (size_t)i * VT_DIM, d_temb, g_vt.ac.time_proj, NULL, 1, VT_DIM, VT_DIM);
    }
    return 0;
}

static int ac_ready(const char *who) {
    if (g_vt.initialized && g_vt.ac_uploaded) return 1;
    vt_set_error("%s: acoustic weights not uploaded", who);
    return 0;
}

static void predict(float *out_c, float *out_u, const float *x_t, const float *llm_hidden, float t_val) {
    float *base = (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
    if (!base) return;
    ac_work w;
    carve(&w, base);
    hipStream_t st = g_vt.stream;
    VT_TRYV(hipMemcpyAsync(w.hidden, llm_hidden, sizeof(float) * VT_DIM, hipMemcpyDefault, st));
    VT_TRYV(hipMemcpyAsync(w.x, x_t, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault, st));
    if (project_times(w.time_tok1, w.temb, &t_val, 1)) return;
    vt_launch_linear(w.llm_tok, w.hidden, g_vt.ac.llm_proj, NULL, 1, VT_DIM, VT_DIM);
    launch_edge(&w, w.time_tok1, 0.f, 0, 0, 1, 0);
    if (run_layers(&w)) return;
    launch_edge(&w, w.time_tok1, 0.f, 1, 0, 0, 0);
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    VT_TRYV(hipMemcpy(out_c, w.vel, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
    if (out_u) VT_TRYV(hipMemcpy(out_u, w.vel + VT_AC_DIM_IN, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault));
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

extern "C" void tts_hip_acoustic_frame(int *out_codes, const float *llm_hidden, const float *x0,
                                       float *out_x) {
    if (!ac_ready("tts_hip_acoustic_frame")) return;
    hipStream_t st = g_vt.stream;
    vt_acoustic_dev *ac = &g_vt.ac;
    float *base = (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
    if (!base) return;
    ac_work w;
    carve(&w, base);
    float ts[AC_STEPS + 1];
    for (int i = 0; i <= AC_STEPS; i++) ts[i] = (float)i / (float)AC_STEPS;
    if (!ac->time_tok_ready) {
        /* the projected time tokens depend on the weights only */
        if (project_times(ac->time_tok, w.temb, ts, AC_STEPS)) return;
        ac->time_tok_ready = 1;
    }
    VT_TRYV(hipMemcpyAsync(w.hidden, llm_hidden, sizeof(float) * VT_DIM, hipMemcpyDefault, st));
    VT_TRYV(hipMemcpyAsync(w.x, x0, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault, st));
    vt_launch_linear(w.logits, w.hidden, ac->semantic_out, ac->semantic_bias, 1, VT_DIM, VT_SEM_PADDED);
    hipLaunchKernelGGL(vt_semantic_argmax_kernel, dim3(1), dim3(1024), 0, st, w.logits, w.codes);
    vt_launch_linear(w.llm_tok, w.hidden, ac->llm_proj, NULL, 1, VT_DIM, VT_DIM);
    /* the flow runs without waiting for the semantic code; an END_AUDIO frame discards it */
    launch_edge(&w, ac->time_tok, 0.f, 0, 0, 1, 0);
    for (int s = 0; s < AC_STEPS; s++) {
        volatile float dt = ts[s + 1] - ts[s];
        if (run_layers(&w)) return;
        const int last = s + 1 == AC_STEPS;
        launch_edge(&w, ac->time_tok + (size_t)(last ? s : s + 1) * VT_DIM, (float)dt, 1, 1, !last, last);
    }
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    VT_TRYV(hipMemcpy(out_codes, w.codes, sizeof(int) * (1 + VT_AC_DIM_IN), hipMemcpyDeviceToHost));
    if (out_x) VT_TRYV(hipMemcpy(out_x, w.x, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDeviceToHost));
    if (out_codes[0] == 1) {                            /* END_AUDIO */
        for (int i = 1; i <= VT_AC_DIM_IN; i++) out_codes[i] = 2;
        if (out_x) memset(out_x, 0, sizeof(float) * VT_AC_DIM_IN);
    }
}
