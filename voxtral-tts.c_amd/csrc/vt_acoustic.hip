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
 * LDS, 12 weight rows at a time streamed straight from HBM into the B operand
 * by one persistent workgroup per CU, its 8 waves splitting K):
 *   RMSNorm + q|k|v            -> qkv [6, 6144]
 *   attention (3x3 per head and branch) + output projection + residual
 *   RMSNorm + gate/up + SiLU*up -> h [6, 9216]
 *   down projection + residual
 * Two small kernels stand between the steps: one closes a step (final norm,
 * 36-wide output projection of both branches), the other applies the guided
 * Euler update and opens the next step (input projection of the new latent,
 * token assembly).
 */
#include "vt_state.h"

#include <math.h>
#include <string.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(1))) const u32x4 ac_gptr_u32x4;

/* Two consecutive 16-byte loads of a lane share a 128-byte line (a load instruction
 * covers 16 weight rows x 64 bytes), so these are ordinary cached loads: the second
 * one must find the line the first one brought in. */
__device__ __forceinline__ u32x4 ac_ldw(const uint16_t *p) { return *(ac_gptr_u32x4 *)p; }

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
    /* units a workgroup takes on a 256-workgroup grid (more on a smaller one: then the buffers are reused) */
    static constexpr int UNITS = PH == AC_W13 ? 6 : PH == AC_QKV ? 2 : 1;
    static constexpr int RED_UNIT = AC_WAVES * AC_ROWS * 16;          /* floats: one unit's partial sums of all waves */
    static constexpr int RED_BYTES = 4 * (UNITS * RED_UNIT + AC_WAVES * 8);
    /* attention + output projection: the k|v columns of the 6 rows, shared by the 4 heads of a group */
    static constexpr int KV_BYTES = PH == AC_WO ? AC_ROWS * 2 * VT_KV_DIM * 4 : 0;
    static constexpr int LDS_BYTES = 2 * PLANE + RED_BYTES + KV_BYTES;
};

/* Activation rows are fetched into registers BEFORE the weight loads of a pass are
 * issued: a wave's loads return in order, so this way the planes can be built while
 * the weights are still streaming in. */
struct ac_attn_regs { f32x4 q[3][4]; f32x4 kv[AC_ROWS * 2 * VT_KV_DIM / 4 / AC_THREADS]; };

/* A wave's own K slice of the 6 rows.  The products of a wave read only the plane columns of its K slice
 * (wave w: columns w * KW .. + KW), so a wave that fetches, scales and converts exactly those columns
 * depends on no other wave before its first matrix instruction: no workgroup barrier between the rows'
 * arrival and the products.  Behind an RMSNorm the planes then hold x * gain and the result is multiplied
 * by 1/rms(x) in the epilogue, from the waves' partial sums of squares (red_ss[wave * 8 + m]). */
template <int KW> struct ac_slice_regs {
    static constexpr int NJ = (KW / 4 + 63) / 64;       /* 16-byte groups per lane and row */
    f32x4 v[AC_ROWS][NJ];
    f32x4 g[NJ];
};

template <int KW>
__device__ __forceinline__ void ac_fetch_slice(ac_slice_regs<KW> &r, const float *src, int src_stride, const float *gain) {
    constexpr int NJ = ac_slice_regs<KW>::NJ, G4 = KW / 4;
    const int lane = vt_lane(), c0 = vt_wave() * KW;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f}, one = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
    for (int m = 0; m < AC_ROWS; m++) {
        const f32x4 *row = reinterpret_cast<const f32x4 *>(src + (size_t)m * src_stride + c0);
#pragma unroll
        for (int j = 0; j < NJ; j++) r.v[m][j] = (64 * (j + 1) <= G4 || lane + 64 * j < G4) ? row[lane + 64 * j] : zero;
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) r.g[j] = one;
    if (gain) {
        const f32x4 *g = reinterpret_cast<const f32x4 *>(gain + c0);
#pragma unroll
        for (int j = 0; j < NJ; j++) r.g[j] = (64 * (j + 1) <= G4 || lane + 64 * j < G4) ? g[lane + 64 * j] : one;
    }
}

template <bool NORM, int KW>
__device__ __forceinline__ void ac_slice_to_planes(unsigned char *hi, unsigned char *lo, int pitch,
                                                   const ac_slice_regs<KW> &r, float *red_ss) {
    constexpr int NJ = ac_slice_regs<KW>::NJ, G4 = KW / 4;
    const int lane = vt_lane(), c0 = vt_wave() * KW;
    if (NORM) {
#pragma unroll
        for (int m = 0; m < AC_ROWS; m++) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const f32x4 v = r.v[m][j];
                ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            }
            ss = vt_wave_sum(ss);
            if (lane == 0) red_ss[vt_wave() * 8 + m] = ss;
        }
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (64 * (j + 1) <= G4 || lane + 64 * j < G4) {
            const int c = c0 + 4 * (lane + 64 * j);
            const f32x4 g = r.g[j];
#pragma unroll
            for (int m = 0; m < AC_ROWS; m++) {
                f32x4 v = r.v[m][j];
                if (NORM) { v.x = __fmul_rn(v.x, g.x); v.y = __fmul_rn(v.y, g.y); v.z = __fmul_rn(v.z, g.z); v.w = __fmul_rn(v.w, g.w); }
                u32x2 sph, spl;
                vt_split_planes4(v.x, v.y, v.z, v.w, sph, spl);
                *reinterpret_cast<u32x2 *>(hi + m * pitch + 2 * c) = sph;
                *reinterpret_cast<u32x2 *>(lo + m * pitch + 2 * c) = spl;
            }
        }
    }
    /* the wave's own stores before its own fragment reads: LDS serves a wave in order */
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

/* Bidirectional attention over the 3 tokens of each branch, straight into the
 * planes that feed the output projection (tts_bidirectional_attention,
 * voxtral_tts_kernels.c:467-525).  8 lanes per (branch, head), 16 dims each.  Every
 * lane keeps its q in registers; k and v, which the 4 heads of a group share, are
 * fetched once and handed round through LDS: each head fetching its own copy made this
 * kernel pull 295 KB of activations through its CU instead of 147 KB.
 * Wave w serves the query heads 4 w .. 4 w + 3 of both branches, i.e. kv head w: their outputs are exactly
 * the plane columns 512 w .. of the wave's own K slice, and the k|v rows they share are the wave's alone. */
__device__ __forceinline__ void ac_fetch_attn(ac_attn_regs &r, const float *qkv) {
    const int lane = vt_lane(), wave = vt_wave(), p = lane >> 3, sub = lane & 7;
    const int br = p >> 2, h = 4 * wave + (p & 3), d0 = sub * 16;
#pragma unroll
    for (int j = 0; j < AC_ROWS; j++) {                         /* row j: k (32 groups of 4) | v (32 groups) of kv head `wave` */
        const int which = lane >> 5, g4 = lane & 31;
        r.kv[j] = *reinterpret_cast<const f32x4 *>(qkv + (size_t)j * VT_QKV_DIM + VT_Q_DIM + which * VT_KV_DIM +
                                                   wave * VT_HEAD_DIM + 4 * g4);
    }
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const float *row = qkv + (size_t)(br * 3 + i) * VT_QKV_DIM;
#pragma unroll
        for (int e = 0; e < 4; e++) r.q[i][e] = *reinterpret_cast<const f32x4 *>(row + h * VT_HEAD_DIM + d0 + 4 * e);
    }
}

/* the wave's k|v into its part of LDS as [row][k 32 | v 32] groups of 4 */
__device__ __forceinline__ void ac_stage_kv(f32x4 *kvl, const ac_attn_regs &r) {
    f32x4 *mine = kvl + vt_wave() * (AC_ROWS * 64);
#pragma unroll
    for (int j = 0; j < AC_ROWS; j++) mine[j * 64 + vt_lane()] = r.kv[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");       /* LDS serves a wave in order */
    __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void ac_attention_to_planes(unsigned char *hi, unsigned char *lo, int pitch,
                                                       const ac_attn_regs &r, const f32x4 *kvl) {
    const int lane = vt_lane(), wave = vt_wave(), p = lane >> 3, sub = lane & 7;
    const int br = p >> 2, h = 4 * wave + (p & 3), d0 = sub * 16;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);
    const f32x4 *mine = kvl + wave * (AC_ROWS * 64);
    f32x4 k[3][4], v[3][4];
#pragma unroll
    for (int j = 0; j < 3; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int at = (br * 3 + j) * 64 + d0 / 4 + e;
            k[j][e] = mine[at];
            v[j][e] = mine[at + 32];
        }
#pragma unroll
    for (int i = 0; i < 3; i++) {
        float s[3];
#pragma unroll
        for (int j = 0; j < 3; j++) {
            float p = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                p = fmaf(r.q[i][e].x, k[j][e].x, p);
                p = fmaf(r.q[i][e].y, k[j][e].y, p);
                p = fmaf(r.q[i][e].z, k[j][e].z, p);
                p = fmaf(r.q[i][e].w, k[j][e].w, p);
            }
            p += vt_dpp<0xB1>(p);                 /* lanes ^1 */
            p += vt_dpp<0x4E>(p);                 /* lanes ^2 */
            p += vt_dpp<0x141>(p);                /* the other quad of the 8-lane group (row_half_mirror) */
            s[j] = __fmul_rn(p, scale);
        }
        const float mx = fmaxf(s[0], fmaxf(s[1], s[2]));
        const float p0 = expf(s[0] - mx), p1 = expf(s[1] - mx), p2 = expf(s[2] - mx);
        const float inv = __fdiv_rn(1.0f, (p0 + p1) + p2);
        unsigned char *ph = hi + (br * 3 + i) * pitch + 2 * (h * VT_HEAD_DIM + d0);
        unsigned char *pl = lo + (br * 3 + i) * pitch + 2 * (h * VT_HEAD_DIM + d0);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float o0 = __fmul_rn(fmaf(p2, v[2][e].x, fmaf(p1, v[1][e].x, p0 * v[0][e].x)), inv);
            const float o1 = __fmul_rn(fmaf(p2, v[2][e].y, fmaf(p1, v[1][e].y, p0 * v[0][e].y)), inv);
            const float o2 = __fmul_rn(fmaf(p2, v[2][e].z, fmaf(p1, v[1][e].z, p0 * v[0][e].z)), inv);
            const float o3 = __fmul_rn(fmaf(p2, v[2][e].w, fmaf(p1, v[1][e].w, p0 * v[0][e].w)), inv);
            u32x2 sph, spl;
            vt_split_planes4(o0, o1, o2, o3, sph, spl);
            const u32x2 vh = sph, vl = spl;
            *reinterpret_cast<u32x2 *>(ph + 8 * e) = vh;
            *reinterpret_cast<u32x2 *>(pl + 8 * e) = vl;
        }
    }
}

/* One persistent workgroup per CU.  A unit is AC_RB consecutive weight rows (12 of the
 * 16 columns of the matrix-core tile: 3072, 6144 and 18432 rows then split evenly over
 * 256 CUs); units are dealt round-robin.  The activation planes are built once per
 * workgroup, while the first unit's weights are already on their way; after that the
 * weights of unit u+1 stream into one register set while unit u is multiplied out of
 * the other.  The down projection (K = 9216) takes its K in three passes and rebuilds
 * the planes for each. */
#define AC_RB 12

template <int PH, int NL>
__device__ __forceinline__ void ac_issue(u32x4 (&wreg)[NL], const uint16_t *p) {
#pragma unroll
    for (int i = 0; i < NL; i++) wreg[i] = ac_ldw(p + 32 * i);
}

template <int NL>
__device__ __forceinline__ void ac_consume(const u32x4 (&wreg)[NL], const unsigned char *fa, const unsigned char *fl,
                                           f32x4 &acc_hi, f32x4 &acc_lo) {
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const bf16x8 b = __builtin_bit_cast(bf16x8, wreg[i]);
        const bf16x8 xh = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(fa + 64 * i));
        const bf16x8 xl = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(fl + 64 * i));
        acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xl, b, acc_lo, 0, 0, 0);
        acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xh, b, acc_hi, 0, 0, 0);
    }
}

/* cross-wave sum of one unit and its epilogue; `red` is this unit's buffer */
/* 1/rms of row m from the waves' partial sums of squares (wave-local planes) */
__device__ __forceinline__ float ac_inv_rms_of(const float *red_ss, int m) {
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < AC_WAVES; w++) tot += red_ss[w * 8 + m];
    return 1.0f / sqrtf(tot / (float)VT_DIM + VT_EPS);
}

/* A wave leaves its partial sums of one unit in that unit's buffer; nobody waits. */
__device__ __forceinline__ void ac_park_unit(float *red, f32x4 acc_hi, f32x4 acc_lo) {
    const int lane = vt_lane(), wave = vt_wave(), col = lane & 15, kg = lane >> 4;
    /* accumulator element v of lane l: activation row 4*(l/16) + v, weight row l%16 */
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = 4 * kg + v;
        if (m < AC_ROWS) red[(wave * AC_ROWS + m) * 16 + col] = acc_hi[v] + acc_lo[v];
    }
}

/* Behind the workgroup's barrier: cross-wave sums and epilogues of the `n` units parked in red (unit j of
 * them is weight rows (u0 + j * G) * 12 ..).  Thread t takes output element t % E of unit t / E. */
template <int PH>
__device__ __forceinline__ void ac_finish_units(const ac_phase_args &a, const float *red, int n, int u0, int G,
                                                bool have_prev, float prev, const float *red_ss) {
    typedef ac_shape<PH> SH;
    constexpr int E = PH == AC_W13 ? AC_ROWS * 8 : AC_ROWS * 16;     /* threads per unit */
    for (int t = (int)threadIdx.x; t < n * E; t += AC_THREADS) {
        const int j = t / E, e = t % E;
        const float *r = red + j * SH::RED_UNIT;
        const int n0 = (u0 + j * G) * AC_RB;
        if (PH == AC_W13) {
            if ((e & 7) < AC_RB / 2) {
                const int m = e >> 3, c = e & 7;
                float g = 0.f, u = 0.f;
#pragma unroll
                for (int w = 0; w < AC_WAVES; w++) {
                    g += r[(w * AC_ROWS + m) * 16 + 2 * c];
                    u += r[(w * AC_ROWS + m) * 16 + 2 * c + 1];
                }
                const float inv = ac_inv_rms_of(red_ss, m);
                g = __fmul_rn(g, inv);
                u = __fmul_rn(u, inv);
                a.out[(size_t)m * VT_FFN + (n0 >> 1) + c] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
            }
        } else if ((e & 15) < AC_RB) {
            const int m = e >> 4, c = e & 15;
            float y = 0.f;
#pragma unroll
            for (int w = 0; w < AC_WAVES; w++) y += r[(w * AC_ROWS + m) * 16 + c];
            if (PH == AC_QKV) {
                a.out[(size_t)m * VT_QKV_DIM + n0 + c] = __fmul_rn(y, ac_inv_rms_of(red_ss, m));
            } else {
                float *p = a.out + (size_t)m * VT_DIM + n0 + c;
                *p = __fadd_rn(have_prev && j == 0 ? prev : *p, y);
            }
        }
    }
}

template <int PH>
__global__ void __launch_bounds__(AC_THREADS)
vt_ac_phase_kernel(ac_phase_args a, int n_units) {
    typedef ac_shape<PH> SH;
    extern __shared__ __attribute__((aligned(16))) unsigned char ac_lds[];
    unsigned char *hi = ac_lds, *lo = ac_lds + SH::PLANE;
    float *red = reinterpret_cast<float *>(ac_lds + 2 * SH::PLANE);          /* UNITS x [8 waves][6][16] */
    float *red_ss = red + SH::UNITS * SH::RED_UNIT;                          /* [8 waves][8] */
    const int lane = vt_lane(), wave = vt_wave();
    const int col = lane & 15, kg = lane >> 4;
    const bool live = col < AC_RB;
    const int G = (int)gridDim.x;
    int u = (int)blockIdx.x;
    if (u >= n_units) return;
    /* this lane's weight row inside unit 0, at this wave's K slice; the four spare columns of
     * the tile repeat row 0 (same cache lines, results unused) */
    const uint16_t *wbase = a.W + (size_t)(live ? col : 0) * SH::KTOT + wave * SH::KW + 8 * kg;
    const size_t unit_stride = (size_t)AC_RB * SH::KTOT;
    const int arow = col < AC_ROWS ? col : 0;          /* rows 6..15 of the A operand are don't-care */
    const unsigned char *fa = hi + arow * SH::PITCH + 2 * (wave * SH::KW + 8 * kg);
    const unsigned char *fl = lo + arow * SH::PITCH + 2 * (wave * SH::KW + 8 * kg);
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    u32x4 w0[SH::NL], w1[SH::NL];
    /* the residual this workgroup's first unit is added to is requested before everything else (a
     * load of its own at the end of the kernel would cost a round trip to memory after the last
     * product); every thread asks, the ones without an output element for element 0 */
    const int first_unit = u;
    float prev = 0.f;
    if (PH == AC_WO || PH == AC_W2) {
        const int t = (int)threadIdx.x;
        const bool fin = t < AC_ROWS * 16 && (t & 15) < AC_RB;
        prev = a.out[(size_t)(fin ? t >> 4 : 0) * VT_DIM + u * AC_RB + (fin ? t & 15 : 0)];
    }

    /* behind an RMSNorm the planes hold x * gain; the epilogue multiplies by 1/rms(x) */
    const float *scale_ss = (PH == AC_QKV || PH == AC_W13) ? red_ss : nullptr;
    constexpr bool RES = PH == AC_WO || PH == AC_W2;
    int k = 0, u0 = u;                                  /* units parked, and the first of them */
    auto flush = [&] {
        __syncthreads();
        ac_finish_units<PH>(a, red, k, u0, G, RES && u0 == first_unit, prev, scale_ss);
        __syncthreads();                                /* the buffers are free again */
        u0 += k * G;
        k = 0;
    };
    if (SH::NPASS == 1) {
        if (PH != AC_WO) {
            /* every wave for itself: its K slice of the rows, no workgroup barrier before the products */
            ac_slice_regs<SH::KW> sr;
            ac_fetch_slice<SH::KW>(sr, a.in, VT_DIM, a.gain);
            ac_issue<PH>(w0, wbase + u * unit_stride);
            ac_slice_to_planes<true, SH::KW>(hi, lo, SH::PITCH, sr, red_ss);
        } else {
            ac_attn_regs ra;
            ac_fetch_attn(ra, a.in);
            ac_issue<PH>(w0, wbase + u * unit_stride);
            f32x4 *kvl = reinterpret_cast<f32x4 *>(ac_lds + 2 * SH::PLANE + SH::RED_BYTES);
            ac_stage_kv(kvl, ra);
            ac_attention_to_planes(hi, lo, SH::PITCH, ra, kvl);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        /* The request for unit u + G is never issued under a condition of its own: the compiler
         * counts outstanding loads statically, and behind a conditional request it would make the
         * product of unit u wait for unit u + G as well (which is what the two register sets are
         * there to avoid).  The last unit of a workgroup takes the branch without a request.
         * A wave parks its partial sums of a unit in that unit's buffer and goes on: the waves of a
         * workgroup meet once, behind the last unit (or when all buffers are full, on a small grid). */
        for (;;) {
            int nx = u + G;
            if (nx >= n_units) {
                f32x4 ah = zero4, al = zero4;
                ac_consume(w0, fa, fl, ah, al);
                ac_park_unit(red + k * SH::RED_UNIT, ah, al);
                k++;
                break;
            }
            {
                ac_issue<PH>(w1, wbase + nx * unit_stride);
                __builtin_amdgcn_sched_barrier(0);
                f32x4 ah = zero4, al = zero4;
                ac_consume(w0, fa, fl, ah, al);
                ac_park_unit(red + k * SH::RED_UNIT, ah, al);
                if (++k == SH::UNITS) flush();
                u = nx;
            }
            nx = u + G;
            if (nx >= n_units) {
                f32x4 ah = zero4, al = zero4;
                ac_consume(w1, fa, fl, ah, al);
                ac_park_unit(red + k * SH::RED_UNIT, ah, al);
                k++;
                break;
            }
            {
                ac_issue<PH>(w0, wbase + nx * unit_stride);
                __builtin_amdgcn_sched_barrier(0);
                f32x4 ah = zero4, al = zero4;
                ac_consume(w1, fa, fl, ah, al);
                ac_park_unit(red + k * SH::RED_UNIT, ah, al);
                if (++k == SH::UNITS) flush();
                u = nx;
            }
        }
    } else {
        for (; u < n_units; u += G) {
            const uint16_t *wp = wbase + u * unit_stride;
            ac_slice_regs<SH::KW> sr;
            ac_fetch_slice<SH::KW>(sr, a.in, VT_FFN, NULL);
            u32x4 wreg[2][SH::NL];
            ac_issue<PH>(wreg[0], wp);
            f32x4 ah = zero4, al = zero4;
#pragma unroll
            for (int pass = 0; pass < SH::NPASS; pass++) {
                ac_slice_to_planes<false, SH::KW>(hi, lo, SH::PITCH, sr, red_ss);
                if (pass + 1 < SH::NPASS) {
                    ac_fetch_slice<SH::KW>(sr, a.in + (pass + 1) * SH::KP, VT_FFN, NULL);
                    ac_issue<PH>(wreg[(pass + 1) & 1], wp + (pass + 1) * SH::KP);
                }
                ac_consume(wreg[pass & 1], fa, fl, ah, al);
            }
            ac_park_unit(red + k * SH::RED_UNIT, ah, al);
            if (++k == SH::UNITS) flush();
        }
    }
    if (k) {
        __syncthreads();
        ac_finish_units<PH>(a, red, k, u0, G, RES && u0 == first_unit, prev, scale_ss);
    }
}

/* ---- step boundary ------------------------------------------------------------------
 * Two small launches: `back` closes a step (final norm of token 0 of both branches, the 72
 * dot products of the 36-wide output projection), `front` applies the guided Euler update,
 * quantises at the end of the frame, and opens the next step (36-term input projection of the
 * new latent, token assembly).  Both used to be one workgroup, which then pulled the two
 * 221 KB matrices through a single CU (18 us per step); spread over 5 and 3 workgroups the
 * same arithmetic, element for element, takes a few microseconds per launch.  The latent is
 * read from x_in and written to x_out by workgroup 0 only (every workgroup of `front` applies
 * the update for itself; in place, a late workgroup would apply it twice). */

struct ac_edge_args {
    const float *tok_in;          /* [6,3072] after the last layer (back) */
    float *tok_out;               /* [6,3072] for the next step (front, when do_front) */
    const float *norm;            /* final norm gains */
    const uint16_t *acoustic_out; /* [36,3072] */
    const uint16_t *input_proj;   /* [3072,36] */
    const float *time_tok;        /* [3072] projected time token of the next step */
    const float *llm_tok;         /* [3072] projected LLM token */
    const float *x_in;            /* [36] latent */
    float *x_out;                 /* [36] latent after the update (== x_in values without do_euler) */
    float *vel;                   /* [72] cond | uncond velocities (written by back, read by front) */
    int *codes;                   /* [37] (FSQ codes at 1..36 when do_fsq) */
    float dt;
    int do_euler, do_front, do_fsq;
};

#define AC_BACK_WGS 5             /* x 16 waves >= 72 dot products */
#define AC_FRONT_WGS 3            /* x 1024 threads = 3072 token columns */

__global__ void __launch_bounds__(1024)
vt_ac_edge_back_kernel(ac_edge_args a) {
    __shared__ float red[2][16];
    __shared__ float s_inv[2];
    __shared__ __attribute__((aligned(16))) float s_xn[2][VT_DIM];
    const int t = (int)threadIdx.x, lane = vt_lane(), wave = vt_wave();
    /* this wave's row of the projection is requested first: it does not depend on the tokens */
    const int o = (int)blockIdx.x * 16 + wave;
    const bool mine = o < 2 * VT_AC_DIM_IN;
    const int ob = mine ? o / VT_AC_DIM_IN : 0, orow = mine ? o % VT_AC_DIM_IN : 0;
    u32x4 w[VT_DIM / 512];
#pragma unroll
    for (int i = 0; i < VT_DIM / 512; i++)
        w[i] = *reinterpret_cast<const u32x4 *>(a.acoustic_out + (size_t)orow * VT_DIM + 8 * (lane + 64 * i));
    /* final RMSNorm of token 0 of each branch (rows 0 and 3), then the 36-wide projection
     * (voxtral_tts_acoustic.c:255-261); every workgroup normalises for itself */
    float v[2][3];
#pragma unroll
    for (int b = 0; b < 2; b++) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 3; j++) {
            v[b][j] = a.tok_in[(size_t)(3 * b) * VT_DIM + t + 1024 * j];
            ss = fmaf(v[b][j], v[b][j], ss);
        }
        ss = vt_wave_sum(ss);
        if (lane == 0) red[b][wave] = ss;
    }
    __syncthreads();
    if (t < 2) {
        float tot = 0.f;
        for (int k = 0; k < 16; k++) tot += red[t][k];
        s_inv[t] = 1.0f / sqrtf(tot / (float)VT_DIM + VT_EPS);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const float g = a.norm[t + 1024 * j];
        s_xn[0][t + 1024 * j] = __fmul_rn(__fmul_rn(v[0][j], s_inv[0]), g);
        s_xn[1][t + 1024 * j] = __fmul_rn(__fmul_rn(v[1][j], s_inv[1]), g);
    }
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < VT_DIM / 512; i++) {
        const int c = 8 * (lane + 64 * i);
        const f32x4 xa = *reinterpret_cast<const f32x4 *>(&s_xn[ob][c]);
        const f32x4 xb = *reinterpret_cast<const f32x4 *>(&s_xn[ob][c + 4]);
        acc = vt_dot8(w[i], xa, xb, acc);
    }
    acc = vt_wave_sum(acc);
    if (mine && lane == 0) a.vel[o] = acc;
}

__global__ void __launch_bounds__(1024)
vt_ac_edge_front_kernel(ac_edge_args a) {
    __shared__ float s_vel[2 * VT_AC_DIM_IN];
    __shared__ float s_x[VT_AC_DIM_IN];
    const int t = (int)threadIdx.x;
    const int c = t + 1024 * (int)blockIdx.x;            /* this thread's token column */
    /* the column's row of the input projection does not depend on the latent: requested first */
    u32x2 wr[VT_AC_DIM_IN / 4];
    if (a.do_front) {
        const u32x2 *p = reinterpret_cast<const u32x2 *>(a.input_proj + (size_t)c * VT_AC_DIM_IN);
#pragma unroll
        for (int k4 = 0; k4 < VT_AC_DIM_IN / 4; k4++) wr[k4] = p[k4];
    }
    if (t < VT_AC_DIM_IN) s_x[t] = a.x_in[t];
    if (a.do_euler && t < 2 * VT_AC_DIM_IN) s_vel[t] = a.vel[t];
    __syncthreads();
    if (t < VT_AC_DIM_IN) {
        float xn = s_x[t];
        if (a.do_euler) {
            /* x += (1.2*vc + (1-1.2)*vu) * dt, each product rounded (voxtral_tts_acoustic.c:350-354) */
            const float p = __fmul_rn(1.2f, s_vel[t]);
            const float q = __fmul_rn(1.0f - 1.2f, s_vel[VT_AC_DIM_IN + t]);
            xn = __fadd_rn(xn, __fmul_rn(__fadd_rn(p, q), a.dt));
        }
        s_x[t] = xn;
        if (blockIdx.x == 0) {
            a.x_out[t] = xn;
            if (a.do_fsq) {
                /* voxtral_tts_acoustic.c:358-372 */
                float v = xn;
                if (v > 1.0f) v = 1.0f;
                if (v < -1.0f) v = -1.0f;
                const float scaled = __fmul_rn(__fdiv_rn(__fadd_rn(v, 1.0f), 2.0f), 20.0f);
                int q = (int)__fadd_rn(scaled, 0.5f);
                if (q < 0) q = 0;
                if (q > 20) q = 20;
                a.codes[t + 1] = q + 2;
            }
        }
    }
    __syncthreads();
    if (a.do_front) {
        /* tokens of both branches: [noise, time, llm] and [noise, time, 0]; the noise token is
         * the 36-term input projection in the CPU order (voxtral_tts_kernels.c:152-185) */
        float acc = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < VT_AC_DIM_IN / 4; k4++) {
            const u32x2 w = wr[k4];
            acc = __fadd_rn(acc, __fmul_rn(vt_bf16_lo(w.x), s_x[4 * k4]));
            acc = __fadd_rn(acc, __fmul_rn(vt_bf16_hi(w.x), s_x[4 * k4 + 1]));
            acc = __fadd_rn(acc, __fmul_rn(vt_bf16_lo(w.y), s_x[4 * k4 + 2]));
            acc = __fadd_rn(acc, __fmul_rn(vt_bf16_hi(w.y), s_x[4 * k4 + 3]));
        }
        const float tm = a.time_tok[c];
        a.tok_out[c] = acc;
        a.tok_out[VT_DIM + c] = tm;
        a.tok_out[2 * VT_DIM + c] = a.llm_tok[c];
        a.tok_out[3 * VT_DIM + c] = acc;
        a.tok_out[4 * VT_DIM + c] = tm;
        a.tok_out[5 * VT_DIM + c] = 0.f;
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
    float *tok, *qkv, *h, *llm_tok, *hidden, *x, *x2, *vel, *temb, *time_tok1, *logits;
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
    w->x2 = w->vel + 80;                                 /* vel uses 72 of its 128 floats */
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
    const int n_units = n_rows / AC_RB;
    const int most = g_vt.ac_grid > 0 && g_vt.ac_grid < g_vt.n_cu ? g_vt.ac_grid : g_vt.n_cu;
    const int grid = n_units < most ? n_units : most;
    hipLaunchKernelGGL(vt_ac_phase_kernel<PH>, dim3(grid), dim3(AC_THREADS), lds, g_vt.stream, a, n_units);
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

/* For other translation units of the library: the four phase launches of acoustic layer `layer` on
 * the work area (phase 0..3 = that launch alone, 4 = all four in order), and the work area itself. */
int vt_ac_launch_layer_phase(int layer, int phase) {
    if (!g_vt.initialized || !g_vt.ac_uploaded) { vt_set_error("acoustic weights not uploaded"); return -1; }
    float *base = (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
    if (!base || layer < 0 || layer >= TTS_HIP_AC_LAYERS) return -1;
    ac_work w;
    carve(&w, base);
    const vt_layer_dev *L = &g_vt.ac.layers[layer];
    int r = 0;
    if (phase == AC_QKV || phase == 4) r |= launch_phase<AC_QKV>(L->wqkv, w.tok, L->attn_norm, w.qkv, VT_QKV_DIM);
    if (phase == AC_WO || phase == 4) r |= launch_phase<AC_WO>(L->wo, w.qkv, NULL, w.tok, VT_DIM);
    if (phase == AC_W13 || phase == 4) r |= launch_phase<AC_W13>(L->w13, w.tok, L->ffn_norm, w.h, 2 * VT_FFN);
    if (phase == AC_W2 || phase == 4) r |= launch_phase<AC_W2>(L->w2, w.h, NULL, w.tok, VT_DIM);
    return r;
}

float *vt_ac_work_area(size_t *n_floats) {
    *n_floats = AC_WORK_FLOATS;
    return (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
}

/* One step boundary.  The latent ping-pongs between w->x and w->x2: `flip` counts the front
 * launches of the frame so far; the caller keeps it. */
static void launch_edge(const ac_work *w, const float *time_tok, const float *llm_tok, float dt, int back, int euler,
                        int front, int fsq, int *flip) {
    const vt_acoustic_dev *ac = &g_vt.ac;
    ac_edge_args a;
    a.tok_in = w->tok; a.tok_out = w->tok; a.norm = ac->norm; a.acoustic_out = ac->acoustic_out;
    a.input_proj = ac->input_proj; a.time_tok = time_tok; a.llm_tok = llm_tok; a.vel = w->vel;
    a.codes = w->codes; a.dt = dt; a.do_euler = euler; a.do_front = front; a.do_fsq = fsq;
    a.x_in = (*flip & 1) ? w->x2 : w->x;
    a.x_out = (*flip & 1) ? w->x : w->x2;
    if (back) hipLaunchKernelGGL(vt_ac_edge_back_kernel, dim3(AC_BACK_WGS), dim3(1024), 0, g_vt.stream, a);
    if (euler || front || fsq) {
        hipLaunchKernelGGL(vt_ac_edge_front_kernel, dim3(front ? AC_FRONT_WGS : 1), dim3(1024), 0, g_vt.stream, a);
        *flip += 1;
    }
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

/* The reference asks for one velocity at a time (voxtral_tts_acoustic.c:345-348): first with
 * the LLM hidden state, then with a zero one, for the same latent and time, 7 times per frame
 * with the same hidden state and on a fixed time grid.  A pass here always computes both
 * branches, so the host side remembers what such a caller will ask for next:
 *   - the unconditional velocity of the last (latent, time),
 *   - the projected LLM token of the last hidden state,
 *   - the projected time tokens of the grid t = i/7.
 * All of it is dropped when weights are uploaded (time_tok_ready == 0). */
static struct {
    int uncond_valid, hidden_valid;
    float x[VT_AC_DIM_IN], t, vu[VT_AC_DIM_IN];
    float hidden[VT_DIM];
} s_memo;

static int ensure_time_grid(float *d_temb) {
    vt_acoustic_dev *ac = &g_vt.ac;
    if (ac->time_tok_ready) return 0;
    float ts[AC_STEPS];
    for (int i = 0; i < AC_STEPS; i++) ts[i] = (float)i / (float)AC_STEPS;
    if (project_times(ac->time_tok, d_temb, ts, AC_STEPS)) return -1;
    ac->time_tok_ready = 1;
    s_memo.uncond_valid = s_memo.hidden_valid = 0;
    return 0;
}

static void predict(float *out_c, float *out_u, const float *x_t, const float *llm_hidden, float t_val) {
    float *base = (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
    if (!base) return;
    ac_work w;
    carve(&w, base);
    hipStream_t st = g_vt.stream;
    vt_acoustic_dev *ac = &g_vt.ac;
    if (ensure_time_grid(w.temb)) return;
    int zero_hidden = 1;
    for (int i = 0; i < VT_DIM && zero_hidden; i++) zero_hidden = llm_hidden[i] == 0.0f;
    if (!out_u && zero_hidden && s_memo.uncond_valid && s_memo.t == t_val &&
        memcmp(s_memo.x, x_t, sizeof s_memo.x) == 0) {
        memcpy(out_c, s_memo.vu, sizeof s_memo.vu);
        return;
    }
    /* time token: from the grid when t is a grid point, else projected now */
    const float *time_tok = w.time_tok1;
    int on_grid = 0;
    for (int i = 0; i < AC_STEPS && !on_grid; i++)
        if (t_val == (float)i / (float)AC_STEPS) { time_tok = ac->time_tok + (size_t)i * VT_DIM; on_grid = 1; }
    if (!on_grid && project_times(w.time_tok1, w.temb, &t_val, 1)) return;
    /* LLM token: row AC_STEPS of the token cache */
    float *llm_tok = ac->time_tok + (size_t)AC_STEPS * VT_DIM;
    if (!s_memo.hidden_valid || memcmp(s_memo.hidden, llm_hidden, sizeof s_memo.hidden) != 0) {
        VT_TRYV(hipStreamSynchronize(st));
        memcpy(g_vt.h_pin, llm_hidden, sizeof(float) * VT_DIM);
        VT_TRYV(hipMemcpyAsync(w.hidden, g_vt.h_pin, sizeof(float) * VT_DIM, hipMemcpyHostToDevice, st));
        vt_launch_linear(llm_tok, w.hidden, ac->llm_proj, NULL, 1, VT_DIM, VT_DIM);
        memcpy(s_memo.hidden, llm_hidden, sizeof s_memo.hidden);
        s_memo.hidden_valid = 1;
    }
    VT_TRYV(hipMemcpyAsync(w.x, x_t, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault, st));
    int flip = 0;
    launch_edge(&w, time_tok, llm_tok, 0.f, 0, 0, 1, 0, &flip);
    if (run_layers(&w)) return;
    launch_edge(&w, time_tok, llm_tok, 0.f, 1, 0, 0, 0, &flip);
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    float vel[2 * VT_AC_DIM_IN];
    VT_TRYV(hipMemcpy(vel, w.vel, sizeof vel, hipMemcpyDeviceToHost));
    memcpy(out_c, vel, sizeof(float) * VT_AC_DIM_IN);
    if (out_u) memcpy(out_u, vel + VT_AC_DIM_IN, sizeof(float) * VT_AC_DIM_IN);
    memcpy(s_memo.x, x_t, sizeof s_memo.x);
    memcpy(s_memo.vu, vel + VT_AC_DIM_IN, sizeof s_memo.vu);
    s_memo.t = t_val;
    s_memo.uncond_valid = 1;
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

/* Enqueues one frame: semantic head + argmax, 7 guided Euler steps, FSQ.  d_or_h_hidden may
 * be a host or a device pointer.  Codes end up in w->codes, the latent in w->x; nothing is
 * synchronised. */
static int enqueue_frame(ac_work *w, const float *d_or_h_hidden, const float *x0) {
    hipStream_t st = g_vt.stream;
    vt_acoustic_dev *ac = &g_vt.ac;
    float *base = (float *)vt_scratch(sizeof(float) * AC_WORK_FLOATS);
    if (!base) return -1;
    carve(w, base);
    float ts[AC_STEPS + 1];
    for (int i = 0; i <= AC_STEPS; i++) ts[i] = (float)i / (float)AC_STEPS;
    if (ensure_time_grid(w->temb)) return -1;            /* the projected time tokens depend on the weights only */
    if (vt_check(hipMemcpyAsync(w->hidden, d_or_h_hidden, sizeof(float) * VT_DIM, hipMemcpyDefault, st), "frame hidden")) return -1;
    if (vt_check(hipMemcpyAsync(w->x, x0, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDefault, st), "frame noise")) return -1;
    vt_launch_linear(w->logits, w->hidden, ac->semantic_out, ac->semantic_bias, 1, VT_DIM, VT_SEM_PADDED);
    hipLaunchKernelGGL(vt_semantic_argmax_kernel, dim3(1), dim3(1024), 0, st, w->logits, w->codes);
    vt_launch_linear(w->llm_tok, w->hidden, ac->llm_proj, NULL, 1, VT_DIM, VT_DIM);
    /* the flow runs without waiting for the semantic code; an END_AUDIO frame discards it */
    int flip = 0;                                        /* 1 + AC_STEPS front launches: the latent ends in w->x */
    launch_edge(w, ac->time_tok, w->llm_tok, 0.f, 0, 0, 1, 0, &flip);
    for (int s = 0; s < AC_STEPS; s++) {
        volatile float dt = ts[s + 1] - ts[s];
        if (run_layers(w)) return -1;
        const int last = s + 1 == AC_STEPS;
        launch_edge(w, ac->time_tok + (size_t)(last ? s : s + 1) * VT_DIM, w->llm_tok, (float)dt, 1, 1, !last, last, &flip);
    }
    return vt_check(hipGetLastError(), "frame launch");
}

static void finish_frame(const ac_work *w, int *out_codes, float *out_x) {
    /* codes, latent and the backbone step's "gave up" word come back through pinned memory behind ONE wait
     * (three blocking copies were 1 % of a turn of the generation loop) */
    hipStream_t st = g_vt.stream;
    int *pin_codes = (int *)g_vt.h_pin, *pin_flag = (int *)(g_vt.h_pin + 128);
    float *pin_x = g_vt.h_pin + 64;
    VT_TRYV(hipMemcpyAsync(pin_codes, w->codes, sizeof(int) * (1 + VT_AC_DIM_IN), hipMemcpyDeviceToHost, st));
    VT_TRYV(hipMemcpyAsync(pin_x, w->x, sizeof(float) * VT_AC_DIM_IN, hipMemcpyDeviceToHost, st));
    VT_TRYV(hipMemcpyAsync(pin_flag, g_vt.d_abort, sizeof(int), hipMemcpyDeviceToHost, st));
    VT_TRYV(hipStreamSynchronize(st));
    if (g_vt.step_pending) {                /* the backbone step in front of this frame: was it abandoned? */
        g_vt.step_pending = 0;
        if (pin_flag[0]) { (void)vt_step_poll_abort_now(); return; }
    }
    memcpy(out_codes, pin_codes, sizeof(int) * (1 + VT_AC_DIM_IN));
    if (out_x) memcpy(out_x, pin_x, sizeof(float) * VT_AC_DIM_IN);
    if (out_codes[0] == 1) {                            /* END_AUDIO */
        for (int i = 1; i <= VT_AC_DIM_IN; i++) out_codes[i] = 2;
        if (out_x) memset(out_x, 0, sizeof(float) * VT_AC_DIM_IN);
    }
}

extern "C" void tts_hip_acoustic_frame(int *out_codes, const float *llm_hidden, const float *x0,
                                       float *out_x) {
    if (!ac_ready("tts_hip_acoustic_frame")) return;
    ac_work w;
    if (enqueue_frame(&w, llm_hidden, x0)) return;
    finish_frame(&w, out_codes, out_x);
}

/* ---- audio-code embedding and the per-frame loop -------------------------------------- */

/* out[i] = sum over the 37 codebooks, in codebook order, of row offsets[cb] + codes[cb] of the
 * bf16 table, starting from 0 (tts_audio_embed_forward, voxtral_tts_voice.c:292-315): the same
 * fp32 additions in the same order, so the result is bit-equal to the CPU's. */
__global__ void vt_audio_embed_kernel(float *out, const uint16_t *emb, const int *offsets, const int *codes,
                                      int total_rows) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i >= VT_DIM) return;
    float acc = 0.0f;
    for (int cb = 0; cb < 1 + VT_AC_DIM_IN; cb++) {
        int row = offsets[cb] + codes[cb];
        row = row < 0 ? 0 : (row >= total_rows ? total_rows - 1 : row);
        acc = __fadd_rn(acc, __uint_as_float((unsigned)emb[(size_t)row * VT_DIM + i] << 16));
    }
    out[i] = acc;
}

extern "C" int tts_hip_upload_audio_embeddings(const uint16_t *emb_bf16, int total_rows, const int *offsets) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_upload_audio_embeddings: backend not initialised"); return -1; }
    if (!emb_bf16 || !offsets || total_rows < 1) { vt_set_error("tts_hip_upload_audio_embeddings: bad arguments"); return -1; }
    vt_acoustic_dev *ac = &g_vt.ac;
    VT_TRY(hipStreamSynchronize(g_vt.stream));
    if (ac->audio_emb) (void)hipFree(ac->audio_emb);
    if (ac->audio_offsets) (void)hipFree(ac->audio_offsets);
    ac->audio_emb = NULL;
    ac->audio_offsets = NULL;
    ac->audio_rows = 0;
    const size_t bytes = (size_t)total_rows * VT_DIM * 2;
    if (!(ac->audio_emb = (uint16_t *)vt_dev_alloc(bytes))) return -1;
    if (!(ac->audio_offsets = (int *)vt_dev_alloc(sizeof(int) * 2 * (1 + VT_AC_DIM_IN)))) return -1;
    VT_TRY(hipMemcpy(ac->audio_emb, emb_bf16, bytes, hipMemcpyDefault));
    VT_TRY(hipMemcpy(ac->audio_offsets, offsets, sizeof(int) * (1 + VT_AC_DIM_IN), hipMemcpyDefault));
    ac->audio_rows = total_rows;
    return 0;
}

static int embed_ready(const char *who) {
    if (g_vt.initialized && g_vt.ac.audio_rows > 0) return 1;
    vt_set_error("%s: audio embeddings not uploaded", who);
    return 0;
}

/* host codes [37] -> host embedding [3072]; synchronous */
extern "C" void tts_hip_audio_embed(float *out_embed, const int *codes) {
    if (!embed_ready("tts_hip_audio_embed")) return;
    vt_acoustic_dev *ac = &g_vt.ac;
    hipStream_t st = g_vt.stream;
    int *d_codes = ac->audio_offsets + (1 + VT_AC_DIM_IN);
    VT_TRYV(hipStreamSynchronize(st));
    VT_TRYV(hipMemcpy(d_codes, codes, sizeof(int) * (1 + VT_AC_DIM_IN), hipMemcpyHostToDevice));
    hipLaunchKernelGGL(vt_audio_embed_kernel, dim3(VT_DIM / 256), dim3(256), 0, st, g_vt.d_embed, ac->audio_emb,
                       ac->audio_offsets, d_codes, ac->audio_rows);
    VT_TRYV(hipStreamSynchronize(st));
    VT_TRYV(hipMemcpy(out_embed, g_vt.d_embed, sizeof(float) * VT_DIM, hipMemcpyDeviceToHost));
}

/* One turn of the generation loop (voxtral_tts.c:301-321) without leaving the device in
 * between: backbone step at cache position pos on d_embed -> hidden -> frame of 37 codes ->
 * embedding of those codes back into d_embed.  x0 is the frame's noise (host, 36 floats: the
 * caller keeps the RNG).  Returns the codes; after an END_AUDIO frame d_embed is not meaningful. */
extern "C" void tts_hip_generate_frame(int *out_codes, float *d_embed, const float *x0, int pos) {
    if (!ac_ready("tts_hip_generate_frame") || !embed_ready("tts_hip_generate_frame")) return;
    if (g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_generate_frame: no backbone weights uploaded"); return; }
    if (vt_run_step(g_vt.d_layers, g_vt.n_dec_layers, 0, g_vt.d_dec_norm, d_embed, g_vt.d_hidden, pos)) return;
    ac_work w;
    if (enqueue_frame(&w, g_vt.d_hidden, x0)) return;
    vt_acoustic_dev *ac = &g_vt.ac;
    hipLaunchKernelGGL(vt_audio_embed_kernel, dim3(VT_DIM / 256), dim3(256), 0, g_vt.stream, d_embed, ac->audio_emb,
                       ac->audio_offsets, w.codes, ac->audio_rows);
    finish_frame(&w, out_codes, NULL);
}
