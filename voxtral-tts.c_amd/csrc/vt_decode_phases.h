/*
 * vt_decode_phases.h - the five phases of one decoder layer at batch 1, as
 * device functions shared by the per-phase kernels and by the persistent
 * whole-step kernel.
 *
 * Every GEMV phase streams bf16 weight rows with 16-byte non-temporal loads:
 * a wave owns whole rows (or a fixed k-range of rows), each lane keeps its
 * slice of the activation vector in registers (lane l holds elements
 * c*512 + l*8 .. +8 of every 512-element chunk c), products are accumulated
 * with fp32 FMA per lane and summed across the wave in a fixed DPP order.
 * Rows are kept in a ring of D row buffers, so D rows of loads are in flight
 * per wave; the first D rows of a phase can be requested before the grid
 * barrier that precedes the phase (weights do not depend on activations).
 *
 * The small vectors that one phase hands to the next (residual stream, q,
 * attention output, SwiGLU output, the appended K/V row, attention partials)
 * cross workgroups and therefore XCDs: they are written through to memory
 * (vt_stc) and read past the L2 (vt_ldc / vt_stage), once per workgroup into
 * LDS, from where every wave takes its register slice.
 *
 * Operation order follows the reference CPU decode step
 * (voxtral_tts_llm.c:205-264): RMSNorm -> q,k,v -> RoPE -> cache append ->
 * attention -> wo + residual -> RMSNorm -> w1,w3 -> SiLU*up -> w2 + residual.
 */
#ifndef VT_DECODE_PHASES_H
#define VT_DECODE_PHASES_H

#include "vt_device.h"

#define VT_RING 18            /* 16-byte buffers per lane in the row ring */
#define VT_ATT_STRIDE 132     /* floats per attention partial: m, l, pad, pad, o[128] */
#ifndef VT_ATT_MIN_CHUNK
#define VT_ATT_MIN_CHUNK 64   /* positions per attention workgroup before the cache is split further */
#endif
#define VT_LDS_X 9216         /* staged activation vector (largest: the SwiGLU output) */
#define VT_LDS_Y 512          /* row results of one workgroup */
#define VT_LDS_FLOATS (VT_LDS_X + VT_LDS_Y)

/* Device-side weights of one layer, laid out at upload:
 *   wqkv = [wq ; wk ; wv]            [6144, 3072]
 *   w13  = rows interleaved (w1 row j, w3 row j)   [18432, 3072]     */
struct vt_layer_dev {
    const uint16_t *wqkv;
    const uint16_t *wo;
    const uint16_t *w13;
    const uint16_t *w2;
    const float *attn_norm;
    const float *ffn_norm;
};

struct vt_step_args {
    const vt_layer_dev *layers;
    int n_layers;
    int first_layer;              /* global index of layers[0] in the KV cache */
    const float *final_norm;      /* NULL: skip the final RMSNorm */
    float *kv_k, *kv_v;           /* f32 [layers, kv_max, 1024] */
    int kv_max;
    int pos;
    const float *rope;            /* f32 [kv_max, 64, 2] (cos, sin) */
    const float *in_embed;        /* f32 [3072] */
    float *out_hidden;            /* f32 [3072] */
    float *x;                     /* residual stream */
    float *q, *attn, *h;          /* [4096], [4096], [9216] */
    float *att_part;              /* [32 heads, n_chunks, VT_ATT_STRIDE] */
    unsigned int *att_cnt;        /* [n_layers * 8], zero at phase start */
};

/* ---- activation vectors: memory -> LDS -> register slices ------------------- */

/* Coherent 16-byte load (device scope: served past this XCD's L2). */
__device__ __forceinline__ f32x4 vt_ldc4(const float *base, int idx4, int n_floats) {
    __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, n_floats * 4, 0x00020000);
    u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, idx4 * 16, 0, 16 /* sc1 */);
    f32x4 f;
    f.x = __uint_as_float(v.x); f.y = __uint_as_float(v.y);
    f.z = __uint_as_float(v.z); f.w = __uint_as_float(v.w);
    return f;
}

/* The whole workgroup copies n floats (n % 4 == 0) of a handed-over vector into LDS. */
__device__ __forceinline__ void vt_stage(float *lds_x, const float *src, int n) {
    f32x4 *dst = reinterpret_cast<f32x4 *>(lds_x);
    for (int i = (int)threadIdx.x; i < n / 4; i += (int)blockDim.x) dst[i] = vt_ldc4(src, i, n);
    __syncthreads();
}

template <int NK>
__device__ __forceinline__ void vt_slice_lds(f32x4 (&xa)[NK], f32x4 (&xb)[NK], const float *lds_x, int kofs) {
    const int lane = vt_lane();
#pragma unroll
    for (int c = 0; c < NK; c++) {
        const f32x4 *p = reinterpret_cast<const f32x4 *>(lds_x + kofs + c * 512 + lane * 8);
        xa[c] = p[0];
        xb[c] = p[1];
    }
}

template <int NK>
__device__ __forceinline__ void vt_slice_global(f32x4 (&xa)[NK], f32x4 (&xb)[NK], const float *x, int kofs) {
    const int lane = vt_lane();
#pragma unroll
    for (int c = 0; c < NK; c++) {
        const f32x4 *p = reinterpret_cast<const f32x4 *>(x + kofs + c * 512 + lane * 8);
        xa[c] = p[0];
        xb[c] = p[1];
    }
}

/* RMSNorm of the staged 3072-vector, every wave for itself (NK = 6 covers it):
 * out = (x * 1/sqrt(mean(x^2)+eps)) * w  (voxtral_tts_kernels.c:333-349). */
__device__ __forceinline__ void vt_rmsnorm_slice(f32x4 (&xa)[6], f32x4 (&xb)[6],
                                                 const float *lds_x, const float *w) {
    f32x4 wa[6], wb[6];
    vt_slice_global<6>(wa, wb, w, 0);
    vt_slice_lds<6>(xa, xb, lds_x, 0);
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 6; c++) {
        ss = fmaf(xa[c].x, xa[c].x, ss); ss = fmaf(xa[c].y, xa[c].y, ss);
        ss = fmaf(xa[c].z, xa[c].z, ss); ss = fmaf(xa[c].w, xa[c].w, ss);
        ss = fmaf(xb[c].x, xb[c].x, ss); ss = fmaf(xb[c].y, xb[c].y, ss);
        ss = fmaf(xb[c].z, xb[c].z, ss); ss = fmaf(xb[c].w, xb[c].w, ss);
    }
    ss = vt_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)VT_DIM + VT_EPS);
#pragma unroll
    for (int c = 0; c < 6; c++) {
        xa[c] = (xa[c] * inv) * wa[c];
        xb[c] = (xb[c] * inv) * wb[c];
    }
}

/* ---- row ring ------------------------------------------------------------- */

/* Which rows of a phase a wave owns. */
struct vt_rows {
    int r0;        /* first global row of this wave (k-range [kofs, kofs+NK*512)) */
    int nr;        /* rows owned by this wave (may be 0) */
    int kofs;
    int wg_row0;   /* first global row of the workgroup */
    int wg_nrows;
    int part;      /* k-split index of this wave */
};

/* Split `n_rows` rows over the grid (contiguous blocks, `align` rows granularity)
 * and over the waves of the workgroup; KS waves share a row and split K. */
template <int KS>
__device__ __forceinline__ vt_rows vt_split_rows(int n_rows, int align, int k_per_part) {
    vt_rows r;
    const int G = (int)gridDim.x, wg = (int)blockIdx.x;
    const int nw = (int)(blockDim.x >> 6), wave = vt_wave();
    const int per_wg = vt_rows_per_wg(n_rows, align, G);
    r.wg_row0 = wg * per_wg;
    int nrows = n_rows - r.wg_row0;
    nrows = nrows < 0 ? 0 : (nrows > per_wg ? per_wg : nrows);
    r.wg_nrows = nrows;
    const int groups = nw / KS;
    const int grp = wave / KS;
    r.part = wave % KS;
    const int per_grp = (nrows + groups - 1) / groups;
    int g0 = grp * per_grp;
    int gn = nrows - g0;
    gn = gn < 0 ? 0 : (gn > per_grp ? per_grp : gn);
    r.r0 = r.wg_row0 + g0;
    r.nr = gn;
    r.kofs = r.part * k_per_part;
    return r;
}

/* Request the first D rows of a wave's share.  The persistent kernel asks for the first
 * VT_HEAD_SLOTS slots as soon as the previous phase has multiplied its ring out (PART_HEAD)
 * and for the others after it has handed its results over (PART_TAIL): 6 KB per wave is
 * 48 KB per CU, about what a CU accepts as outstanding loads; more would hold up the
 * acknowledgement of the hand-over stores that the barrier waits for. */
enum { VT_PART_ALL = 0, VT_PART_HEAD = 1, VT_PART_TAIL = 2 };
#ifndef VT_HEAD_SLOTS
#define VT_HEAD_SLOTS 5        /* ring slots (KB per wave) requested ahead of the hand-over (4 / 5 / 6 / 7 / 8: 1.200 / 1.190 / 1.194 / 1.200 / 1.222 ms/frame) */
#endif

/* Only the ring slots [slot_lo, slot_hi) are requested: the output projection leaves the last 6
 * slots of the ring unused, so the gate|up rows that live there are requested a phase early. */
template <int NK, int D>
__device__ __forceinline__ void vt_ring_prefetch(u32x4 (&ring)[VT_RING], const uint16_t *W,
                                                 int row_len, const vt_rows &r, int part = VT_PART_ALL,
                                                 int slot_lo = 0, int slot_hi = VT_RING) {
    static_assert(NK * D <= VT_RING, "ring too small");
    const uint16_t *base = W + (size_t)r.r0 * row_len + r.kofs + vt_lane() * 8;
#pragma unroll
    for (int j = 0; j < D; j++) {
        if (j < r.nr) {
#pragma unroll
            for (int c = 0; c < NK; c++) {
                const int slot = j * NK + c;
                const bool head = slot - slot_lo < VT_HEAD_SLOTS;
                if (slot >= slot_lo && slot < slot_hi && (part == VT_PART_ALL || (part == VT_PART_HEAD) == head))
                    ring[slot] = vt_ldw(base + (size_t)j * row_len + c * 512);
            }
        }
    }
}

/* Consume the wave's rows: y_lds[part * wg_nrows + local_row] = partial dot.
 *
 * The compiler counts outstanding loads statically: behind a load that is issued under a
 * condition it has to wait as if that load were not there, i.e. for everything.  With the row
 * count as a template parameter the loop below unrolls into straight-line code in which every
 * request is unconditional, and each row then waits for exactly the loads older than its own:
 * the D - 1 younger rows stay in flight while it is multiplied.  The scheduling barriers keep a
 * row's requests where they are written, behind the last use of the registers they overwrite. */
template <int NK, int D, int NR>
__device__ __forceinline__ void vt_ring_run_fixed(u32x4 (&ring)[VT_RING], const uint16_t *W,
                                                  int row_len, const vt_rows &r,
                                                  const f32x4 (&xa)[NK], const f32x4 (&xb)[NK],
                                                  float *y_lds) {
    const uint16_t *base = W + (size_t)r.r0 * row_len + r.kofs + vt_lane() * 8;
    float *y = y_lds + r.part * r.wg_nrows + (r.r0 - r.wg_row0);
#pragma unroll
    for (int row = 0; row < NR; row++) {
        const int j = row % D;
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int c = 0; c < NK; c += 2) {
            a0 = vt_dot8(ring[j * NK + c], xa[c], xb[c], a0);
            if (c + 1 < NK) a1 = vt_dot8(ring[j * NK + c + 1], xa[c + 1], xb[c + 1], a1);
        }
        if (row + D < NR) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < NK; c++)
                ring[j * NK + c] = vt_ldw(base + (size_t)(row + D) * row_len + c * 512);
            __builtin_amdgcn_sched_barrier(0);
        }
        const float s = vt_wave_sum(a0 + a1);
        if (vt_lane() == 0) y[row] = s;
    }
}

/* Any row count: rows and requests under run-time conditions (see above for what that costs). */
template <int NK, int D>
__device__ __forceinline__ void vt_ring_run_any(u32x4 (&ring)[VT_RING], const uint16_t *W,
                                                int row_len, const vt_rows &r,
                                                const f32x4 (&xa)[NK], const f32x4 (&xb)[NK],
                                                float *y_lds) {
    const uint16_t *base = W + (size_t)r.r0 * row_len + r.kofs + vt_lane() * 8;
    float *y = y_lds + r.part * r.wg_nrows + (r.r0 - r.wg_row0);
    for (int i = 0; i < r.nr; i += D) {
#pragma unroll
        for (int j = 0; j < D; j++) {
            const int row = i + j;
            if (row < r.nr) {
                float a0 = 0.f, a1 = 0.f;
#pragma unroll
                for (int c = 0; c < NK; c += 2) {
                    a0 = vt_dot8(ring[j * NK + c], xa[c], xb[c], a0);
                    if (c + 1 < NK) a1 = vt_dot8(ring[j * NK + c + 1], xa[c + 1], xb[c + 1], a1);
                }
                if (row + D < r.nr) {
#pragma unroll
                    for (int c = 0; c < NK; c++)
                        ring[j * NK + c] = vt_ldw(base + (size_t)(row + D) * row_len + c * 512);
                }
                const float s = vt_wave_sum(a0 + a1);
                if (vt_lane() == 0) y[row] = s;
            }
        }
    }
}

/* NR: the row count of a wave on a 256-workgroup grid, where the straight-line version runs. */
template <int NK, int D, int NR>
__device__ __forceinline__ void vt_ring_run(u32x4 (&ring)[VT_RING], const uint16_t *W,
                                            int row_len, const vt_rows &r,
                                            const f32x4 (&xa)[NK], const f32x4 (&xb)[NK],
                                            float *y_lds) {
    if (r.nr == NR) vt_ring_run_fixed<NK, D, NR>(ring, W, row_len, r, xa, xb, y_lds);
    else vt_ring_run_any<NK, D>(ring, W, row_len, r, xa, xb, y_lds);
}

/* ---- phase 1: RMSNorm + [wq;wk;wv] + RoPE + cache append ------------------ */

__device__ __forceinline__ vt_rows vt_qkv_rows() { return vt_split_rows<1>(VT_QKV_DIM, VT_QKV_ALIGN, 0); }

__device__ __forceinline__ void vt_qkv_prefetch(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                                int part = VT_PART_ALL) {
    vt_ring_prefetch<6, 3>(ring, L.wqkv, VT_DIM, vt_qkv_rows(), part);
}

struct vt_nothing { __device__ __forceinline__ void operator()() const {} };

/* `after_run` is called when the ring has been multiplied out and is free again, before the
 * results are stored. */
template <class AR = vt_nothing>
__device__ __forceinline__ void vt_qkv_body(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                            const vt_step_args &a, int layer,
                                            const float *x_in, float *lds, AR after_run = AR()) {
    const vt_rows r = vt_qkv_rows();
    float *lds_y = lds + VT_LDS_X;
    vt_stage(lds, x_in, VT_DIM);
    f32x4 xa[6], xb[6];
    vt_rmsnorm_slice(xa, xb, lds, L.attn_norm);
    vt_ring_run<6, 3, 3>(ring, L.wqkv, VT_DIM, r, xa, xb, lds_y);
    after_run();
    __syncthreads();
    /* RoPE on adjacent pairs (voxtral_tts_kernels.c:616-634), then q to its
     * buffer and k, v straight into row `pos` of the cache. */
    const float *cs = a.rope + (size_t)a.pos * VT_HEAD_DIM;
    const size_t kv_row = ((size_t)(a.first_layer + layer) * a.kv_max + a.pos) * VT_KV_DIM;
    for (int t = (int)threadIdx.x; t < r.wg_nrows / 2; t += (int)blockDim.x) {
        const int g = r.wg_row0 + 2 * t;
        const float v0 = lds_y[2 * t], v1 = lds_y[2 * t + 1];
        if (g < VT_Q_DIM + VT_KV_DIM) {
            const int d = (g & (VT_HEAD_DIM - 1)) >> 1;
            const float c = cs[2 * d], s = cs[2 * d + 1];
            const float o0 = v0 * c - v1 * s;
            const float o1 = v0 * s + v1 * c;
            float *dst = g < VT_Q_DIM ? a.q + g : a.kv_k + kv_row + (g - VT_Q_DIM);
            vt_stc(dst, o0);
            vt_stc(dst + 1, o1);
        } else {
            float *dst = a.kv_v + kv_row + (g - VT_Q_DIM - VT_KV_DIM);
            vt_stc(dst, v0);
            vt_stc(dst + 1, v1);
        }
    }
}

/* ---- phase 2: GQA attention of one query over the cache ------------------- */
/* Workgroup = (kv head, chunk of positions); chunks hold at least
 * VT_ATT_MIN_CHUNK positions, so short caches use one workgroup per kv head
 * and need no cross-workgroup merge.  A wave walks its positions four at a
 * time (all K and V rows of a batch are requested before any is used); lanes
 * 16g..16g+15 serve query head 4*kvh+g and own 8 of the 128 dims.  Partials
 * (max, sum, o[128]) are merged over the waves in LDS; with several chunks
 * they are written per chunk and the last workgroup to finish a kv head
 * merges them and normalises (online-softmax algebra of
 * voxtral_tts_kernels.c:426-462). */
__device__ __forceinline__ void vt_attn_geometry(int n, int nch_max, int nw, int &cs, int &nch) {
    nch = (n + VT_ATT_MIN_CHUNK - 1) / VT_ATT_MIN_CHUNK;
    /* at most three quarters of the grid: the rest prefetches gate|up rows into L2 meanwhile */
    if (nch > nch_max * 3 / 4) nch = nch_max * 3 / 4;
    if (nch < 1) nch = 1;
    cs = (n + nch - 1) / nch;
    cs = (cs + nw - 1) / nw * nw;
    nch = (n + cs - 1) / cs;
}

/* Caches of fewer than VT_ATT_DIRECT_MAX positions: one workgroup per QUERY head (or several, each
 * with a share of the positions, see vt_attn_split), no merge by a last arriver and so no
 * store / counter / reload round trips inside the phase.
 * Lanes 16g..16g+15 of a wave serve position slot g and own 8 of the 128 dims, so a wave
 * works on 4 positions at once and the workgroup on 32; a batch of 4 such rounds (128
 * positions) has all its K and V rows requested before any is used.  Each of the 32 lane
 * groups keeps its own online-softmax state; they are merged through LDS at the end.  The
 * four workgroups of a kv head sit on one XCD (blockIdx % 8) and share its rows in that L2. */
#ifndef VT_ATT_DIRECT_MAX
#define VT_ATT_DIRECT_MAX 4096     /* measured up to 4000 positions: 1.470 against 1.621 ms/frame of the chunked schedule */
#endif

/* K and V rows of one batch: 4 rounds of one position per lane group */
struct vt_att_rows { f32x4 ka[4], kb[4], va[4], vb[4]; };

__device__ __forceinline__ bool vt_attn_is_direct(const vt_step_args &a) {
    return a.pos < VT_ATT_DIRECT_MAX && (int)gridDim.x >= VT_HEADS;
}

/* From a few hundred positions on, what the direct schedule costs is the K and V rows a query-head
 * workgroup pulls through its CU (1 KB per position).  The positions of a head are then dealt to 2
 * or 8 workgroups (every 2nd / 8th batch slot each); each leaves an un-normalised partial (max,
 * sum, o[128]) and the output projection combines them while it stages the vector, so the phase
 * still has no round trip of its own.  What a part costs is that combination (every workgroup of
 * the output projection reads all partials: 16 KB per part), and 8 parts take the whole grid, so
 * that no workgroup is left to prefetch gate|up rows into L2; on the other hand 8 parts cover 1024
 * positions in a single batch of requests.  Hence the thresholds (measured, ms/frame at 26 layers:
 * 2 parts 1.245 against 1.263 unsplit at 400 positions; 8 parts 1.264 against 1.274 with 2 parts at
 * 640 and 1.262 against 1.256 at 520; 4 parts were never the best: 1.274 at 640, 1.277 at 768 against
 * 1.267 with 8; 6 parts need two batches where 8 need one: 1.376 against 1.268 at 900). */
#ifndef VT_ATT_SPLIT2_MIN
#define VT_ATT_SPLIT2_MIN 384
#endif
#ifndef VT_ATT_SPLIT8_MIN
#define VT_ATT_SPLIT8_MIN 576
#endif
#define VT_ATT_SPLIT_MAX 8
__device__ __forceinline__ int vt_attn_split(const vt_step_args &a) {
    if (!vt_attn_is_direct(a)) return 1;
    const int G = (int)gridDim.x;
    if (a.pos >= VT_ATT_SPLIT8_MIN && G >= 8 * VT_HEADS && (G & 7) == 0) return 8;
    if (a.pos >= VT_ATT_SPLIT2_MIN && G >= 2 * VT_HEADS && (G & 7) == 0) return 2;
    return 1;
}

/* Requests the rows jb, jb + stride, ... of kv head kvh (clamped to `last`; rows beyond it are
 * loaded but never used). */
__device__ __forceinline__ void vt_attn_fetch(vt_att_rows &r, const vt_step_args &a, int layer, int kvh,
                                              int jb, int stride, int last) {
    const int sub = vt_lane() & 15;
    const size_t off = (size_t)(a.first_layer + layer) * a.kv_max * VT_KV_DIM + kvh * VT_HEAD_DIM + sub * 8;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int j = max(min(jb + u * stride, last), 0);
        const f32x4 *kp = reinterpret_cast<const f32x4 *>(a.kv_k + off + (size_t)j * VT_KV_DIM);
        const f32x4 *vp = reinterpret_cast<const f32x4 *>(a.kv_v + off + (size_t)j * VT_KV_DIM);
        r.ka[u] = kp[0]; r.kb[u] = kp[1];
        r.va[u] = vp[0]; r.vb[u] = vp[1];
    }
}

struct vt_att_state { float m, l; f32x4 oa, ob; };

__device__ __forceinline__ void vt_attn_step(vt_att_state &st, const f32x4 &qa, const f32x4 &qb, const f32x4 &ka,
                                             const f32x4 &kb, const f32x4 &va, const f32x4 &vb, float scale) {
    float s = qa.x * ka.x;
    s = fmaf(qa.y, ka.y, s); s = fmaf(qa.z, ka.z, s); s = fmaf(qa.w, ka.w, s);
    s = fmaf(qb.x, kb.x, s); s = fmaf(qb.y, kb.y, s); s = fmaf(qb.z, kb.z, s);
    s = fmaf(qb.w, kb.w, s);
    s = vt_row16_sum(s) * scale;
    const float mn = fmaxf(st.m, s);
    const float corr = __expf(st.m - mn), p = __expf(s - mn);
    st.l = fmaf(st.l, corr, p);
    st.oa = st.oa * corr + va * p;
    st.ob = st.ob * corr + vb * p;
    st.m = mn;
}

__device__ __forceinline__ void vt_attn_direct(const vt_step_args &a, int layer, float *lds) {
    const int wg = (int)blockIdx.x;
    const int NS = vt_attn_split(a);
    if (wg >= VT_HEADS * NS) return;
    int kvh, head, part_no;
    vt_attn_direct_map(wg, &kvh, &head, &part_no);
    const int nw = (int)(blockDim.x >> 6), wave = vt_wave(), lane = vt_lane();
    const int grp = lane >> 4, sub = lane & 15;
    const int slot = wave * 4 + grp, nslot = nw * 4;
    const int gslot = part_no * nslot + slot, gstride = nslot * NS;     /* slot and stride over all parts */
    const int n = a.pos + 1;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);
    const f32x4 qa = vt_ldc4(a.q, (head * VT_HEAD_DIM + sub * 8) / 4, VT_Q_DIM);
    const f32x4 qb = vt_ldc4(a.q, (head * VT_HEAD_DIM + sub * 8) / 4 + 1, VT_Q_DIM);
    vt_att_state st = {-1e30f, 0.f, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int jb = gslot; jb < n; jb += 4 * gstride) {
        vt_att_rows r;
        vt_attn_fetch(r, a, layer, kvh, jb, gstride, n - 1);
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (jb + u * gstride < n) vt_attn_step(st, qa, qb, r.ka[u], r.kb[u], r.va[u], r.vb[u], scale);
    }

    /* merge the lane groups of the workgroup: idle slots hold (m = -1e30, l = 0, o = 0) */
    float *mine = lds + slot * VT_ATT_STRIDE;                  /* [nslot][VT_ATT_STRIDE] */
    if (sub == 0) { mine[0] = st.m; mine[1] = st.l; }
    *reinterpret_cast<f32x4 *>(mine + 4 + sub * 8) = st.oa;
    *reinterpret_cast<f32x4 *>(mine + 8 + sub * 8) = st.ob;
    __syncthreads();
    float *wgt = lds + nslot * VT_ATT_STRIDE;                  /* [nslot] weights exp(m_s - M) */
    if (wave == 0) {
        const float ms = lane < nslot ? lds[lane * VT_ATT_STRIDE] : -1e30f;
        float M = vt_row16_max(ms);
        M = fmaxf(fmaxf(vt_readlane(M, 0), vt_readlane(M, 16)), fmaxf(vt_readlane(M, 32), vt_readlane(M, 48)));
        if (lane < nslot) wgt[lane] = __expf(ms - M);
        if (lane == 0) wgt[nslot] = M;
    }
    __syncthreads();
    const int d = (int)threadIdx.x;
    if (d < VT_HEAD_DIM) {
        float Ls = 0.f, O = 0.f;
        for (int w = 0; w < nslot; w++) {
            const float e = wgt[w];
            Ls = fmaf(lds[w * VT_ATT_STRIDE + 1], e, Ls);
            O = fmaf(lds[w * VT_ATT_STRIDE + 4 + d], e, O);
        }
        if (NS == 1) {
            vt_stc(a.attn + head * VT_HEAD_DIM + d, O * (1.0f / Ls));
        } else {
            /* a part without positions leaves (max -1e30, sum 0, o 0): weight 0 in the combination */
            float *dst = a.att_part + (size_t)(head * VT_ATT_SPLIT_MAX + part_no) * VT_ATT_STRIDE;
            if (d == 0) { vt_stc(dst, wgt[nslot]); vt_stc(dst + 1, Ls); }
            vt_stc(dst + 4 + d, O);
        }
    }
}

/* The i-th of the workgroups whose q|k|v rows attention workgroup `wg` of the direct schedule reads
 * (vt_rowsplit.h: the same row split as vt_qkv_rows(); at most 7 + 7 + 7 on 256 workgroups). */
__device__ __forceinline__ int vt_attn_producer(int wg, int i) { return vt_attn_producer_of((int)gridDim.x, wg, i); }

/* The output projection's input vector into LDS: the attention output as it stands, or the
 * combination of the NS partials per head the split schedule left (online-softmax algebra of
 * voxtral_tts_kernels.c:426-462, parts in ascending order). */
template <int NS>
__device__ __forceinline__ void vt_stage_attn_parts(float *lds_x, const vt_step_args &a) {
    f32x4 *dst = reinterpret_cast<f32x4 *>(lds_x);
    const int total = VT_HEADS * VT_ATT_SPLIT_MAX * VT_ATT_STRIDE;
    for (int i = (int)threadIdx.x; i < VT_Q_DIM / 4; i += (int)blockDim.x) {
        const int head = i >> 5, d4 = i & 31;
        const float *src = a.att_part + (size_t)head * VT_ATT_SPLIT_MAX * VT_ATT_STRIDE;
        float m[NS], l[NS];
        f32x4 o[NS];
#pragma unroll
        for (int c = 0; c < NS; c++) {
            m[c] = vt_ldc(src + c * VT_ATT_STRIDE);
            l[c] = vt_ldc(src + c * VT_ATT_STRIDE + 1);
            o[c] = vt_ldc4(a.att_part, (head * VT_ATT_SPLIT_MAX + c) * (VT_ATT_STRIDE / 4) + 1 + d4, total);
        }
        float M = m[0];
#pragma unroll
        for (int c = 1; c < NS; c++) M = fmaxf(M, m[c]);
        float Ls = 0.f;
        f32x4 O = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NS; c++) {
            const float e = __expf(m[c] - M);
            Ls = fmaf(l[c], e, Ls);
            O.x = fmaf(o[c].x, e, O.x); O.y = fmaf(o[c].y, e, O.y);
            O.z = fmaf(o[c].z, e, O.z); O.w = fmaf(o[c].w, e, O.w);
        }
        const float inv = 1.0f / Ls;
        dst[i] = f32x4{O.x * inv, O.y * inv, O.z * inv, O.w * inv};
    }
    __syncthreads();
}

__device__ __forceinline__ void vt_stage_attn(float *lds_x, const vt_step_args &a) {
    const int NS = vt_attn_split(a);
    if (NS == 8) vt_stage_attn_parts<8>(lds_x, a);
    else if (NS == 2) vt_stage_attn_parts<2>(lds_x, a);
    else vt_stage(lds_x, a.attn, VT_Q_DIM);
}

/* While a layer's attention runs on 32 workgroups, the others pull the K and V rows that the
 * NEXT layer's attention will read into the L2 of the XCD that will read them (kv head =
 * blockIdx % 8, one lane per 128-byte line, plain loads).  The rows are small (1 KB per position
 * and kv head) and nothing else allocates in L2 in between - weights stream with the
 * non-temporal hint - so the next attention finds them there instead of in HBM.  Wave 0 stays
 * out of it: it polls the barrier. */
__device__ __forceinline__ void vt_kv_l2_prefetch(const vt_step_args &a, int layer, int busy) {
    const int G = (int)gridDim.x, wg = (int)blockIdx.x, nw = (int)(blockDim.x >> 6);
    if ((G & 7) || wg < busy || vt_wave() == 0) return;
    const int idle0 = busy >> 3;                                /* workgroups per XCD that run the attention */
    const int me = (((wg >> 3) - idle0) * (nw - 1) + vt_wave() - 1) * VT_WAVE + vt_lane();
    const int n_lanes = ((G >> 3) - idle0) * (nw - 1) * VT_WAVE;
    const int lines_per_row = VT_HEAD_DIM * 4 / 128;            /* 4 */
    const int total = 2 * a.pos * lines_per_row;                /* K and V rows 0 .. pos - 1 */
    const size_t base = (size_t)(a.first_layer + layer) * a.kv_max * VT_KV_DIM + (wg & 7) * VT_HEAD_DIM;
    unsigned acc = 0u;
    for (int g0 = me; g0 < total; g0 += 4 * n_lanes) {
        unsigned v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int g = min(g0 + u * n_lanes, total - 1);     /* past the end: the last line once more */
            const int line = g % lines_per_row, row = (g / lines_per_row) % a.pos, kv = g / (lines_per_row * a.pos);
            const float *p = (kv ? a.kv_v : a.kv_k) + base + (size_t)row * VT_KV_DIM + line * 32;
            v[u] = *reinterpret_cast<const unsigned *>(p);
        }
        acc ^= (v[0] ^ v[1]) ^ (v[2] ^ v[3]);
    }
    asm volatile("" ::"v"(acc));
}

/* Workgroups 0 .. busy-1 run the attention of this step (busy is a multiple of 8: the same number
 * on every XCD); the others have the phase to themselves and prefetch into their L2. */
__device__ __forceinline__ int vt_attn_busy(const vt_step_args &a) {
    if (vt_attn_is_direct(a)) return VT_HEADS * vt_attn_split(a);
    const int nch_max = (int)gridDim.x / VT_KV_HEADS;
    int cs, nch;
    vt_attn_geometry(a.pos + 1, nch_max, (int)(blockDim.x >> 6), cs, nch);
    return nch * VT_KV_HEADS;
}

__device__ __forceinline__ void vt_attn_phase(const vt_step_args &a, int layer, float *lds) {
    if (vt_attn_is_direct(a)) { vt_attn_direct(a, layer, lds); return; }
    const int G = (int)gridDim.x;
    const int nch_max = G / VT_KV_HEADS;
    const int wg = (int)blockIdx.x;
    if (wg >= nch_max * VT_KV_HEADS) return;
    const int kvh = wg % VT_KV_HEADS, chunk = wg / VT_KV_HEADS;
    const int nw = (int)(blockDim.x >> 6), wave = vt_wave(), lane = vt_lane();
    const int n = a.pos + 1;
    int cs, nch;
    vt_attn_geometry(n, nch_max, nw, cs, nch);
    if (chunk >= nch) return;
    const int j0 = chunk * cs, j1 = min(n, j0 + cs);

    const int grp = lane >> 4, sub = lane & 15;
    const int head = kvh * 4 + grp;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);
    const f32x4 qa = vt_ldc4(a.q, (head * VT_HEAD_DIM + sub * 8) / 4, VT_Q_DIM);
    const f32x4 qb = vt_ldc4(a.q, (head * VT_HEAD_DIM + sub * 8) / 4 + 1, VT_Q_DIM);
    const size_t layer_base = (size_t)(a.first_layer + layer) * a.kv_max * VT_KV_DIM;
    const float *kbase = a.kv_k + layer_base + kvh * VT_HEAD_DIM + sub * 8;
    const float *vbase = a.kv_v + layer_base + kvh * VT_HEAD_DIM + sub * 8;

    float m = -1e30f, l = 0.f;
    f32x4 oa = {0.f, 0.f, 0.f, 0.f}, ob = {0.f, 0.f, 0.f, 0.f};
    for (int jb = j0 + wave; jb < j1; jb += 4 * nw) {
        f32x4 ka[4], kb[4], va[4], vb[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = min(jb + u * nw, j1 - 1);        /* clamped rows are loaded but not used */
            const f32x4 *kp = reinterpret_cast<const f32x4 *>(kbase + (size_t)j * VT_KV_DIM);
            const f32x4 *vp = reinterpret_cast<const f32x4 *>(vbase + (size_t)j * VT_KV_DIM);
            ka[u] = kp[0]; kb[u] = kp[1];
            va[u] = vp[0]; vb[u] = vp[1];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (jb + u * nw < j1) {
                float s = qa.x * ka[u].x;
                s = fmaf(qa.y, ka[u].y, s); s = fmaf(qa.z, ka[u].z, s); s = fmaf(qa.w, ka[u].w, s);
                s = fmaf(qb.x, kb[u].x, s); s = fmaf(qb.y, kb[u].y, s); s = fmaf(qb.z, kb[u].z, s);
                s = fmaf(qb.w, kb[u].w, s);
                s = vt_row16_sum(s) * scale;
                const float mn = fmaxf(m, s);
                const float corr = expf(m - mn), p = expf(s - mn);
                l = fmaf(l, corr, p);
                oa = oa * corr + va[u] * p;
                ob = ob * corr + vb[u] * p;
                m = mn;
            }
        }
    }
    /* merge the waves of this workgroup */
    float *part = lds;                                   /* [nw][4][VT_ATT_STRIDE] */
    float *mine = part + (wave * 4 + grp) * VT_ATT_STRIDE;
    if (sub == 0) { mine[0] = m; mine[1] = l; }
    *reinterpret_cast<f32x4 *>(mine + 4 + sub * 8) = oa;
    *reinterpret_cast<f32x4 *>(mine + 8 + sub * 8) = ob;
    __syncthreads();
    for (int t = (int)threadIdx.x; t < 4 * VT_HEAD_DIM; t += (int)blockDim.x) {
        const int g = t >> 7, d = t & 127;
        float M = -1e30f;
        for (int w = 0; w < nw; w++) M = fmaxf(M, part[(w * 4 + g) * VT_ATT_STRIDE]);
        float Ls = 0.f, O = 0.f;
        for (int w = 0; w < nw; w++) {
            const float *pw = part + (w * 4 + g) * VT_ATT_STRIDE;
            const float e = expf(pw[0] - M);
            Ls = fmaf(pw[1], e, Ls);
            O = fmaf(pw[4 + d], e, O);
        }
        if (nch == 1) {
            vt_stc(a.attn + (kvh * 4 + g) * VT_HEAD_DIM + d, O * (1.0f / Ls));
        } else {
            float *dst = a.att_part + ((size_t)(kvh * 4 + g) * nch_max + chunk) * VT_ATT_STRIDE;
            if (d == 0) { vt_stc(dst, M); vt_stc(dst + 1, Ls); }
            vt_stc(dst + 4 + d, O);
        }
    }
    if (nch == 1) return;
    /* last workgroup of this kv head merges the chunks */
    __shared__ int s_last;
    __builtin_amdgcn_s_waitcnt(0x0F70);                  /* partial stores acknowledged */
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned old = __hip_atomic_fetch_add(a.att_cnt + layer * VT_KV_HEADS + kvh, 1u,
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (unsigned)(nch - 1));
    }
    __syncthreads();
    if (!s_last) return;
    float *ml = lds;                                      /* [4][nch][2] staged (max, sum) pairs */
    for (int t = (int)threadIdx.x; t < 4 * nch; t += (int)blockDim.x) {
        const int g = t / nch, c = t % nch;
        const float *src = a.att_part + ((size_t)(kvh * 4 + g) * nch_max + c) * VT_ATT_STRIDE;
        ml[2 * t] = vt_ldc(src);
        ml[2 * t + 1] = vt_ldc(src + 1);
    }
    __syncthreads();
    for (int t = (int)threadIdx.x; t < 4 * VT_HEAD_DIM; t += (int)blockDim.x) {
        const int g = t >> 7, d = t & 127;
        const float *src = a.att_part + (size_t)(kvh * 4 + g) * nch_max * VT_ATT_STRIDE + 4 + d;
        float M = -1e30f;
        for (int c = 0; c < nch; c++) M = fmaxf(M, ml[2 * (g * nch + c)]);
        float Ls = 0.f, O = 0.f;
        for (int c0 = 0; c0 < nch; c0 += 4) {
            float o[4];
#pragma unroll
            for (int u = 0; u < 4; u++) o[u] = vt_ldc(src + (size_t)min(c0 + u, nch - 1) * VT_ATT_STRIDE);
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (c0 + u < nch) {
                    const float e = expf(ml[2 * (g * nch + c0 + u)] - M);
                    Ls = fmaf(ml[2 * (g * nch + c0 + u) + 1], e, Ls);
                    O = fmaf(o[u], e, O);
                }
            }
        }
        vt_stc(a.attn + (kvh * 4 + g) * VT_HEAD_DIM + d, O * (1.0f / Ls));
    }
}

/* ---- phase 3: x = x_in + wo * attn ---------------------------------------- */

__device__ __forceinline__ vt_rows vt_wo_rows() { return vt_split_rows<2>(VT_DIM, 1, VT_Q_DIM / 2); }

__device__ __forceinline__ void vt_wo_prefetch(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                               int part = VT_PART_ALL) {
    vt_ring_prefetch<4, 4>(ring, L.wo, VT_Q_DIM, vt_wo_rows(), part);
}

template <class AR = vt_nothing>
__device__ __forceinline__ void vt_wo_body(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                           const vt_step_args &a, const float *x_in, float *lds,
                                           AR after_run = AR()) {
    const vt_rows r = vt_wo_rows();
    float *lds_y = lds + VT_LDS_X;
    vt_stage_attn(lds, a);
    f32x4 xa[4], xb[4];
    vt_slice_lds<4>(xa, xb, lds, r.kofs);
    /* the residual value of this thread's row, requested before any bulk load of the next phase */
    const int tr = (int)threadIdx.x < r.wg_nrows ? (int)threadIdx.x : 0;
    const float prev = vt_ldc(x_in + r.wg_row0 + tr);
    vt_ring_run<4, 4, 3>(ring, L.wo, VT_Q_DIM, r, xa, xb, lds_y);
    after_run();
    __syncthreads();
    for (int t = (int)threadIdx.x; t < r.wg_nrows; t += (int)blockDim.x) {
        const float y = lds_y[t] + lds_y[r.wg_nrows + t];
        vt_stc(a.x + r.wg_row0 + t, (t == tr ? prev : vt_ldc(x_in + r.wg_row0 + t)) + y);
    }
}

/* ---- phase 4: RMSNorm + [w1|w3] + SiLU(gate)*up --------------------------- */

__device__ __forceinline__ vt_rows vt_w13_rows() { return vt_split_rows<1>(2 * VT_FFN, 2, 0); }

#define VT_WO_SLOTS 12         /* ring slots the output projection uses (3 rows x 4 KB per wave) */

__device__ __forceinline__ void vt_w13_prefetch(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                                int part = VT_PART_ALL, int slot_lo = 0, int slot_hi = VT_RING) {
    vt_ring_prefetch<6, 3>(ring, L.w13, VT_DIM, vt_w13_rows(), part, slot_lo, slot_hi);
}

/* The same idle workgroups also pull the last VT_L2_ROWS gate|up rows of every wave of their XCD
 * into its L2; those rows are multiplied two phases later and then come from the L2 instead of
 * HBM, which is idle now. */
#ifndef VT_L2_ROWS
#define VT_L2_ROWS 2
#endif
#ifndef VT_L2_SKIP
#define VT_L2_SKIP 24          /* lines of the first prefetched row that are left out: 1.5 rows fit the L2 as well as 2 */
#endif

__device__ __forceinline__ void vt_w13_l2_prefetch(const vt_layer_dev &L, int busy) {
    const int G = (int)gridDim.x, wg = (int)blockIdx.x, nw = (int)(blockDim.x >> 6);
    if ((G & 7) || wg < busy || vt_wave() == 0) return;
    const int per_x = G >> 3, idle0 = busy >> 3;
    const int me = (((wg >> 3) - idle0) * (nw - 1) + vt_wave() - 1) * VT_WAVE + vt_lane();
    const int n_lanes = (per_x - idle0) * (nw - 1) * VT_WAVE;
    const int per_wg = vt_rows_per_wg(2 * VT_FFN, 2, G);
    const int per_wave = (per_wg + nw - 1) / nw;
    const int lines_per_row = VT_DIM * 2 / 128;
    const int total = per_x * nw * VT_L2_ROWS * lines_per_row;
    /* four lines per turn, requested without a condition (a line that is not wanted is replaced by
     * the first line of the matrix): with one conditional load per turn every turn waits for its
     * own load */
    unsigned acc = 0u;
    for (int g0 = me; g0 < total; g0 += 4 * n_lanes) {
        unsigned v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int g = g0 + u * n_lanes;
            const int line = g % lines_per_row, t = g / lines_per_row;
            const int rr = t % VT_L2_ROWS, wv = (t / VT_L2_ROWS) % nw, i = t / (VT_L2_ROWS * nw);
            const int row = ((wg & 7) + 8 * i) * per_wg + wv * per_wave + per_wave - VT_L2_ROWS + rr;
            const bool want = g < total && row < 2 * VT_FFN && !(rr == 0 && line < VT_L2_SKIP);
            const size_t at = want ? (size_t)row * VT_DIM + line * 64 : 0;
            v[u] = *reinterpret_cast<const unsigned *>(L.w13 + at);
        }
        acc ^= (v[0] ^ v[1]) ^ (v[2] ^ v[3]);
    }
    asm volatile("" ::"v"(acc));
}

template <class AR = vt_nothing>
__device__ __forceinline__ void vt_w13_body(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                            const vt_step_args &a, float *lds, AR after_run = AR()) {
    const vt_rows r = vt_w13_rows();
    float *lds_y = lds + VT_LDS_X;
    vt_stage(lds, a.x, VT_DIM);
    f32x4 xa[6], xb[6];
    vt_rmsnorm_slice(xa, xb, lds, L.ffn_norm);
    vt_ring_run<6, 3, 9>(ring, L.w13, VT_DIM, r, xa, xb, lds_y);
    after_run();
    __syncthreads();
    for (int t = (int)threadIdx.x; t < r.wg_nrows / 2; t += (int)blockDim.x) {
        const float g = lds_y[2 * t], u = lds_y[2 * t + 1];
        const float sg = g / (1.0f + expf(-g));                      /* voxtral_tts_kernels.c:361-366 */
        vt_stc(a.h + r.wg_row0 / 2 + t, sg * u);
    }
}

/* ---- phase 5: x += w2 * h -------------------------------------------------- */

__device__ __forceinline__ vt_rows vt_w2_rows() { return vt_split_rows<2>(VT_DIM, 1, VT_FFN / 2); }

__device__ __forceinline__ void vt_w2_prefetch(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                               int part = VT_PART_ALL) {
    vt_ring_prefetch<9, 2>(ring, L.w2, VT_FFN, vt_w2_rows(), part);
}

/* out_direct: also write the result rows to a.out_hidden (the last layer of a step without a final norm:
 * the output is then complete when the kernel ends and needs no hand-over of its own). */
template <class AR = vt_nothing>
__device__ __forceinline__ void vt_w2_body(u32x4 (&ring)[VT_RING], const vt_layer_dev &L,
                                           const vt_step_args &a, float *lds, AR after_run = AR(),
                                           bool out_direct = false) {
    const vt_rows r = vt_w2_rows();
    float *lds_y = lds + VT_LDS_X;
    vt_stage(lds, a.h, VT_FFN);
    f32x4 xa[9], xb[9];
    vt_slice_lds<9>(xa, xb, lds, r.kofs);
    const int tr = (int)threadIdx.x < r.wg_nrows ? (int)threadIdx.x : 0;
    const float prev = vt_ldc(a.x + r.wg_row0 + tr);
    vt_ring_run<9, 2, 3>(ring, L.w2, VT_FFN, r, xa, xb, lds_y);
    after_run();
    __syncthreads();
    for (int t = (int)threadIdx.x; t < r.wg_nrows; t += (int)blockDim.x) {
        const float y = lds_y[t] + lds_y[r.wg_nrows + t];
        const float v = (t == tr ? prev : vt_ldc(a.x + r.wg_row0 + t)) + y;
        vt_stc(a.x + r.wg_row0 + t, v);
        if (out_direct) a.out_hidden[r.wg_row0 + t] = v;
    }
}

/* ---- RMSNorm of one row by one workgroup ------------------------------------ */

template <bool COHERENT>
__device__ __forceinline__ void vt_block_rmsnorm(float *out, const float *x, const float *w,
                                                 int dim, float eps, float *lds) {
    float ss = 0.f;
    for (int i = (int)threadIdx.x; i < dim; i += (int)blockDim.x) {
        const float v = COHERENT ? vt_ldc(x + i) : x[i];
        ss = fmaf(v, v, ss);
    }
    ss = vt_wave_sum(ss);
    if (vt_lane() == 0) lds[vt_wave()] = ss;
    __syncthreads();
    float tot = 0.f;
    for (int w_ = 0; w_ < (int)(blockDim.x >> 6); w_++) tot += lds[w_];
    const float inv = 1.0f / sqrtf(tot / (float)dim + eps);
    for (int i = (int)threadIdx.x; i < dim; i += (int)blockDim.x) {
        const float v = COHERENT ? vt_ldc(x + i) : x[i];
        out[i] = (v * inv) * w[i];
    }
    __syncthreads();
}

#endif /* VT_DECODE_PHASES_H */
