/*
 * vt_decode_stream.hip - the whole-step decode kernel for a 256-CU device:
 * weight streaming decoupled from synchronisation.
 *
 * One workgroup per CU, 7 waves: 6 STREAM waves and 1 CONTROL wave.
 *
 *  - A stream wave does nothing but read bf16 weights and multiply.  The
 *    weights of a phase that belong to a workgroup are one contiguous block,
 *    cut into UNITS of 512 elements (one 16-byte load per lane, 1 KB per
 *    wave); the rows of every phase divide by 6 (24, 12, 72, 12 per workgroup),
 *    so stream wave w owns whole rows: a contiguous run of units per phase.
 *    Its units of a whole layer form a fixed program of 150 positions, kept in
 *    a register ring of 25 slots (150 = 6 x 25, so the slot of a position is
 *    the same in every layer and all ring indices are compile-time constants).
 *    Consuming position p immediately requests position p + 25, whichever
 *    phase or layer that is: 25 KB per wave, 150 KB per CU, are always in
 *    flight or landed, independent of any barrier.  A row's units are summed
 *    in registers, reduced over the wave with DPP and left in LDS.  The loop
 *    has no data-dependent branch, so the compiler's wait counts on the ring
 *    stay exact: a unit waits only for its own load.
 *
 *  - The control wave owns every access that is NOT a weight: it reads the
 *    vector a phase consumes (coherently, past the L2), normalises it
 *    (RMSNorm) and puts it in LDS for the stream waves; it sums the row
 *    partials, applies RoPE / SwiGLU / the residual, writes the outputs
 *    through to memory, runs the grid barrier (per-workgroup epoch flags,
 *    no read-modify-write) and computes the attention of its chunk of the KV
 *    cache.  Vector-memory results return in order within a wave, so a wave
 *    with ~40 weight loads in flight would see every poll or hand-over read
 *    queue behind them; keeping those accesses on a wave that never streams
 *    keeps the synchronisation path at memory latency while HBM stays busy.
 *
 * Phase order and arithmetic follow the reference CPU step
 * (voxtral_tts_llm.c:205-267); this kernel replaces tts_cuda_llm_forward's
 * launch sequence (voxtral_tts_cuda.cu:710-797).
 */
#include "vt_state.h"

#define VS_NCW 6                 /* stream waves per workgroup */
#define VS_THREADS ((VS_NCW + 1) * VT_WAVE)
#define VS_RING 25               /* ring slots (16 B per lane each) */
#define VS_PROG 150              /* positions per layer = 6 * VS_RING */
#define VS_LDS_X 9216            /* staged vector (largest: SwiGLU output) */
#define VS_LDS_Y 128             /* row results of one phase (largest: 72) */
#define VS_ATT_MAXCH 16          /* attention chunks per kv head */

/* One phase as seen by a workgroup of a 256-workgroup grid: `rows` consecutive
 * rows of `nk` 512-element units each, one contiguous block of memory.  Every
 * stream wave owns rows/6 whole rows = `own` consecutive units, at program
 * positions p0 .. p0+own-1.  The run of the last phase carries two spare
 * positions (k = own + 2) that repeat the wave's last unit, which makes the
 * program 150 = 6 x 25 positions long. */
struct vs_phase { int p0, k, own, nk, rows, row_len; };

__device__ __forceinline__ vs_phase vs_phase_of(int ph) {
    switch (ph) {
    case 0:  return vs_phase{0, 24, 24, 6, 24, VT_DIM};         /* [wq;wk;wv]: 4 rows x 6 units per wave */
    case 1:  return vs_phase{24, 16, 16, 8, 12, VT_Q_DIM};      /* wo:      2 rows x 8 units  */
    case 2:  return vs_phase{40, 72, 72, 6, 72, VT_DIM};        /* [w1|w3]: 12 rows x 6 units */
    default: return vs_phase{112, 38, 36, 18, 12, VT_FFN};      /* w2:      2 rows x 18 units (+2 spare) */
    }
}
__device__ __forceinline__ int vs_phase_at(int pos) { return pos < 24 ? 0 : pos < 40 ? 1 : pos < 112 ? 2 : 3; }

/* The layer table is read-only for the whole kernel: reading it through the
 * constant address space makes these uniform loads scalar, so they do not sit
 * in the vector-memory queue behind the weight stream. */
__device__ __forceinline__ vt_layer_dev vs_layer(const vt_layer_dev *layers, int l) {
    typedef __attribute__((address_space(4))) const vt_layer_dev cl_t;
    const cl_t *p = (const cl_t *)layers;
    vt_layer_dev L;
    L.wqkv = p[l].wqkv; L.wo = p[l].wo; L.w13 = p[l].w13; L.w2 = p[l].w2;
    L.attn_norm = p[l].attn_norm; L.ffn_norm = p[l].ffn_norm;
    return L;
}

__device__ __forceinline__ const uint16_t *vs_weights(const vt_layer_dev &L, int ph) {
    return ph == 0 ? L.wqkv : ph == 1 ? L.wo : ph == 2 ? L.w13 : L.w2;
}

/* Address of program position `pos` (0..149) of layer L for stream wave cw. */
__device__ __forceinline__ const uint16_t *vs_unit_ptr(const vt_layer_dev &L, int pos, int cw, int lane) {
    const int ph = vs_phase_at(pos);
    const vs_phase P = vs_phase_of(ph);
    const int k = pos - P.p0;
    const int e = cw * P.own + (k < P.own ? k : P.own - 1);
    const uint16_t *blk = vs_weights(L, ph) + (size_t)blockIdx.x * P.rows * P.row_len;
    return blk + (size_t)e * 512 + lane * 8;
}

/* Stream wave, compute half: consume slots [k0, k1) of the run of phase PH.
 * The units of a row are accumulated in registers; at the (compile-time) end of
 * each row the wave reduces with DPP and lane 63 leaves the dot product in LDS.
 * No load is issued here and nothing branches on data, so the compiler's wait
 * counts on the ring stay exact: a unit waits for its own load only. */
template <int PH>
__device__ __forceinline__ void vs_consume(const u32x4 (&ring)[VS_RING], int cw, int lane,
                                           const float *xs, float *yp, int k0, int k1,
                                           float &a0, float &a1) {
    const vs_phase P = vs_phase_of(PH);
    const int rows_per_wave = P.own / P.nk;
    const f32x4 *xv = reinterpret_cast<const f32x4 *>(xs + lane * 8);
#pragma unroll
    for (int k = k0; k < k1; k++) {
        if (k < P.own) {                                       /* compile-time: spare slots hold no work */
            const int chunk = k % P.nk;
            const f32x4 xa = xv[chunk * 128], xb = xv[chunk * 128 + 1];
            const u32x4 w = ring[(P.p0 + k) % VS_RING];
            a0 = fmaf(vt_bf16_lo(w.x), xa.x, a0); a1 = fmaf(vt_bf16_lo(w.z), xb.x, a1);
            a0 = fmaf(vt_bf16_hi(w.x), xa.y, a0); a1 = fmaf(vt_bf16_hi(w.z), xb.y, a1);
            a0 = fmaf(vt_bf16_lo(w.y), xa.z, a0); a1 = fmaf(vt_bf16_lo(w.w), xb.z, a1);
            a0 = fmaf(vt_bf16_hi(w.y), xa.w, a0); a1 = fmaf(vt_bf16_hi(w.w), xb.w, a1);
            if (chunk == P.nk - 1) {                           /* compile-time: end of a row */
                const float sum = vt_wave_sum_lane63(a0 + a1);
                if (lane == VT_WAVE - 1) yp[cw * rows_per_wave + k / P.nk] = sum;
                a0 = 0.f; a1 = 0.f;
            }
        }
    }
}

/* `s_waitcnt vmcnt(n)` alone (expcnt and lgkmcnt left unconstrained). */
#define VS_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (7 << 4) | (15 << 8) | (((n) >> 4) << 14))

/* Stream wave, memory half: refill the slots of positions [k0, k1) of the run of
 * phase PH with the positions 25 ahead - of this layer, or of the next one (Ln).
 * When there is no next layer `dummy` is non-NULL and 1 KB of a small resident
 * block is requested instead, at no HBM cost.  Requests are paced: a wave keeps
 * at most VS_PACE loads outstanding, so the CU's memory queue stays short and
 * the control wave's polls and hand-over reads do not wait behind a long line of
 * weight requests. */
#ifndef VS_PACE
#define VS_PACE 8
#endif
template <int PH>
__device__ __forceinline__ void vs_refill(u32x4 (&ring)[VS_RING], const vt_layer_dev &Lc,
                                          const vt_layer_dev &Ln, const uint16_t *dummy, int cw,
                                          int lane, int k0, int k1) {
    const vs_phase P = vs_phase_of(PH);
#pragma unroll
    for (int k = k0; k < k1; k++) {
        const int pos = P.p0 + k;
        const int nxt = pos + VS_RING;
        const uint16_t *p = nxt < VS_PROG ? vs_unit_ptr(Lc, nxt, cw, lane)
                                          : vs_unit_ptr(Ln, nxt - VS_PROG, cw, lane);
        if (nxt >= VS_PROG) p = dummy ? dummy + lane * 8 : p;
        VS_VMCNT(VS_PACE - 1);
        ring[pos % VS_RING] = vt_ldw(p);
    }
}

/* One phase of a stream wave: ring-sized blocks are consumed and refilled in turn;
 * the last block is consumed, the workgroup barrier S2 releases the control wave,
 * and only then is that block refilled - those requests travel while the control
 * wave runs the epilogue, the grid barrier and the next hand-over. */
template <int PH>
__device__ __forceinline__ void vs_phase_run(u32x4 (&ring)[VS_RING], const vt_layer_dev &Lc,
                                             const vt_layer_dev &Ln, const uint16_t *dummy, int cw,
                                             int lane, const float *xs, float *yp) {
    const vs_phase P = vs_phase_of(PH);
    float a0 = 0.f, a1 = 0.f;
    int k0 = 0;
#pragma unroll
    for (; k0 + VS_RING < P.k; k0 += VS_RING) {
        vs_consume<PH>(ring, cw, lane, xs, yp, k0, k0 + VS_RING, a0, a1);
        vs_refill<PH>(ring, Lc, Ln, dummy, cw, lane, k0, k0 + VS_RING);
    }
    vs_consume<PH>(ring, cw, lane, xs, yp, k0, P.k, a0, a1);
    __syncthreads();                                              /* S2 */
    vs_refill<PH>(ring, Lc, Ln, dummy, cw, lane, k0, P.k);
}

/* ---- control wave helpers ---------------------------------------------------- */

struct vs_sync {
    unsigned *flags;
    int *abort_flag;
    unsigned epoch;
    unsigned long long timeout;
};

/* All of this wave's earlier stores are acknowledged before the flag is written. */
__device__ __forceinline__ void vs_arrive(vs_sync &gs, int lane) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (lane == 0) vt_stc_u32(gs.flags + blockIdx.x, gs.epoch);
}

__device__ __forceinline__ bool vs_wait(vs_sync &gs, int lane) {
    const int G = (int)gridDim.x;
    const unsigned long long t0 = wall_clock64();
    int ok = 1;
    for (;;) {
        int done = 1;
        for (int i = lane; i < G; i += VT_WAVE) done &= (int)(vt_ldc_u32(gs.flags + i) - gs.epoch) >= 0;
        if (__all(done)) break;
        if (__hip_atomic_load(gs.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
            wall_clock64() - t0 > gs.timeout) {
            ok = 0;
            break;
        }
    }
    ok = __all(ok);
    if (!ok && lane == 0) __hip_atomic_store(gs.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    gs.epoch += 1u;
    return ok != 0;
}

/* Copy n floats (n % 256 == 0) of a handed-over vector into LDS with this wave alone. */
__device__ __forceinline__ void vs_stage(float *xs, const float *src, int n, int lane) {
    f32x4 *dst = reinterpret_cast<f32x4 *>(xs);
    for (int i0 = 0; i0 < n / 4; i0 += 8 * VT_WAVE) {
        f32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + u * VT_WAVE + lane;
            v[u] = vt_ldc4(src, i < n / 4 ? i : 0, n);
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int i = i0 + u * VT_WAVE + lane;
            if (i < n / 4) dst[i] = v[u];
        }
    }
}

/* RMSNorm of a handed-over 3072-vector into LDS (voxtral_tts_kernels.c:333-349);
 * the gains `w` were read ahead of time into wv. */
__device__ __forceinline__ void vs_stage_norm(float *xs, const float *src, const f32x4 (&wv)[12], int lane) {
    f32x4 v[12];
#pragma unroll
    for (int u = 0; u < 12; u++) v[u] = vt_ldc4(src, u * VT_WAVE + lane, VT_DIM);
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 12; u++) {
        ss = fmaf(v[u].x, v[u].x, ss); ss = fmaf(v[u].y, v[u].y, ss);
        ss = fmaf(v[u].z, v[u].z, ss); ss = fmaf(v[u].w, v[u].w, ss);
    }
    ss = vt_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)VT_DIM + VT_EPS);
    f32x4 *dst = reinterpret_cast<f32x4 *>(xs);
#pragma unroll
    for (int u = 0; u < 12; u++) dst[u * VT_WAVE + lane] = (v[u] * inv) * wv[u];
}

__device__ __forceinline__ void vs_load_gains(f32x4 (&wv)[12], const float *w, int lane) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(w);
#pragma unroll
    for (int u = 0; u < 12; u++) wv[u] = p[u * VT_WAVE + lane];
}

/* ---- attention on the control wave -------------------------------------------- */
/* Control wave of workgroup (kvh = wg % 8, chunk = wg / 8) covers `cs` cache
 * positions of one kv head for its 4 query heads.  Lanes 16g..16g+15 take
 * positions j0+g, j0+g+4, ... and own dims sub*8..+8 of the row; every lane
 * group keeps the online-softmax state of all 4 heads (algebra of
 * voxtral_tts_kernels.c:426-462), the groups are merged by lane exchange, the
 * chunk's (max, sum, o[128]) per head is written through, and the last chunk to
 * finish a kv head merges the chunks and writes the normalised output. */
__device__ __forceinline__ void vs_att_xmerge(float &m, float &l, f32x4 &oa, f32x4 &ob, int step, int lane) {
    const float m2 = __shfl_xor(m, step), l2 = __shfl_xor(l, step);
    f32x4 pa, pb;
    pa.x = __shfl_xor(oa.x, step); pa.y = __shfl_xor(oa.y, step);
    pa.z = __shfl_xor(oa.z, step); pa.w = __shfl_xor(oa.w, step);
    pb.x = __shfl_xor(ob.x, step); pb.y = __shfl_xor(ob.y, step);
    pb.z = __shfl_xor(ob.z, step); pb.w = __shfl_xor(ob.w, step);
    const float M = fmaxf(m, m2);
    const float e1 = __expf(m - M), e2 = __expf(m2 - M);
    const bool lo = (lane & step) == 0;       /* lower lane's term first on both sides: same bits */
    l = lo ? l * e1 + l2 * e2 : l2 * e2 + l * e1;
    oa = lo ? oa * e1 + pa * e2 : pa * e2 + oa * e1;
    ob = lo ? ob * e1 + pb * e2 : pb * e2 + ob * e1;
    m = M;
}

__device__ __forceinline__ void vs_att_geometry(int n, int &cs, int &nch) {
    cs = 16 * ((n + 16 * VS_ATT_MAXCH - 1) / (16 * VS_ATT_MAXCH));
    nch = (n + cs - 1) / cs;
}

__device__ __forceinline__ void vs_attention(const vt_step_args &a, int layer, int lane) {
    const int wg = (int)blockIdx.x;
    const int kvh = wg % VT_KV_HEADS, chunk = wg / VT_KV_HEADS;
    const int n = a.pos + 1;
    int cs, nch;
    vs_att_geometry(n, cs, nch);
    if (chunk >= nch) return;
    const int j0 = chunk * cs, j1 = min(n, j0 + cs);
    const int grp = lane >> 4, sub = lane & 15;
    const float scale = 1.0f / sqrtf((float)VT_HEAD_DIM);

    f32x4 qa[4], qb[4];
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
        qa[hh] = vt_ldc4(a.q, ((kvh * 4 + hh) * VT_HEAD_DIM + sub * 8) / 4, VT_Q_DIM);
        qb[hh] = vt_ldc4(a.q, ((kvh * 4 + hh) * VT_HEAD_DIM + sub * 8) / 4 + 1, VT_Q_DIM);
    }
    const size_t layer_base = (size_t)(a.first_layer + layer) * a.kv_max * VT_KV_DIM;
    const float *kbase = a.kv_k + layer_base + kvh * VT_HEAD_DIM + sub * 8;
    const float *vbase = a.kv_v + layer_base + kvh * VT_HEAD_DIM + sub * 8;

    float m[4], l[4];
    f32x4 oa[4], ob[4];
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
        m[hh] = -1e30f; l[hh] = 0.f;
        oa[hh] = (f32x4){0.f, 0.f, 0.f, 0.f};
        ob[hh] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    for (int jb = j0 + grp; jb < j1 + 3; jb += 16) {           /* wave-uniform trip count */
        f32x4 ka[4], kb[4], va[4], vb[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = min(jb + 4 * u, j1 - 1);              /* clamped rows are loaded, not used */
            const f32x4 *kp = reinterpret_cast<const f32x4 *>(kbase + (size_t)j * VT_KV_DIM);
            const f32x4 *vp = reinterpret_cast<const f32x4 *>(vbase + (size_t)j * VT_KV_DIM);
            ka[u] = kp[0]; kb[u] = kp[1];
            va[u] = vp[0]; vb[u] = vp[1];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const bool valid = jb + 4 * u < j1;                  /* uniform inside a 16-lane row */
#pragma unroll
            for (int hh = 0; hh < 4; hh++) {
                float s = qa[hh].x * ka[u].x;
                s = fmaf(qa[hh].y, ka[u].y, s); s = fmaf(qa[hh].z, ka[u].z, s);
                s = fmaf(qa[hh].w, ka[u].w, s); s = fmaf(qb[hh].x, kb[u].x, s);
                s = fmaf(qb[hh].y, kb[u].y, s); s = fmaf(qb[hh].z, kb[u].z, s);
                s = fmaf(qb[hh].w, kb[u].w, s);
                s = vt_row16_sum(s) * scale;
                if (valid) {
                    const float mn = fmaxf(m[hh], s);
                    const float corr = __expf(m[hh] - mn), p = __expf(s - mn);
                    l[hh] = fmaf(l[hh], corr, p);
                    oa[hh] = oa[hh] * corr + va[u] * p;
                    ob[hh] = ob[hh] * corr + vb[u] * p;
                    m[hh] = mn;
                }
            }
        }
    }
    /* merge the 4 lane groups; group g then keeps head g */
    float mm = 0.f, ll = 0.f;
    f32x4 oam = {0.f, 0.f, 0.f, 0.f}, obm = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int hh = 0; hh < 4; hh++) {
        vs_att_xmerge(m[hh], l[hh], oa[hh], ob[hh], 16, lane);
        vs_att_xmerge(m[hh], l[hh], oa[hh], ob[hh], 32, lane);
        if (grp == hh) { mm = m[hh]; ll = l[hh]; oam = oa[hh]; obm = ob[hh]; }
    }
    const int head = kvh * 4 + grp;
    float *out = a.attn + head * VT_HEAD_DIM + sub * 8;
    if (nch == 1) {
        const float inv = 1.0f / ll;
        vt_stc(out + 0, oam.x * inv); vt_stc(out + 1, oam.y * inv);
        vt_stc(out + 2, oam.z * inv); vt_stc(out + 3, oam.w * inv);
        vt_stc(out + 4, obm.x * inv); vt_stc(out + 5, obm.y * inv);
        vt_stc(out + 6, obm.z * inv); vt_stc(out + 7, obm.w * inv);
        return;
    }
    float *part = a.att_part + ((size_t)head * VS_ATT_MAXCH + chunk) * VT_ATT_STRIDE;
    if (sub == 0) { vt_stc(part, mm); vt_stc(part + 1, ll); }
    vt_stc(part + 4 + sub * 8 + 0, oam.x); vt_stc(part + 4 + sub * 8 + 1, oam.y);
    vt_stc(part + 4 + sub * 8 + 2, oam.z); vt_stc(part + 4 + sub * 8 + 3, oam.w);
    vt_stc(part + 4 + sub * 8 + 4, obm.x); vt_stc(part + 4 + sub * 8 + 5, obm.y);
    vt_stc(part + 4 + sub * 8 + 6, obm.z); vt_stc(part + 4 + sub * 8 + 7, obm.w);
    __builtin_amdgcn_s_waitcnt(0x0F70);                          /* partial acknowledged */
    unsigned old = 0;
    if (lane == 0)
        old = __hip_atomic_fetch_add(a.att_cnt + layer * VT_KV_HEADS + kvh, 1u, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
    old = (unsigned)__builtin_amdgcn_readfirstlane((int)old);
    if (old != (unsigned)(nch - 1)) return;
    /* last chunk of this kv head: merge all chunks of head `head` in chunk order */
    const float *src = a.att_part + (size_t)head * VS_ATT_MAXCH * VT_ATT_STRIDE;
    float cm[VS_ATT_MAXCH];
#pragma unroll
    for (int c = 0; c < VS_ATT_MAXCH; c++) cm[c] = vt_ldc(src + (c < nch ? c : nch - 1) * VT_ATT_STRIDE);
    float M = -1e30f;
#pragma unroll
    for (int c = 0; c < VS_ATT_MAXCH; c++) if (c < nch) M = fmaxf(M, cm[c]);
    float Ls = 0.f;
    f32x4 Oa = {0.f, 0.f, 0.f, 0.f}, Ob = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c0 = 0; c0 < VS_ATT_MAXCH; c0 += 8) {
        if (c0 < nch) {                                           /* wave-uniform */
            float cl[8];
            f32x4 ca[8], cb[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int cc = c0 + u < nch ? c0 + u : nch - 1;
                cl[u] = vt_ldc(src + cc * VT_ATT_STRIDE + 1);
                ca[u] = vt_ldc4(src, (cc * VT_ATT_STRIDE + 4 + sub * 8) / 4, VS_ATT_MAXCH * VT_ATT_STRIDE);
                cb[u] = vt_ldc4(src, (cc * VT_ATT_STRIDE + 4 + sub * 8) / 4 + 1, VS_ATT_MAXCH * VT_ATT_STRIDE);
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (c0 + u < nch) {
                    const float e = __expf(cm[c0 + u] - M);
                    Ls = fmaf(cl[u], e, Ls);
                    Oa = Oa + ca[u] * e;
                    Ob = Ob + cb[u] * e;
                }
            }
        }
    }
    const float inv = 1.0f / Ls;
    vt_stc(out + 0, Oa.x * inv); vt_stc(out + 1, Oa.y * inv);
    vt_stc(out + 2, Oa.z * inv); vt_stc(out + 3, Oa.w * inv);
    vt_stc(out + 4, Ob.x * inv); vt_stc(out + 5, Ob.y * inv);
    vt_stc(out + 6, Ob.z * inv); vt_stc(out + 7, Ob.w * inv);
}

/* ---- the kernel ------------------------------------------------------------------ */
/* The two roles run disjoint loops that meet at the same sequence of workgroup
 * barriers: per phase one after the control wave has staged the input vector
 * (S1) and one after the stream waves have left their partials (S2).  The
 * control wave raises s_abort before an S1 when a grid barrier timed out;
 * every wave tests it right after that S1 and leaves. */

__device__ __forceinline__ void vs_stream_loop(const vt_step_args &a, const uint16_t *dummy, int cw,
                                               int lane, const float *xs, float *yp,
                                               const int *s_abort) {
    u32x4 ring[VS_RING];
    {
        const vt_layer_dev L0 = vs_layer(a.layers, 0);
#pragma unroll
        for (int p = 0; p < VS_RING; p++) ring[p] = vt_ldw(vs_unit_ptr(L0, p, cw, lane));
    }
    __syncthreads();                                              /* start */
    for (int l = 0; l < a.n_layers; l++) {
        const vt_layer_dev Lc = vs_layer(a.layers, l);
        const bool more = l + 1 < a.n_layers;
        const vt_layer_dev Ln = vs_layer(a.layers, more ? l + 1 : l);
        const uint16_t *nonext = more ? nullptr : dummy;
        __syncthreads();                                          /* S1 qkv */
        if (*s_abort) return;
        vs_phase_run<0>(ring, Lc, Ln, nonext, cw, lane, xs, yp);    /* holds S2 qkv */
        __syncthreads();                                          /* S1 wo */
        if (*s_abort) return;
        vs_phase_run<1>(ring, Lc, Ln, nonext, cw, lane, xs, yp);    /* holds S2 wo */
        __syncthreads();                                          /* S1 w13 */
        if (*s_abort) return;
        vs_phase_run<2>(ring, Lc, Ln, nonext, cw, lane, xs, yp);    /* holds S2 w13 */
        __syncthreads();                                          /* S1 w2 */
        if (*s_abort) return;
        vs_phase_run<3>(ring, Lc, Ln, nonext, cw, lane, xs, yp);    /* holds S2 w2 */
    }
}

#ifdef VT_TRACE
/* Build-time instrumentation (never in the shipped library): the control waves of
 * workgroups 0 and gridDim.x-1 record the 100 MHz wall clock along the step. */
__device__ unsigned long long vs_trace_buf[2 * 4096];
__device__ __forceinline__ void vs_tr(int &n, int lane) {
    if (lane == 0 && (blockIdx.x == 0 || blockIdx.x == gridDim.x - 1) && n < 4096)
        vs_trace_buf[(blockIdx.x ? 4096 : 0) + n] = wall_clock64();
    n++;
}
extern "C" void tts_hip_stream_trace_read(unsigned long long *out) {
    (void)hipDeviceSynchronize();
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(vs_trace_buf), sizeof(unsigned long long) * 2 * 4096);
}
#define VS_TR() vs_tr(tn, lane)
#else
#define VS_TR() ((void)0)
#endif

__device__ __forceinline__ void vs_control_loop(const vt_step_args &a, vs_sync gs, int lane,
                                                float *xs, const float *yp, int *s_abort) {
    const int wg = (int)blockIdx.x;
    int tn = 0;
    (void)tn;
    if (wg == 0)
        for (int t = lane; t < a.n_layers * VT_KV_HEADS; t += VT_WAVE) vt_stc_u32(a.att_cnt + t, 0u);
    if (lane == 0) *s_abort = 0;
    __syncthreads();                                              /* start */
    const float *x_in = a.in_embed;
    bool ok = true;
    /* wo and w2 give this workgroup the same 12 rows of the residual stream:
     * lane t carries row wg*12 + t across the whole step */
    float xrow = lane < 12 ? a.in_embed[wg * 12 + lane] : 0.f;
    for (int l = 0; l < a.n_layers; l++) {
        const vt_layer_dev Lc = vs_layer(a.layers, l);
        f32x4 gains[12];
        /* ---- phase 1: RMSNorm + [wq;wk;wv] + RoPE + cache append ---- */
        VS_TR();                                                  /* 0 layer start */
        vs_load_gains(gains, Lc.attn_norm, lane);
        vs_stage_norm(xs, x_in, gains, lane);
        VS_TR();                                                  /* 1 staged */
        __syncthreads();                                          /* S1 qkv */
        __syncthreads();                                          /* S2 qkv */
        VS_TR();                                                  /* 2 consumed */
        {
            const vs_phase P = vs_phase_of(0);
            if (lane < P.rows / 2) {
                const int g = wg * P.rows + 2 * lane;
                const float v0 = yp[2 * lane], v1 = yp[2 * lane + 1];
                const size_t kv_row = ((size_t)(a.first_layer + l) * a.kv_max + a.pos) * VT_KV_DIM;
                if (g < VT_Q_DIM + VT_KV_DIM) {
                    const float *cs = a.rope + (size_t)a.pos * VT_HEAD_DIM;
                    const int d = (g & (VT_HEAD_DIM - 1)) >> 1;
                    const float c = cs[2 * d], s = cs[2 * d + 1];
                    float *dst = g < VT_Q_DIM ? a.q + g : a.kv_k + kv_row + (g - VT_Q_DIM);
                    vt_stc(dst, v0 * c - v1 * s);
                    vt_stc(dst + 1, v0 * s + v1 * c);
                } else {
                    float *dst = a.kv_v + kv_row + (g - VT_Q_DIM - VT_KV_DIM);
                    vt_stc(dst, v0);
                    vt_stc(dst + 1, v1);
                }
            }
        }
        vs_arrive(gs, lane);
        VS_TR();                                                  /* 3 arrived */
        ok = vs_wait(gs, lane);
        VS_TR();                                                  /* 4 released */
        /* ---- phase 2: attention ---- */
        if (ok) {
            vs_attention(a, l, lane);
            vs_arrive(gs, lane);
            VS_TR();                                              /* 5 attention done, arrived */
            ok = vs_wait(gs, lane);
            VS_TR();                                              /* 6 released */
        }
        /* ---- phase 3: x = x_in + wo * attn ---- */
        if (ok) vs_stage(xs, a.attn, VT_Q_DIM, lane);
        else if (lane == 0) *s_abort = 1;
        VS_TR();                                                  /* 7 staged */
        __syncthreads();                                          /* S1 wo */
        if (!ok) return;
        vs_load_gains(gains, Lc.ffn_norm, lane);
        __syncthreads();                                          /* S2 wo */
        VS_TR();                                                  /* 8 consumed */
        {
            const vs_phase P = vs_phase_of(1);
            if (lane < P.rows) {
                xrow = xrow + yp[lane];
                vt_stc(a.x + wg * P.rows + lane, xrow);
            }
        }
        vs_arrive(gs, lane);
        VS_TR();                                                  /* 9 arrived */
        ok = vs_wait(gs, lane);
        VS_TR();                                                  /* 10 released */
        /* ---- phase 4: RMSNorm + [w1|w3] + SiLU(gate)*up ---- */
        if (ok) vs_stage_norm(xs, a.x, gains, lane);
        else if (lane == 0) *s_abort = 1;
        VS_TR();                                                  /* 11 staged */
        __syncthreads();                                          /* S1 w13 */
        if (!ok) return;
        __syncthreads();                                          /* S2 w13 */
        VS_TR();                                                  /* 12 consumed */
        {
            const vs_phase P = vs_phase_of(2);
            if (lane < P.rows / 2) {
                const float g = yp[2 * lane], u = yp[2 * lane + 1];
                const float sg = g / (1.0f + expf(-g));                 /* voxtral_tts_kernels.c:361-366 */
                vt_stc(a.h + wg * (P.rows / 2) + lane, sg * u);
            }
        }
        vs_arrive(gs, lane);
        VS_TR();                                                  /* 13 arrived */
        ok = vs_wait(gs, lane);
        VS_TR();                                                  /* 14 released */
        /* ---- phase 5: x += w2 * h ---- */
        if (ok) vs_stage(xs, a.h, VT_FFN, lane);
        else if (lane == 0) *s_abort = 1;
        VS_TR();                                                  /* 15 staged */
        __syncthreads();                                          /* S1 w2 */
        if (!ok) return;
        __syncthreads();                                          /* S2 w2 */
        VS_TR();                                                  /* 16 consumed */
        {
            const vs_phase P = vs_phase_of(3);
            if (lane < P.rows) {
                xrow = xrow + yp[lane];
                vt_stc(a.x + wg * P.rows + lane, xrow);
            }
        }
        vs_arrive(gs, lane);
        VS_TR();                                                  /* 17 arrived */
        ok = vs_wait(gs, lane);
        VS_TR();                                                  /* 18 released */
        if (!ok) {
            if (lane == 0) *s_abort = 1;
            /* the stream waves test the flag after their next S1; meet them there */
            if (l + 1 < a.n_layers) __syncthreads();
            return;
        }
        x_in = a.x;
    }
    /* final RMSNorm (or a plain copy of the residual stream) by workgroup 0 */
    if (wg == 0) {
        if (a.final_norm) {
            f32x4 gains[12];
            vs_load_gains(gains, a.final_norm, lane);
            vs_stage_norm(xs, a.x, gains, lane);
        } else {
            vs_stage(xs, a.x, VT_DIM, lane);
        }
        const f32x4 *src = reinterpret_cast<const f32x4 *>(xs);
        f32x4 *dst = reinterpret_cast<f32x4 *>(a.out_hidden);
        for (int i = lane; i < VT_DIM / 4; i += VT_WAVE) dst[i] = src[i];
    }
}

__global__ void __launch_bounds__(VS_THREADS)
vt_decode_stream_kernel(vt_step_args a, vs_sync gs, const uint16_t *dummy) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ int s_abort;
    float *xs = lds, *yp = lds + VS_LDS_X;
    const int lane = vt_lane();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (wave == VS_NCW) vs_control_loop(a, gs, lane, xs, yp, &s_abort);
    else vs_stream_loop(a, dummy, wave, lane, xs, yp, &s_abort);
}

/* ---- host side --------------------------------------------------------------------- */

int vt_stream_supported(void) { return g_vt.grid == 256; }

int vt_run_step_stream(const vt_step_args &a) {
    static int attr_set = 0;
    const size_t lds_bytes = sizeof(float) * (VS_LDS_X + VS_LDS_Y);
    size_t dyn = g_vt.step_dyn_lds > lds_bytes ? g_vt.step_dyn_lds : lds_bytes;
    if (!attr_set) {
        if (vt_check(hipFuncSetAttribute((const void *)vt_decode_stream_kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn),
                     "hipFuncSetAttribute"))
            return -1;
        attr_set = 1;
    }
    vs_sync gs;
    gs.flags = g_vt.d_bar_flags;
    gs.abort_flag = g_vt.d_abort;
    gs.epoch = g_vt.bar_epoch + 1u;
    gs.timeout = g_vt.bar_timeout ? g_vt.bar_timeout : 20000000ull;   /* default 0.2 s of the 100 MHz wall clock */
    g_vt.bar_epoch += 5u * (unsigned)a.n_layers;
    hipLaunchKernelGGL(vt_decode_stream_kernel, dim3(g_vt.grid), dim3(VS_THREADS), dyn, g_vt.stream,
                       a, gs, (const uint16_t *)g_vt.d_dummy);
    return vt_check(hipGetLastError(), "decode step launch");
}
