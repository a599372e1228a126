/*
 * vt_gemm.hip - bf16 MFMA matrix product for rows of activations (seq_len > 1):
 * C[M,N] = X[M,K] * W[N,K]^T with fp32 accumulation, the sequence-level linear
 * of the CPU path (tts_linear_nobias_bf16 with seq_len > 1,
 * voxtral_tts_kernels.c:187-198, and the triple loop it falls to, :127-138).
 *
 * Weights are bf16 already.  The fp32 activations are carried as two bf16
 * planes, hi = bf16(x) and lo = bf16(x - hi), so that hi + lo represents x to
 * about 2^-17 relative; every weight tile is multiplied with both planes
 * (two MFMAs per tile pair) and the sums land in the same fp32 accumulator.
 * That keeps the result within a few fp32 ulps of the sequential CPU sum while
 * all products run on the matrix cores.
 *
 * Tiling: workgroup tile 128 x 128, K step 64, four waves in a 2 x 2 grid of
 * 64 x 64 wave tiles, v_mfma_f32_32x32x16_bf16.  Tiles are staged through LDS
 * with a row pitch of 144 bytes (128 of data + 16 of padding): the 16 lanes of
 * a 16-byte fragment read then cover all 64 banks once.  One LDS stage; the
 * next K step is fetched into registers while the current one is multiplied,
 * the fragments of the next 16-wide slice are read while the current slice is
 * multiplied, and two workgroups share a CU.  Workgroups that need the same weight tile
 * (the M tiles of one N tile) get consecutive slots on one XCD, so the tile is
 * fetched from HBM once and served from that XCD's L2 afterwards.  Long K can
 * be cut into `splits` ranges that write separate partial planes; the caller
 * adds them in a fixed order (vt_residual_norm_split_kernel).
 */
#include "vt_state.h"
#include "vt_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(1))) const u32x4 vt_gptr_u32x4;

#define GM_TILE 128
#define GM_BK   64
#define GM_ROWB 144
#define GM_MAT  (GM_TILE * GM_ROWB)

__device__ __forceinline__ u32x4 gm_ld(const uint16_t *p) { return *(vt_gptr_u32x4 *)p; }
__device__ __forceinline__ bf16x8 gm_frag(const unsigned char *p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(p));
}

__global__ void __launch_bounds__(256, 2)
vt_gemm_mfma_kernel(float *C, const uint16_t *Ahi, const uint16_t *Alo, const uint16_t *W,
                    int M, int N, int K, int k_split, int m_tiles, int n_tiles, int ldc, size_t plane_stride) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[3 * GM_MAT];
    const int id = (int)blockIdx.x;
    int mt, nt, sp;
    if ((n_tiles & 7) == 0) {
        /* slot id lands on XCD id % 8: keep the M tiles of one N tile there */
        const int x = id & 7, q = id >> 3, r = q / m_tiles, npx = n_tiles >> 3;
        mt = q % m_tiles;
        nt = (r % npx) * 8 + x;
        sp = r / npx;
    } else {
        const int r = id / m_tiles;
        mt = id % m_tiles;
        nt = r % n_tiles;
        sp = r / n_tiles;
    }
    const int t = (int)threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = t >> 3, lc = t & 7;               /* staging: row lr + 32 i, 16-byte chunk lc */
    const int k0 = sp * k_split, tiles = k_split / GM_BK;

    const uint16_t *pa[4], *pl[4], *pw[4];
    bool live[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int gm = mt * GM_TILE + lr + 32 * i;
        live[i] = gm < M;
        const size_t ao = (size_t)(live[i] ? gm : 0) * K + k0 + lc * 8;
        pa[i] = Ahi + ao;
        pl[i] = Alo + ao;
        pw[i] = W + (size_t)(nt * GM_TILE + lr + 32 * i) * K + k0 + lc * 8;
    }

    /* the next K step is fetched into registers while the current one is multiplied */
    u32x4 ra[4], rl[4], rb[4];
    const u32x4 zero = {0u, 0u, 0u, 0u};
    auto fetch = [&](int kt) {
        const int adv = kt * GM_BK;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            ra[i] = live[i] ? gm_ld(pa[i] + adv) : zero;
            rl[i] = live[i] ? gm_ld(pl[i] + adv) : zero;
            rb[i] = gm_ld(pw[i] + adv);
        }
    };
    fetch(0);

    f32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    const int st_off = lr * GM_ROWB + lc * 16;
    const int fa_off = (64 * wm + (lane & 31)) * GM_ROWB + (lane >> 5) * 16;
    const int fb_off = (64 * wn + (lane & 31)) * GM_ROWB + (lane >> 5) * 16 + 2 * GM_MAT;

    /* fragments of one 16-wide slice: hi, lo of two row blocks and the weights of two column blocks */
    struct frags { bf16x8 fa[2], fl[2], fb[2]; };
    auto read_frags = [&](frags &f, int ks) {
#pragma unroll
        for (int b = 0; b < 2; b++) {
            f.fa[b] = gm_frag(lds + fa_off + 32 * b * GM_ROWB + ks * 32);
            f.fl[b] = gm_frag(lds + GM_MAT + fa_off + 32 * b * GM_ROWB + ks * 32);
            f.fb[b] = gm_frag(lds + fb_off + 32 * b * GM_ROWB + ks * 32);
        }
    };
    auto mma = [&](const frags &f) {
        /* four independent accumulators between two products into the same one */
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.fl[a], f.fb[b], acc[a][b], 0, 0, 0);
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.fa[a], f.fb[b], acc[a][b], 0, 0, 0);
    };

    for (int kt = 0; kt < tiles; kt++) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<u32x4 *>(lds + st_off + 32 * i * GM_ROWB) = ra[i];
            *reinterpret_cast<u32x4 *>(lds + GM_MAT + st_off + 32 * i * GM_ROWB) = rl[i];
            *reinterpret_cast<u32x4 *>(lds + 2 * GM_MAT + st_off + 32 * i * GM_ROWB) = rb[i];
        }
        __syncthreads();
        if (kt + 1 < tiles) fetch(kt + 1);
        /* the fragments of slice ks+1 are read while slice ks is multiplied */
        frags f0, f1;
        read_frags(f0, 0);
        read_frags(f1, 1);
        mma(f0);
        read_frags(f0, 2);
        mma(f1);
        read_frags(f1, 3);
        mma(f0);
        mma(f1);
    }

    /* accumulator element v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 */
    float *Cs = C + (size_t)sp * plane_stride;
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int col = nt * GM_TILE + 64 * wn + 32 * b + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = mt * GM_TILE + 64 * wm + 32 * a + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < M) Cs[(size_t)row * ldc + col] = acc[a][b][v];
            }
        }
}

/* ---- the same product, 128 x 256 tile, one workgroup per CU ---------------------------
 * What bounds the 128 x 128 kernel above is the LDS: a 64 x 64 wave tile reads 24 KB of fragments
 * (two activation planes and the weights) per 32 matrix instructions, three quarters of the LDS
 * bandwidth of a CU with four waves at it, and every K step is a store -> barrier -> read chain.
 * Here a wave owns 128 rows x 64 columns: the weights of its 64 columns are nobody else's in the
 * workgroup, so they go from global memory straight into the B operand registers, and only the
 * activation planes, which all four waves share, pass through the LDS: 8 KB of fragment reads per
 * 16 matrix instructions, half the LDS bandwidth.  Two LDS stages: the planes of K step kt + 1
 * are written while step kt is multiplied, one barrier per step; the global loads of step kt + 2
 * are in flight meanwhile (every request unconditional, so the waits count exactly).  One
 * workgroup of four waves per CU (a wave may then use the whole register file of its SIMD: 128
 * accumulator registers, two sets of weight registers, two sets of fragments).
 * The k order inside a matrix instruction is free as long as both operands agree: lane group g
 * (lane / 32) takes k = 32 g + 8 ks .. + 8 of the 64-wide step in slice ks.
 * A lane's operand is 8 consecutive k of ONE weight row, and the 32 lanes of a group are 32
 * different rows: read from the row-major matrix, every load instruction touches 32 lines 6 KB
 * apart, and the CU's address pipeline, not the matrix cores, sets the pace (measured: 434 against
 * 518 TFLOP/s).  The backbone therefore keeps a second copy of its matrices in fragment order,
 * written once at upload by vt_frag_layout_kernel: every load is then 1 KB of consecutive bytes.
 * Needs N % 256 == 0 and K % 128 == 0: a cut is a whole number of pairs of K steps, and the cuts of one
 * product may differ by one pair (64 steps in 5 cuts: 14, 14, 12, 12, 12), so that the cut count can be
 * chosen to fill the CUs (48 tiles x 5 = 240 items) rather than to divide K. */
#define GW_TM 128
#define GW_TN 256
#define GW_PLANE (GW_TM * GM_ROWB)
#define GW_STAGE (2 * GW_PLANE)
#define GW_LDS (2 * GW_STAGE)

struct gw_bregs { u32x4 v[2][4]; };          /* [column block][slice] */
struct gw_aregs { u32x4 hi[4], lo[4]; };     /* staging: rows lr + 32 i */
struct gw_frags { bf16x8 hi[4], lo[4]; };    /* one 16-wide slice of the 128 rows, both planes */

/* A launch runs one or two sets of equal work items; workgroup i takes item i of each set in turn (a set
 * may have fewer items than the grid).  The second set lets a product whose tile count is not a multiple
 * of the CU count finish its last tiles as K cuts spread over all CUs inside the same launch. */
struct gw_part {
    float *C;                /* output of this set: `splits` planes, plane_stride floats apart, row pitch ldc */
    const uint16_t *Wf;      /* fragment-order weights of the set's first column */
    size_t plane_stride;
    int ldc, n_tiles, splits, k_pairs;   /* k_pairs: K / 128, dealt out over the `splits` cuts */
    /* gate|up product in the paired column order (vt_launch_frag_layout with pair = 1): instead of C, the
     * (hi, lo) planes of SiLU(gate) * up, row pitch ldh; the set's first column is h column h_col0 */
    uint16_t *h_hi, *h_lo;
    int ldh, h_col0;
};
struct gw_plan { gw_part part[2]; int n_parts; };

/* Stores of results that another workgroup of the SAME launch will read (the persistent layer kernel
 * below): written through to memory, because every XCD has its own L2.  COH = false: plain stores (a
 * kernel boundary makes them visible). */
template <bool COH> __device__ __forceinline__ void gw_st_f32(float *p, float v) {
    if (COH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}
template <bool COH> __device__ __forceinline__ void gw_st_u16(uint16_t *p, uint16_t v) {
    if (COH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

/* Item `id` of the set P (id < m_tiles * P.n_tiles * P.splits): one 128 x 256 tile over one K cut.  Returns
 * the item's M tile. */
template <bool COH>
__device__ __forceinline__ int gw_run_item(const gw_part &P, int id, const uint16_t *Ahi, const uint16_t *Alo, int M,
                                           int K, int m_tiles, unsigned char *lds) {
    const int n_tiles = P.n_tiles, ldc = P.ldc, items = m_tiles * n_tiles * P.splits;
    float *C = P.C;
    const uint16_t *Wf = P.Wf;
    const size_t plane_stride = P.plane_stride;
    /* Slot id lands on XCD id % 8.  An XCD takes a run of consecutive items, M tile fastest, then N tile,
     * then K cut: the M tiles of a (K cut, N tile) pair share its weights, the N tiles of a K cut share the
     * activation planes of that cut, and both then leave the memory side once per XCD instead of once per
     * workgroup (the two slices are the same size: 128 rows x 4 bytes against 256 rows x 2 bytes). */
    const int li = (items & 7) == 0 ? (id & 7) * (items >> 3) + (id >> 3) : id;
    const int mt = li % m_tiles, ci = li / m_tiles, nt = ci % n_tiles, sp = ci / n_tiles;
    const int t = (int)threadIdx.x, lane = t & 63, wave = t >> 6;
    const int lr = t >> 3, lc = t & 7;               /* staging: row lr + 32 i, 16-byte chunk lc */
    /* K is dealt out in pairs of 64-wide steps; the first k_pairs % splits cuts take one pair more */
    const int pq = P.k_pairs / P.splits, pr = P.k_pairs % P.splits;
    const int k0 = 2 * GM_BK * (sp * pq + (sp < pr ? sp : pr)), tiles = 2 * (pq + (sp < pr ? 1 : 0));

    /* rows past M read row 0 of the tile again: their products land in accumulator rows that are
     * never stored (the rows of a matrix instruction do not mix), so nothing has to be zeroed */
    const uint16_t *pa[4], *pl[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int gm = mt * GW_TM + lr + 32 * i;
        const size_t ao = (size_t)(gm < M ? gm : mt * GW_TM) * K + k0 + lc * 8;
        pa[i] = Ahi + ao;
        pl[i] = Alo + ao;
    }
    const size_t b_blk = (size_t)32 * K;

    auto fetch_a = [&](gw_aregs &r, int kt) {
        const int adv = (kt < tiles ? kt : tiles - 1) * GM_BK;      /* past the end: the last step once more */
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r.hi[i] = gm_ld(pa[i] + adv);
            r.lo[i] = gm_ld(pl[i] + adv);
        }
    };
    /* weights in fragment order (vt_frag_layout_kernel): the 1 KB of slice j of K step ks of column block
     * nb is contiguous, lane l's 16 bytes at 16 l */
    const uint16_t *pf = Wf + (size_t)(nt * GW_TN + 64 * wave) * K + (size_t)k0 * 32 + lane * 8;
    auto fetch_b_slice = [&](gw_bregs &r, int kt, int j) {
        const int adv = (kt < tiles ? kt : tiles - 1) * 2048;
        r.v[0][j] = gm_ld(pf + adv + 512 * j);
        r.v[1][j] = gm_ld(pf + b_blk + adv + 512 * j);
    };
    const int st_off = lr * GM_ROWB + lc * 16;
    auto store_a = [&](const gw_aregs &r, int stage) {
        unsigned char *base = lds + stage * GW_STAGE + st_off;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<u32x4 *>(base + 32 * i * GM_ROWB) = r.hi[i];
            *reinterpret_cast<u32x4 *>(base + GW_PLANE + 32 * i * GM_ROWB) = r.lo[i];
        }
    };

    f32x16 acc[4][2];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    const int fa_off = (lane & 31) * GM_ROWB + (lane >> 5) * 64;
    auto read_frags = [&](gw_frags &f, int stage, int ks) {
        const unsigned char *base = lds + stage * GW_STAGE + fa_off + ks * 16;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            f.hi[a] = gm_frag(base + 32 * a * GM_ROWB);
            f.lo[a] = gm_frag(base + GW_PLANE + 32 * a * GM_ROWB);
        }
    };
    auto mma = [&](const gw_frags &f, const gw_bregs &rb, int ks) {
        const bf16x8 b0 = __builtin_bit_cast(bf16x8, rb.v[0][ks]), b1 = __builtin_bit_cast(bf16x8, rb.v[1][ks]);
#pragma unroll
        for (int a = 0; a < 4; a++) {
            acc[a][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.lo[a], b0, acc[a][0], 0, 0, 0);
            acc[a][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.lo[a], b1, acc[a][1], 0, 0, 0);
        }
#pragma unroll
        for (int a = 0; a < 4; a++) {
            acc[a][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.hi[a], b0, acc[a][0], 0, 0, 0);
            acc[a][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.hi[a], b1, acc[a][1], 0, 0, 0);
        }
    };

    /* One K step: stage `stage` holds the planes of step kt and `cur` its weights; `ra` holds the planes
     * of step kt + 1 (requested a step ago); f0 already holds the fragments of slice 0.  Four regions of
     * sixteen matrix instructions each; the other instructions of a region (the fragment reads of the next
     * slice, in the first region also the LDS stores of step kt + 1 and the plane requests of step kt + 2,
     * in the others the two weight requests that refill the slice just used) are dealt out between the
     * matrix instructions, one after every second, so that the matrix pipe never waits for a block of
     * them to issue.  The step's one barrier stands in front of the last region: by then every wave has
     * issued (and waited for) its stores into the other stage and its last reads of this one, so the first
     * fragments of step kt + 1 are read under the last sixteen matrix instructions of step kt. */
    gw_aregs ra;
    gw_frags f0, f1;
#define GW_FENCE() __builtin_amdgcn_sched_barrier(0)
#define GW_MFMA2() __builtin_amdgcn_sched_group_barrier(0x008, 2, 0)
#define GW_DSR1() __builtin_amdgcn_sched_group_barrier(0x100, 1, 0)
#define GW_DSW1() __builtin_amdgcn_sched_group_barrier(0x200, 1, 0)
#define GW_VMR1() __builtin_amdgcn_sched_group_barrier(0x020, 1, 0)
    auto step = [&](int kt, int stage, gw_bregs &cur) {
        GW_FENCE();
        store_a(ra, stage ^ 1);
        fetch_a(ra, kt + 2);
        read_frags(f1, stage, 1);
        mma(f0, cur, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) { GW_MFMA2(); GW_DSR1(); GW_DSW1(); GW_VMR1(); }
        GW_FENCE();
        fetch_b_slice(cur, kt + 2, 0);
        read_frags(f0, stage, 2);
        mma(f1, cur, 1);
#pragma unroll
        for (int i = 0; i < 8; i++) { GW_MFMA2(); GW_DSR1(); if (i < 2) GW_VMR1(); }
        GW_FENCE();
        fetch_b_slice(cur, kt + 2, 1);
        read_frags(f1, stage, 3);
        mma(f0, cur, 2);
#pragma unroll
        for (int i = 0; i < 8; i++) { GW_MFMA2(); GW_DSR1(); if (i < 2) GW_VMR1(); }
        GW_FENCE();
        __syncthreads();
        GW_FENCE();
        fetch_b_slice(cur, kt + 2, 2);
        read_frags(f0, stage ^ 1, 0);
        mma(f1, cur, 3);
#pragma unroll
        for (int i = 0; i < 8; i++) { GW_MFMA2(); GW_DSR1(); if (i < 2) GW_VMR1(); }
        GW_FENCE();
        fetch_b_slice(cur, kt + 2, 3);
    };

    gw_bregs b0, b1;
    fetch_a(ra, 0);
#pragma unroll
    for (int j = 0; j < 4; j++) fetch_b_slice(b0, 0, j);
    store_a(ra, 0);
    fetch_a(ra, 1);
#pragma unroll
    for (int j = 0; j < 4; j++) fetch_b_slice(b1, 1, j);
    __syncthreads();
    read_frags(f0, 0, 0);
    for (int kt = 0; kt < tiles; kt += 2) {
        step(kt, 0, b0);
        step(kt + 1, 1, b1);
    }
#undef GW_MFMA2
#undef GW_DSR1
#undef GW_DSW1
#undef GW_VMR1
#undef GW_FENCE

    /* accumulator element v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 */
    if (P.h_hi) {
        /* a wave's two column blocks are the gates and the ups of the same 32 h columns
         * (voxtral_tts_llm.c:346-350) */
        const int hc = P.h_col0 + nt * (GW_TN / 2) + 32 * wave + (lane & 31);
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = mt * GW_TM + 32 * a + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const float g = acc[a][0][v], u = acc[a][1][v];
                const float h = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), u);
                unsigned sh, sl;
                vt_split_planes2(h, 0.f, sh, sl);
                if (row < M) {
                    gw_st_u16<COH>(P.h_hi + (size_t)row * P.ldh + hc, (uint16_t)sh);
                    gw_st_u16<COH>(P.h_lo + (size_t)row * P.ldh + hc, (uint16_t)sl);
                }
            }
    } else {
    float *Cs = C + (size_t)sp * plane_stride;
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int col = nt * GW_TN + 64 * wave + 32 * b + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = mt * GW_TM + 32 * a + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < M) gw_st_f32<COH>(Cs + (size_t)row * ldc + col, acc[a][b][v]);
            }
        }
    }
    __syncthreads();                 /* the next item refills the LDS stages */
    return mt;
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
vt_gemm_wide_kernel(gw_plan plan, const uint16_t *Ahi, const uint16_t *Alo, int M, int K, int m_tiles) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int id = (int)blockIdx.x;
    for (int pi = 0; pi < plan.n_parts; pi++) {
        const gw_part &P = plan.part[pi];
        if (id < m_tiles * P.n_tiles * P.splits) (void)gw_run_item<false>(P, id, Ahi, Alo, M, K, m_tiles, lds);
    }
}

/* ---- one layer's products as ONE persistent launch ----------------------------------------------
 * Behind the attention, a prefill layer is a chain of four products with row passes between them
 * (voxtral_tts_llm.c:326-366): output projection -> residual + RMSNorm -> gate|up with SiLU*up -> down
 * projection -> residual + next layer's RMSNorm -> next layer's q|k|v.  As separate launches every link of
 * that chain pays a dispatch, an empty device at its start and a drain at its end.  Here the whole chain
 * is one list of work items in dependency order (tile items of the products, two-row items of the row
 * passes); workgroup w of a grid of one workgroup per CU takes items w, w + G, w + 2G, ...  An item of
 * M tile m (128 rows) waits until the items it reads from have counted themselves into that tile's
 * counter (a bounded poll, as in vt_device.h), so only the rows that depend on each other wait for each
 * other, a workgroup that is done early goes on to its next item, and nothing is dispatched in between.
 * Items are numbered in dependency order and every workgroup takes its items in ascending order, so the
 * lowest unfinished item can always run: the grid cannot deadlock as long as it is resident at once.
 *
 * Data that one item writes and another reads crosses XCDs, each with an L2 of its own: results are
 * written through (agent-scope stores) and every buffer of the chain is written exactly once per launch,
 * before anybody reads it, so no L2 can hold an older copy of a line and the products keep reading their
 * operands through the cache; the row passes read past it (each value is read once anyway).
 * The arithmetic is that of the separate launches, element for element: same K cuts, same tile walk, the
 * same sums in the same order. */
#define PF_MAX_TILES 64                 /* M tiles (8192 rows) */
enum { PF_GEMM = 0, PF_NORM = 1, PF_TAIL = 2 };
enum { PF_S_WO = 0, PF_S_NORM1, PF_S_W13, PF_S_W13T, PF_S_TAIL, PF_S_W2, PF_S_NORM2, PF_S_QKV, PF_N_STAGES };

struct pf_stage {
    int type, first, count;          /* items first .. first + count - 1 of the launch */
    int dep[2];                      /* stages whose items of the same M tile must all be done (-1: none) */
    /* PF_GEMM */
    gw_part P;
    const uint16_t *Ahi, *Alo;
    int K;
    /* PF_NORM: x += sum of `splits` planes; planes of rmsnorm(x) * w (w may be NULL) */
    float *x;
    const float *part;
    int splits;
    size_t part_stride;
    const float *w;
    uint16_t *hi, *lo;
    /* PF_TAIL: vt_swiglu_pair_tail_kernel's arguments */
    int ldh, h_col0, planes, tw;
};

struct pf_plan {
    pf_stage st[PF_N_STAGES];
    int total, M, m_tiles;
    unsigned *cnt;                   /* [PF_N_STAGES][PF_MAX_TILES], zero at launch */
    unsigned target[PF_N_STAGES];    /* items of a full M tile in each stage (the last tile of a row stage may have fewer: see pf_target) */
    int *abort_flag;
    unsigned long long timeout;
};

/* Buffer accesses with the device-scope bit (sc1): `p` is the same in every lane (it becomes the
 * descriptor's base), the element index is per lane and stays below 2^31 bytes (the launcher checks the
 * buffer sizes). */
__device__ __forceinline__ __amdgpu_buffer_rsrc_t pf_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, 0x7ffffff0, 0x00020000);
}
__device__ __forceinline__ f32x4 pf_ldc4(const float *p, size_t idx) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(pf_rsrc(p), (int)(idx * 4), 0, 16 /* sc1 */);
    return f32x4{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
}
__device__ __forceinline__ void pf_stc4(float *p, size_t idx, f32x4 v) {
    const u32x4 u = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
    __builtin_amdgcn_raw_buffer_store_b128(u, pf_rsrc(p), (int)(idx * 4), 0, 16 /* sc1 */);
}
__device__ __forceinline__ void pf_stc2(uint16_t *p, size_t idx, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, pf_rsrc(p), (int)(idx * 2), 0, 16 /* sc1 */);
}

/* Items of M tile m that stage s counts: all of a tile's product items, or one per two rows of the tile */
__device__ __forceinline__ unsigned pf_target(const pf_plan &pl, int s, int m) {
    if (pl.st[s].type == PF_GEMM) return pl.target[s];
    const int rows = min(GW_TM, pl.M - m * GW_TM);
    return (unsigned)((rows + 1) / 2);
}

/* residual + RMSNorm + plane split of rows row0, row0 + 1 (vt_residual_norm_split_kernel's arithmetic, 256
 * threads per row); all loads of both rows are requested before the first is used */
__device__ __forceinline__ void pf_norm_rows(const pf_stage &st, int row0, int M, float *red) {
    constexpr int NJ = VT_DIM / 1024;
    const int t = (int)threadIdx.x;
    f32x4 v[2][NJ], pp[2][NJ];
    const int n_rows = min(2, M - row0);
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const size_t row = (size_t)(r < n_rows ? row0 + r : row0);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const size_t i = row * VT_DIM + 4 * ((size_t)t + 256 * j);
            v[r][j] = pf_ldc4(st.x, i);
            pp[r][j] = pf_ldc4(st.part, i);
        }
    }
    for (int s = 1; s < st.splits; s++) {
        f32x4 q[2][NJ];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const size_t row = (size_t)(r < n_rows ? row0 + r : row0);
#pragma unroll
            for (int j = 0; j < NJ; j++) q[r][j] = pf_ldc4(st.part + (size_t)s * st.part_stride, row * VT_DIM + 4 * ((size_t)t + 256 * j));
        }
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                f32x4 &p = pp[r][j];
                const f32x4 qq = q[r][j];
                p.x = __fadd_rn(p.x, qq.x); p.y = __fadd_rn(p.y, qq.y); p.z = __fadd_rn(p.z, qq.z); p.w = __fadd_rn(p.w, qq.w);
            }
    }
    float ss[2] = {0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 2; r++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            f32x4 a = v[r][j];
            const f32x4 p = pp[r][j];
            a.x = __fadd_rn(a.x, p.x); a.y = __fadd_rn(a.y, p.y); a.z = __fadd_rn(a.z, p.z); a.w = __fadd_rn(a.w, p.w);
            v[r][j] = a;
            if (r < n_rows) pf_stc4(st.x, (size_t)(row0 + r) * VT_DIM + 4 * ((size_t)t + 256 * j), a);
            ss[r] = fmaf(a.x, a.x, ss[r]); ss[r] = fmaf(a.y, a.y, ss[r]);
            ss[r] = fmaf(a.z, a.z, ss[r]); ss[r] = fmaf(a.w, a.w, ss[r]);
        }
    if (!st.w) return;
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const float w_sum = vt_wave_sum(ss[r]);
        if (vt_lane() == 0) red[4 * r + vt_wave()] = w_sum;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const float tot = (red[4 * r] + red[4 * r + 1]) + (red[4 * r + 2] + red[4 * r + 3]);
        const float inv = 1.0f / sqrtf(tot / (float)VT_DIM + VT_EPS);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int c = 4 * (t + 256 * j);
            const f32x4 g = *reinterpret_cast<const f32x4 *>(st.w + c);
            u32x2 sph, spl;
            vt_split_planes4(__fmul_rn(__fmul_rn(v[r][j].x, inv), g.x), __fmul_rn(__fmul_rn(v[r][j].y, inv), g.y),
                             __fmul_rn(__fmul_rn(v[r][j].z, inv), g.z), __fmul_rn(__fmul_rn(v[r][j].w, inv), g.w), sph, spl);
            if (r < n_rows) {
                pf_stc2(st.hi, (size_t)(row0 + r) * VT_DIM + c, sph);
                pf_stc2(st.lo, (size_t)(row0 + r) * VT_DIM + c, spl);
            }
        }
    }
    __syncthreads();                 /* red is free again */
}

/* the K-cut tail of the paired gate|up product for rows row0, row0 + 1 (vt_swiglu_pair_tail_kernel's arithmetic;
 * tw / 8 threads per row, tw <= 2048) */
__device__ __forceinline__ void pf_tail_rows(const pf_stage &st, int row0, int M) {
    const int per_row = st.tw / 8, q = (int)threadIdx.x;
    if (q >= per_row) return;
    const int blk = q >> 3, c = (q & 7) * 4;
    const size_t stride = st.part_stride;
    for (int r = 0; r < 2 && row0 + r < M; r++) {
        const size_t at_in = (size_t)(row0 + r) * st.tw + 64 * blk + c;
        f32x4 g = pf_ldc4(st.part, at_in), u = pf_ldc4(st.part, at_in + 32);
        for (int p = 1; p < st.planes; p++) {
            const f32x4 g2 = pf_ldc4(st.part + p * stride, at_in), u2 = pf_ldc4(st.part + p * stride, at_in + 32);
            g.x = __fadd_rn(g.x, g2.x); g.y = __fadd_rn(g.y, g2.y); g.z = __fadd_rn(g.z, g2.z); g.w = __fadd_rn(g.w, g2.w);
            u.x = __fadd_rn(u.x, u2.x); u.y = __fadd_rn(u.y, u2.y); u.z = __fadd_rn(u.z, u2.z); u.w = __fadd_rn(u.w, u2.w);
        }
        const float a = __fmul_rn(__fdiv_rn(g.x, __fadd_rn(1.0f, expf(-g.x))), u.x);
        const float b = __fmul_rn(__fdiv_rn(g.y, __fadd_rn(1.0f, expf(-g.y))), u.y);
        const float cc = __fmul_rn(__fdiv_rn(g.z, __fadd_rn(1.0f, expf(-g.z))), u.z);
        const float d = __fmul_rn(__fdiv_rn(g.w, __fadd_rn(1.0f, expf(-g.w))), u.w);
        u32x2 sph, spl;
        vt_split_planes4(a, b, cc, d, sph, spl);
        const size_t at = (size_t)(row0 + r) * st.ldh + st.h_col0 + 32 * blk + c;
        pf_stc2(st.hi, at, sph);
        pf_stc2(st.lo, at, spl);
    }
}

/* Waits until stage `dep` has counted all its items of M tile m; false when the spin budget ran out or
 * another workgroup has given up (then everybody leaves the kernel). */
__device__ __forceinline__ bool pf_wait(const pf_plan &pl, int dep, int m, int *lds_ok) {
    if (threadIdx.x < VT_WAVE) {
        const unsigned want = pf_target(pl, dep, m);
        const unsigned *c = pl.cnt + dep * PF_MAX_TILES + m;
        const unsigned long long t0 = wall_clock64();
        int ok = 1;
        while (__hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
            if (__hip_atomic_load(pl.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
                wall_clock64() - t0 > pl.timeout) {
                ok = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(8);
        }
        if (!ok && threadIdx.x == 0) __hip_atomic_store(pl.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) *lds_ok = ok;
    }
    __syncthreads();
    vt_compiler_fence();
    return *lds_ok != 0;
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
vt_prefill_layer_kernel(pf_plan pl) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ float s_red[8];
    __shared__ int s_ok;
    for (int g = (int)blockIdx.x; g < pl.total; g += (int)gridDim.x) {
        int s = 0;
        while (s + 1 < PF_N_STAGES && g >= pl.st[s].first + pl.st[s].count) s++;
        const pf_stage &st = pl.st[s];
        const int i = g - st.first;
        int m;
        if (st.type == PF_GEMM) {
            /* the M tile of item i, as gw_run_item maps it */
            const int items = st.count;
            const int li = (items & 7) == 0 ? (i & 7) * (items >> 3) + (i >> 3) : i;
            m = li % pl.m_tiles;
        } else {
            m = (2 * i) / GW_TM;
        }
        for (int d = 0; d < 2; d++)
            if (st.dep[d] >= 0 && !pf_wait(pl, st.dep[d], m, &s_ok)) return;
        if (st.type == PF_GEMM) (void)gw_run_item<true>(st.P, i, st.Ahi, st.Alo, pl.M, st.K, pl.m_tiles, lds);
        else if (st.type == PF_NORM) pf_norm_rows(st, 2 * i, pl.M, s_red);
        else pf_tail_rows(st, 2 * i, pl.M);
        /* this item's results are in memory before it counts itself in */
        vt_compiler_fence();
        __builtin_amdgcn_s_waitcnt(0x0F70);
        vt_compiler_fence();
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_fetch_add(pl.cnt + s * PF_MAX_TILES + m, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

static int pf_ready(void) {
    static int state = 0;                /* 0 not asked, 1 usable, -1 not */
    if (state) return state > 0;
    state = -1;
    if (hipFuncSetAttribute((const void *)vt_prefill_layer_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, GW_LDS) !=
        hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    /* the item counters need every workgroup of the grid on the device at once */
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, vt_prefill_layer_kernel, 256, GW_LDS) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (per_cu >= 1) state = 1;
    return state > 0;
}

int vt_prefill_layer_usable(int M) {
    /* the sc1 accesses take 32-bit byte offsets: the largest buffer (the K-cut planes) stays below 2 GiB */
    return M >= 1 && (M + GW_TM - 1) / GW_TM <= PF_MAX_TILES && (size_t)M * VT_FFN * 4 < ((size_t)1 << 31) && pf_ready();
}

size_t vt_prefill_layer_counter_bytes(void) { return sizeof(unsigned) * PF_N_STAGES * PF_MAX_TILES; }

int vt_launch_prefill_layer(const vt_prefill_layer_args &a) {
    if (!vt_prefill_layer_usable(a.M)) { vt_set_error("prefill layer kernel: not usable for %d rows", a.M); return -1; }
    const int M = a.M, m_tiles = (M + GW_TM - 1) / GW_TM;
    const bool tail = m_tiles == 4;      /* 4 x 72 gate|up tiles on 256 CUs: the last 8 N tiles get their K cut (as vt_launch_gemm_frag_swiglu's callers do) */
    const int n_tail = tail ? 8 * GW_TN : 0, n_main = 2 * VT_FFN - n_tail;
    const size_t ps = (size_t)M * VT_DIM;
    pf_plan pl = {};
    pl.M = M;
    pl.m_tiles = m_tiles;
    pl.cnt = a.cnt;
    pl.abort_flag = a.abort_flag;
    pl.timeout = a.timeout;
    for (int s = 0; s < PF_N_STAGES; s++) { pl.st[s].dep[0] = pl.st[s].dep[1] = -1; pl.st[s].type = PF_GEMM; }
    auto gemm = [&](int s, float *C, const uint16_t *Wf, size_t plane_stride, int ldc, int N, int splits, int K,
                    const uint16_t *Ahi, const uint16_t *Alo, uint16_t *h_hi, uint16_t *h_lo, int dep0, int dep1) {
        pf_stage &st = pl.st[s];
        st.type = PF_GEMM;
        st.P = gw_part{C, Wf, plane_stride, ldc, N / GW_TN, splits, K / (2 * GM_BK), h_hi, h_lo, VT_FFN, 0};
        st.Ahi = Ahi; st.Alo = Alo; st.K = K;
        st.count = Wf ? m_tiles * (N / GW_TN) * splits : 0;
        st.dep[0] = dep0; st.dep[1] = dep1;
        pl.target[s] = (unsigned)((N / GW_TN) * splits);
    };
    auto rows = [&](int s, int type, int dep0, bool present) {
        pf_stage &st = pl.st[s];
        st.type = type;
        st.count = present ? (M + 1) / 2 : 0;
        st.dep[0] = dep0;
    };
    gemm(PF_S_WO, a.part_a, a.wo_f, ps, VT_DIM, VT_DIM, a.fo, VT_Q_DIM, a.attn_hi, a.attn_lo, NULL, NULL, -1, -1);
    rows(PF_S_NORM1, PF_NORM, PF_S_WO, true);
    { pf_stage &st = pl.st[PF_S_NORM1]; st.x = a.x; st.part = a.part_a; st.splits = a.fo; st.part_stride = ps; st.w = a.ffn_norm; st.hi = a.n1_hi; st.lo = a.n1_lo; }
    gemm(PF_S_W13, NULL, a.w13_f, 0, 0, n_main, 1, VT_DIM, a.n1_hi, a.n1_lo, a.h_hi, a.h_lo, PF_S_NORM1, -1);
    gemm(PF_S_W13T, a.tail, tail ? a.w13_f + (size_t)n_main * VT_DIM : NULL, (size_t)M * n_tail, n_tail, tail ? n_tail : GW_TN,
         VT_W13_TAIL_CUT, VT_DIM, a.n1_hi, a.n1_lo, NULL, NULL, PF_S_NORM1, -1);
    rows(PF_S_TAIL, PF_TAIL, PF_S_W13T, tail);
    { pf_stage &st = pl.st[PF_S_TAIL]; st.part = a.tail; st.planes = VT_W13_TAIL_CUT; st.part_stride = (size_t)M * n_tail; st.tw = n_tail;
      st.ldh = VT_FFN; st.h_col0 = n_main / 2; st.hi = a.h_hi; st.lo = a.h_lo; }
    gemm(PF_S_W2, a.part_b, a.w2_f, ps, VT_DIM, VT_DIM, a.fo, VT_FFN, a.h_hi, a.h_lo, NULL, NULL, PF_S_W13, tail ? PF_S_TAIL : -1);
    rows(PF_S_NORM2, PF_NORM, PF_S_W2, true);
    { pf_stage &st = pl.st[PF_S_NORM2]; st.x = a.x; st.part = a.part_b; st.splits = a.fo; st.part_stride = ps; st.w = a.next_norm; st.hi = a.n2_hi; st.lo = a.n2_lo; }
    gemm(PF_S_QKV, a.qkv, a.qkv_next_f, (size_t)M * VT_QKV_DIM, VT_QKV_DIM, VT_QKV_DIM, a.fq, VT_DIM, a.n2_hi, a.n2_lo, NULL, NULL,
         PF_S_NORM2, -1);
    int first = 0;
    for (int s = 0; s < PF_N_STAGES; s++) { pl.st[s].first = first; first += pl.st[s].count; }
    pl.total = first;
    const int grid = g_vt.n_cu < pl.total ? g_vt.n_cu : pl.total;
    hipLaunchKernelGGL(vt_prefill_layer_kernel, dim3(grid), dim3(256), GW_LDS, g_vt.stream, pl);
    return vt_check(hipGetLastError(), "prefill layer launch");
}

static int gm_blocks(size_t n);

int vt_gemm_frag_shape_ok(int N, int K, int splits) {
    return N % GW_TN == 0 && K % (2 * GM_BK) == 0 && splits >= 1 && splits <= K / (2 * GM_BK);
}

static int gw_ready(void) {
    static int attr_set = 0;
    if (!attr_set) {
        if (vt_check(hipFuncSetAttribute((const void *)vt_gemm_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         GW_LDS), "product LDS size"))
            return 0;
        attr_set = 1;
    }
    return 1;
}

void vt_launch_gemm_frag(float *d_C, int ldc, size_t plane_stride, const uint16_t *d_Ahi, const uint16_t *d_Alo,
                         const uint16_t *d_Wf, int M, int N, int K, int splits) {
    if (!gw_ready()) return;
    const int m_tiles = (M + GW_TM - 1) / GW_TM;
    gw_plan plan = {};
    plan.n_parts = 1;
    plan.part[0] = gw_part{d_C, d_Wf, plane_stride, ldc, N / GW_TN, splits, K / (2 * GM_BK), NULL, NULL, 0, 0};
    hipLaunchKernelGGL(vt_gemm_wide_kernel, dim3(m_tiles * (N / GW_TN) * splits), dim3(256), GW_LDS, g_vt.stream,
                       plan, d_Ahi, d_Alo, M, K, m_tiles);
}

/* gate|up product with the SiLU(gate) * up epilogue (weights in the paired fragment order): the first n_main
 * columns go straight into the planes d_hhi / d_hlo [M, ldh]; the other n_tail columns (0: none) have K cut
 * in tail_splits and leave fp32 planes d_tail [tail_splits][M, n_tail] in the paired column order, which
 * vt_launch_swiglu_pair_tail turns into the last n_tail / 2 plane columns.  One launch. */
void vt_launch_gemm_frag_swiglu(uint16_t *d_hhi, uint16_t *d_hlo, int ldh, float *d_tail, const uint16_t *d_Ahi,
                                const uint16_t *d_Alo, const uint16_t *d_Wf, int M, int n_main, int n_tail, int K,
                                int tail_splits) {
    if (!gw_ready()) return;
    const int m_tiles = (M + GW_TM - 1) / GW_TM;
    gw_plan plan = {};
    plan.n_parts = n_tail > 0 ? 2 : 1;
    plan.part[0] = gw_part{NULL, d_Wf, 0, 0, n_main / GW_TN, 1, K / (2 * GM_BK), d_hhi, d_hlo, ldh, 0};
    int items = m_tiles * (n_main / GW_TN);
    if (n_tail > 0) {
        plan.part[1] = gw_part{d_tail, d_Wf + (size_t)n_main * K, (size_t)M * n_tail, n_tail, n_tail / GW_TN, tail_splits,
                               K / (2 * GM_BK), NULL, NULL, 0, 0};
        const int items1 = m_tiles * (n_tail / GW_TN) * tail_splits;
        if (items1 > items) items = items1;
    }
    hipLaunchKernelGGL(vt_gemm_wide_kernel, dim3(items), dim3(256), GW_LDS, g_vt.stream, plan, d_Ahi, d_Alo, M, K, m_tiles);
}

/* Row-major W[N, K] (N % 32 == 0, K % 64 == 0) -> fragment order: the 16 bytes that lane l = 32 g + n % 32
 * feeds to slice j of K step ks of column block nb = n / 32, i.e. W[n][64 ks + 32 g + 8 j .. + 8], go to
 * 16-byte slot ((nb * K/64 + ks) * 4 + j) * 64 + l.  A block of 32 rows occupies the same 32 K elements
 * in both layouts. */
/* pair: W is a gate|up matrix with (gate, up) rows interleaved; fragment column n' of every 64 takes row
 * 64 (n'/64) + 2 (n' % 32) + (n' % 64) / 32, so that a wave of the product (64 columns) holds the gates of 32
 * h columns in its first column block and their ups in the second. */
__global__ void vt_frag_layout_kernel(u32x4 *out, const uint16_t *W, size_t n_slots, int K, int pair) {
    const int ksteps = K / GM_BK;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_slots; i += (size_t)gridDim.x * blockDim.x) {
        const int l = (int)(i & 63), j = (int)((i >> 6) & 3);
        const size_t blk = i >> 8;
        const int ks = (int)(blk % ksteps);
        const size_t nb = blk / ksteps;
        size_t n = nb * 32 + (l & 31);
        if (pair) n = (nb >> 1) * 64 + 2 * (l & 31) + (nb & 1);
        out[i] = gm_ld(W + n * K + 64 * ks + 32 * (l >> 5) + 8 * j);
    }
}

void vt_launch_frag_layout(uint16_t *d_Wf, const uint16_t *d_W, int N, int K, int pair) {
    const size_t n_slots = (size_t)N * K / 8;
    hipLaunchKernelGGL(vt_frag_layout_kernel, dim3(gm_blocks(n_slots)), dim3(256), 0, g_vt.stream, (u32x4 *)d_Wf, d_W,
                       n_slots, K, pair);
}

int vt_gemm_shape_ok(int M, int N, int K, int splits) {
    return M >= 1 && splits >= 1 && N % GM_TILE == 0 && K % splits == 0 && (K / splits) % GM_BK == 0;
}

void vt_launch_gemm_ex(float *d_C, int ldc, size_t plane_stride, const uint16_t *d_Ahi, const uint16_t *d_Alo,
                       const uint16_t *d_W, int M, int N, int K, int splits) {
    const int m_tiles = (M + GM_TILE - 1) / GM_TILE, n_tiles = N / GM_TILE;
    hipLaunchKernelGGL(vt_gemm_mfma_kernel, dim3(m_tiles * n_tiles * splits), dim3(256), 0, g_vt.stream,
                       d_C, d_Ahi, d_Alo, d_W, M, N, K, K / splits, m_tiles, n_tiles, ldc, plane_stride);
}

void vt_launch_gemm(float *d_C, const uint16_t *d_Ahi, const uint16_t *d_Alo, const uint16_t *d_W,
                    int M, int N, int K, int splits) {
    vt_launch_gemm_ex(d_C, N, (size_t)M * N, d_Ahi, d_Alo, d_W, M, N, K, splits);
}

/* ---- fp32 -> (hi, lo) bf16 planes ---------------------------------------------- */

__global__ void vt_split_kernel(uint16_t *hi, uint16_t *lo, const float *x, size_t n2) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n2;
         i += (size_t)gridDim.x * blockDim.x) {
        const f32x2 v = reinterpret_cast<const f32x2 *>(x)[i];
        unsigned h, l;
        vt_split_planes2(v.x, v.y, h, l);
        reinterpret_cast<unsigned *>(hi)[i] = h;
        reinterpret_cast<unsigned *>(lo)[i] = l;
    }
}

static int gm_blocks(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 8192 ? 8192 : b); }

void vt_launch_split(uint16_t *d_hi, uint16_t *d_lo, const float *d_x, size_t n) {
    hipLaunchKernelGGL(vt_split_kernel, dim3(gm_blocks(n / 2)), dim3(256), 0, g_vt.stream, d_hi, d_lo, d_x, n / 2);
}

/* One workgroup per row of 3072 floats (256 threads x 12):
 *   x[row] += part[0][row] + part[1][row] + ...   (splits > 0; fixed order)
 *   (hi, lo)[row] = split(rmsnorm(x[row]) * w)     (w != NULL)
 * The residual add and the normalisation of voxtral_tts_llm.c:332-336,354 /
 * :338-341 in one pass over the row. */
__global__ void __launch_bounds__(256)
vt_residual_norm_split_kernel(float *x, const float *part, int splits, size_t part_stride,
                              const float *w, uint16_t *hi, uint16_t *lo, float eps) {
    /* a thread owns 4 consecutive columns at 4 (t + 256 j): 16-byte loads and stores, 8-byte plane
     * stores (a quarter of the memory instructions of element-wise accesses) */
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    constexpr int NJ = VT_DIM / 1024;
    f32x4 v[NJ];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const size_t i = row * VT_DIM + 4 * ((size_t)threadIdx.x + 256 * j);
        f32x4 a = *reinterpret_cast<const f32x4 *>(x + i);
        if (splits > 0) {
            f32x4 p = *reinterpret_cast<const f32x4 *>(part + i);
            for (int s = 1; s < splits; s++) {
                const f32x4 q = *reinterpret_cast<const f32x4 *>(part + (size_t)s * part_stride + i);
                p.x = __fadd_rn(p.x, q.x); p.y = __fadd_rn(p.y, q.y);
                p.z = __fadd_rn(p.z, q.z); p.w = __fadd_rn(p.w, q.w);
            }
            a.x = __fadd_rn(a.x, p.x); a.y = __fadd_rn(a.y, p.y);
            a.z = __fadd_rn(a.z, p.z); a.w = __fadd_rn(a.w, p.w);
            *reinterpret_cast<f32x4 *>(x + i) = a;
        }
        v[j] = a;
        ss = fmaf(a.x, a.x, ss); ss = fmaf(a.y, a.y, ss);
        ss = fmaf(a.z, a.z, ss); ss = fmaf(a.w, a.w, ss);
    }
    if (!w) return;
    ss = vt_wave_sum(ss);
    if (vt_lane() == 0) red[vt_wave()] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.0f / sqrtf(tot / (float)VT_DIM + eps);
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = 4 * ((int)threadIdx.x + 256 * j);
        const f32x4 g = *reinterpret_cast<const f32x4 *>(w + c);
        u32x2 sph, spl;
        vt_split_planes4(__fmul_rn(__fmul_rn(v[j].x, inv), g.x), __fmul_rn(__fmul_rn(v[j].y, inv), g.y), __fmul_rn(__fmul_rn(v[j].z, inv), g.z), __fmul_rn(__fmul_rn(v[j].w, inv), g.w), sph, spl);
        *reinterpret_cast<u32x2 *>(hi + row * VT_DIM + c) = sph;
        *reinterpret_cast<u32x2 *>(lo + row * VT_DIM + c) = spl;
    }
}

void vt_launch_residual_norm_split(float *d_x, const float *d_part, int splits, size_t part_stride,
                                   const float *d_w, uint16_t *d_hi, uint16_t *d_lo, int rows) {
    hipLaunchKernelGGL(vt_residual_norm_split_kernel, dim3(rows), dim3(256), 0, g_vt.stream, d_x, d_part,
                       splits, part_stride, d_w, d_hi, d_lo, VT_EPS);
}

/* gu [rows, 2*ffn] with (gate, up) adjacent -> (hi, lo) planes of silu(gate)*up
 * (voxtral_tts_llm.c:346-350 on the row-interleaved gate/up matrix).  Columns from
 * tail_col0 on are taken as the sum of `tail_planes` split-K planes [rows, 2*ffn - tail_col0]
 * instead (tail_planes == 0: everything is in gu). */
__global__ void vt_swiglu_split_kernel(uint16_t *hi, uint16_t *lo, const float *gu, size_t n8,
                                       int tail_col0, const float *tail, int tail_planes, size_t tail_stride) {
    /* a thread owns 8 consecutive floats, i.e. 4 (gate, up) pairs: 16-byte loads, 8-byte plane
     * stores; rows and the tail boundary are multiples of 8 columns */
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
         i += (size_t)gridDim.x * blockDim.x) {
        f32x4 g0 = reinterpret_cast<const f32x4 *>(gu)[2 * i];
        f32x4 g1 = reinterpret_cast<const f32x4 *>(gu)[2 * i + 1];
        if (tail_planes > 0) {
            const size_t row = (8 * i) / (2 * VT_FFN);
            const int col = (int)((8 * i) % (2 * VT_FFN));
            if (col >= tail_col0) {
                const int tw = 2 * VT_FFN - tail_col0;
                const float *tp = tail + row * tw + (col - tail_col0);
                g0 = *reinterpret_cast<const f32x4 *>(tp);
                g1 = *reinterpret_cast<const f32x4 *>(tp + 4);
                for (int p = 1; p < tail_planes; p++) {
                    const f32x4 w0 = *reinterpret_cast<const f32x4 *>(tp + p * tail_stride);
                    const f32x4 w1 = *reinterpret_cast<const f32x4 *>(tp + p * tail_stride + 4);
                    g0.x = __fadd_rn(g0.x, w0.x); g0.y = __fadd_rn(g0.y, w0.y);
                    g0.z = __fadd_rn(g0.z, w0.z); g0.w = __fadd_rn(g0.w, w0.w);
                    g1.x = __fadd_rn(g1.x, w1.x); g1.y = __fadd_rn(g1.y, w1.y);
                    g1.z = __fadd_rn(g1.z, w1.z); g1.w = __fadd_rn(g1.w, w1.w);
                }
            }
        }
        const float a = __fmul_rn(__fdiv_rn(g0.x, __fadd_rn(1.0f, expf(-g0.x))), g0.y);
        const float b = __fmul_rn(__fdiv_rn(g0.z, __fadd_rn(1.0f, expf(-g0.z))), g0.w);
        const float c = __fmul_rn(__fdiv_rn(g1.x, __fadd_rn(1.0f, expf(-g1.x))), g1.y);
        const float d = __fmul_rn(__fdiv_rn(g1.z, __fadd_rn(1.0f, expf(-g1.z))), g1.w);
        u32x2 sph, spl;
        vt_split_planes4(a, b, c, d, sph, spl);
        reinterpret_cast<u32x2 *>(hi)[i] = sph;
        reinterpret_cast<u32x2 *>(lo)[i] = spl;
    }
}

void vt_launch_swiglu_split(uint16_t *d_hi, uint16_t *d_lo, const float *d_gu, size_t n_out, int tail_col0,
                            const float *d_tail, int tail_planes, size_t tail_stride) {
    hipLaunchKernelGGL(vt_swiglu_split_kernel, dim3(gm_blocks(n_out / 4)), dim3(256), 0, g_vt.stream, d_hi, d_lo,
                       d_gu, n_out / 4, tail_col0, d_tail, tail_planes, tail_stride);
}

/* The K-cut tail of the paired gate|up product: tail [planes][rows, tw] fp32 in the paired column order
 * (of every 64 columns the first 32 are gates, the other 32 the ups of the same h columns) -> the
 * (hi, lo) planes of SiLU(gate) * up at h columns h_col0 .. h_col0 + tw/2 (row pitch ldh).  A thread owns 4
 * consecutive h columns. */
__global__ void vt_swiglu_pair_tail_kernel(uint16_t *hi, uint16_t *lo, int ldh, int h_col0, const float *tail,
                                           int planes, size_t stride, int rows, int tw) {
    const int per_row = tw / 8;                                   /* threads per row */
    const size_t total = (size_t)rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int row = (int)(i / per_row), q = (int)(i % per_row);
        const int blk = q >> 3, c = (q & 7) * 4;
        const float *tp = tail + (size_t)row * tw + 64 * blk + c;
        f32x4 g = *reinterpret_cast<const f32x4 *>(tp), u = *reinterpret_cast<const f32x4 *>(tp + 32);
        for (int p = 1; p < planes; p++) {
            const f32x4 g2 = *reinterpret_cast<const f32x4 *>(tp + p * stride);
            const f32x4 u2 = *reinterpret_cast<const f32x4 *>(tp + p * stride + 32);
            g.x = __fadd_rn(g.x, g2.x); g.y = __fadd_rn(g.y, g2.y); g.z = __fadd_rn(g.z, g2.z); g.w = __fadd_rn(g.w, g2.w);
            u.x = __fadd_rn(u.x, u2.x); u.y = __fadd_rn(u.y, u2.y); u.z = __fadd_rn(u.z, u2.z); u.w = __fadd_rn(u.w, u2.w);
        }
        const float a = __fmul_rn(__fdiv_rn(g.x, __fadd_rn(1.0f, expf(-g.x))), u.x);
        const float b = __fmul_rn(__fdiv_rn(g.y, __fadd_rn(1.0f, expf(-g.y))), u.y);
        const float cc = __fmul_rn(__fdiv_rn(g.z, __fadd_rn(1.0f, expf(-g.z))), u.z);
        const float d = __fmul_rn(__fdiv_rn(g.w, __fadd_rn(1.0f, expf(-g.w))), u.w);
        u32x2 sph, spl;
        vt_split_planes4(a, b, cc, d, sph, spl);
        const size_t at = (size_t)row * ldh + h_col0 + 32 * blk + c;
        *reinterpret_cast<u32x2 *>(hi + at) = sph;
        *reinterpret_cast<u32x2 *>(lo + at) = spl;
    }
}

void vt_launch_swiglu_pair_tail(uint16_t *d_hi, uint16_t *d_lo, int ldh, int h_col0, const float *d_tail, int planes,
                                size_t stride, int rows, int tw) {
    hipLaunchKernelGGL(vt_swiglu_pair_tail_kernel, dim3(gm_blocks((size_t)rows * tw / 8)), dim3(256), 0, g_vt.stream,
                       d_hi, d_lo, ldh, h_col0, d_tail, planes, stride, rows, tw);
}

/* C = sum of `splits` partial planes (fixed order), for callers that want the plain product. */
__global__ void vt_sum_planes_kernel(float *out, const float *part, int splits, size_t stride, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x) {
        float p = part[i];
        for (int s = 1; s < splits; s++) p = __fadd_rn(p, part[(size_t)s * stride + i]);
        out[i] = p;
    }
}

void vt_launch_sum_planes(float *d_out, const float *d_part, int splits, size_t stride, size_t n) {
    hipLaunchKernelGGL(vt_sum_planes_kernel, dim3(gm_blocks(n)), dim3(256), 0, g_vt.stream, d_out, d_part,
                       splits, stride, n);
}
