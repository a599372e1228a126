/*
 * vt_prefill.hip - backbone prefill over a row block of the sequence (replaces
 * tts_cuda_llm_prefill, voxtral_tts_cuda.cu:806-893; the layer follows
 * voxtral_tts_llm.c:299-366).
 *
 * Per layer: RMSNorm into (hi, lo) bf16 planes -> q|k|v product on the matrix
 * cores -> RoPE + cache append -> causal attention on the fp32 matrix cores
 * -> output projection (K split in 2) -> residual + RMSNorm -> gate/up product
 * -> SiLU*up -> down projection (K split in 3) -> residual fused with the next
 * layer's RMSNorm.  Weights are the fused layouts of the decode path.
 */
#include "vt_state.h"
#include "vt_gemm.h"

#include <math.h>


/* ---- causal attention, 16 queries x 32 keys per matrix-core tile ----------------
 * (tts_causal_attention, voxtral_tts_kernels.c:403-465, for head_dim 128 and four
 * query heads per KV head.)
 *
 * Workgroup = (KV head, HPW of its 4 query heads, block of 16 queries), HPW*NSPLIT
 * waves: wave = (query head, key-tile residue).  The waves of one residue share 32-key
 * K and V tiles in LDS, as (hi, lo) planes laid out as the matrix instructions want them: K as
 * [key][dim] (a lane's operand is 8 consecutive dims of a key), V transposed as [dim][lane
 * group][8 key slots] (a lane's operand is the 8 keys of its group for one dim).  The planes are
 * made once per layer, by vt_kv_image_kernel, in exactly this layout; a workgroup copies a tile's
 * 37 KB image into its LDS (converting in here cost every step 1450 of its 5900 cycles, and every
 * tile is used by 34 workgroups on average).  Both products run on the bf16 matrix cores
 * (v_mfma_f32_16x16x32_bf16) with every fp32 operand split in (hi, lo) bf16 planes as in
 * the projections: a b = hi_a hi_b + hi_a lo_b + lo_a hi_b, 16 mantissa bits per operand,
 * fp32 accumulation; three such instructions take 3/16 of the time of the fp32 ones they
 * replace.  Scores are computed transposed, S^T = K Q^T, so that a lane owns one query:
 * lane l holds query l%16 and the keys 4*(l/16) + v of each 16-key block in accumulator
 * element v.  The softmax state is then per lane (two exchanges across the four lane
 * groups per tile), and the eight probabilities a lane holds are exactly its share of the
 * reduction index of the second product O^T = V^T P^T (the k order inside a matrix
 * instruction is free as long as both operands agree: slot j of lane group g stands for
 * key 16*(j/4) + 4*g + j%4).  Residues are merged through LDS at the end.
 * 16-query blocks give 32 blocks per KV head at 512 queries: with HPW = 2 that is 512
 * workgroups whose work grows with the block index (causal), enough to keep 256 CUs
 * busy when long and short blocks follow each other. */
#define PA_QT 16                  /* queries per workgroup */
#define PA_KROW 272               /* bytes per key of a K plane: 128 bf16 + 16 (16-byte reads over 16 keys cover all banks) */
#define PA_VROW 80                /* bytes per dim of a V plane: 4 lane groups x 8 key slots + 16 */
/* Dim d of V is row d of its plane: the 16 lanes that a 16-byte LDS read serves together (dims 16 b + li of
 * a block) then start 20 li dwords apart, which are 16 different groups of four banks.  (While the tiles were
 * converted in here the rows were skewed to keep the transposed writes free of bank conflicts.) */
#define PA_KPLANE (32 * PA_KROW)
#define PA_VPLANE (VT_HEAD_DIM * PA_VROW)
#define PA_TILE_BYTES (2 * PA_KPLANE + 2 * PA_VPLANE)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

/* eight consecutive k of a matrix-core operand from two fp32 quads: (hi, lo) planes */
__device__ __forceinline__ void pa_planes8(const f32x4 &a, const f32x4 &b, bf16x8 &hi, bf16x8 &lo) {
    unsigned h0, h1, h2, h3, l0, l1, l2, l3;
    vt_split_planes2(a.x, a.y, h0, l0);
    vt_split_planes2(a.z, a.w, h1, l1);
    vt_split_planes2(b.x, b.y, h2, l2);
    vt_split_planes2(b.z, b.w, h3, l3);
    hi = __builtin_bit_cast(bf16x8, u32x4{h0, h1, h2, h3});
    lo = __builtin_bit_cast(bf16x8, u32x4{l0, l1, l2, l3});
}

/* K and V of one layer as the attention wants them in its LDS: per (kv head, tile of 32 keys) the image
 * [K hi plane | K lo plane | V hi plane | V lo plane] described above, img[kvh][tile], so that the attention
 * copies a tile instead of converting it (every tile is read by all later query blocks of 4 heads: at 512
 * rows 34 times on average).  Workgroup = (tile, kv head), 128 threads for K and 128 for V; thread (sg, cg) owns the dims
 * 4*cg .. + 4 of the 8 keys that lane group sg meets in the second product (slot j: key 16*(j/4) + 4*sg +
 * j%4), so that the transposed V write is one 16-byte store per dim and plane.
 * Rows [start_pos, start_pos + S) come from the q|k|v product when qkv != NULL: the sum of `planes`
 * split-K planes (`plane_stride` floats apart, fixed order), k rotated (adjacent pairs,
 * voxtral_tts_kernels.c:616-634; the table holds (cos, sin) per pair), and are appended to the cache on the
 * way (voxtral_tts_llm.c:317-324).  Earlier rows come from the cache; rows from kv_rows on are zeros (their
 * keys are masked).  qkv == NULL: all rows are in the cache (rope is not read). */
__global__ void __launch_bounds__(256)
vt_kv_image_kernel(unsigned char *img, int img_tiles, const float *qkv, int planes, size_t plane_stride,
                   float *kc, float *vc, const float *rope, int start_pos, int kv_rows) {
    /* threads 0..127 make the K planes of the tile, threads 128..255 the V planes */
    const int tile = (int)blockIdx.x, kvh = (int)blockIdx.y;
    const bool is_v = threadIdx.x >= 128;
    const int tl = (int)threadIdx.x & 127, sg = tl >> 5, cg = tl & 31;
    const int col = kvh * VT_HEAD_DIM + 4 * cg;
    float *cache = is_v ? vc : kc;
    f32x4 r8[8];
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    if (qkv && tile * 32 >= start_pos && tile * 32 + 32 <= kv_rows) {
        /* a tile of new rows only (all but the first and the last one of a chunk): every request up front */
        const float *src = qkv + (size_t)(tile * 32 - start_pos) * VT_QKV_DIM + VT_Q_DIM + (is_v ? VT_KV_DIM : 0) + col;
        f32x4 cs[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int row = 16 * (i >> 2) + 4 * sg + (i & 3);
            r8[i] = *reinterpret_cast<const f32x4 *>(src + (size_t)row * VT_QKV_DIM);
            cs[i] = is_v ? zero : *reinterpret_cast<const f32x4 *>(rope + (size_t)(tile * 32 + row) * VT_HEAD_DIM + 4 * cg);
        }
        for (int p = 1; p < planes; p++) {
            f32x4 w[8];
#pragma unroll
            for (int i = 0; i < 8; i++)
                w[i] = *reinterpret_cast<const f32x4 *>(src + p * plane_stride + (size_t)(16 * (i >> 2) + 4 * sg + (i & 3)) * VT_QKV_DIM);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                r8[i].x = __fadd_rn(r8[i].x, w[i].x); r8[i].y = __fadd_rn(r8[i].y, w[i].y);
                r8[i].z = __fadd_rn(r8[i].z, w[i].z); r8[i].w = __fadd_rn(r8[i].w, w[i].w);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int r = tile * 32 + 16 * (i >> 2) + 4 * sg + (i & 3);
            if (!is_v) {
                const f32x4 k = r8[i], c = cs[i];
                r8[i] = f32x4{__fsub_rn(__fmul_rn(k.x, c.x), __fmul_rn(k.y, c.y)), __fadd_rn(__fmul_rn(k.x, c.y), __fmul_rn(k.y, c.x)),
                              __fsub_rn(__fmul_rn(k.z, c.z), __fmul_rn(k.w, c.w)), __fadd_rn(__fmul_rn(k.z, c.w), __fmul_rn(k.w, c.z))};
            }
            *reinterpret_cast<f32x4 *>(cache + (size_t)r * VT_KV_DIM + col) = r8[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int r = tile * 32 + 16 * (i >> 2) + 4 * sg + (i & 3);
            if (r >= kv_rows) {
                r8[i] = zero;
            } else if (qkv && r >= start_pos) {
                const float *src = qkv + (size_t)(r - start_pos) * VT_QKV_DIM + VT_Q_DIM + (is_v ? VT_KV_DIM : 0) + col;
                f32x4 k = *reinterpret_cast<const f32x4 *>(src);
                for (int p = 1; p < planes; p++) {
                    const f32x4 k2 = *reinterpret_cast<const f32x4 *>(src + p * plane_stride);
                    k.x = __fadd_rn(k.x, k2.x); k.y = __fadd_rn(k.y, k2.y); k.z = __fadd_rn(k.z, k2.z); k.w = __fadd_rn(k.w, k2.w);
                }
                if (!is_v) {
                    const f32x4 c = *reinterpret_cast<const f32x4 *>(rope + (size_t)r * VT_HEAD_DIM + 4 * cg);
                    k = f32x4{__fsub_rn(__fmul_rn(k.x, c.x), __fmul_rn(k.y, c.y)), __fadd_rn(__fmul_rn(k.x, c.y), __fmul_rn(k.y, c.x)),
                              __fsub_rn(__fmul_rn(k.z, c.z), __fmul_rn(k.w, c.w)), __fadd_rn(__fmul_rn(k.z, c.w), __fmul_rn(k.w, c.z))};
                }
                *reinterpret_cast<f32x4 *>(cache + (size_t)r * VT_KV_DIM + col) = k;
                r8[i] = k;
            } else {
                r8[i] = *reinterpret_cast<const f32x4 *>(cache + (size_t)r * VT_KV_DIM + col);
            }
        }
    }
    unsigned char *Kt = img + ((size_t)kvh * img_tiles + tile) * PA_TILE_BYTES, *Vt = Kt + 2 * PA_KPLANE;
    if (!is_v) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int row = 16 * (i >> 2) + 4 * sg + (i & 3);
            u32x2 h, l;
            vt_split_planes4(r8[i].x, r8[i].y, r8[i].z, r8[i].w, h, l);
            *reinterpret_cast<u32x2 *>(Kt + row * PA_KROW + 8 * cg) = h;
            *reinterpret_cast<u32x2 *>(Kt + PA_KPLANE + row * PA_KROW + 8 * cg) = l;
        }
    } else {
#pragma unroll
        for (int d = 0; d < 4; d++) {
            bf16x8 h, l;
            pa_planes8(f32x4{r8[0][d], r8[1][d], r8[2][d], r8[3][d]}, f32x4{r8[4][d], r8[5][d], r8[6][d], r8[7][d]}, h, l);
            *reinterpret_cast<bf16x8 *>(Vt + (4 * cg + d) * PA_VROW + 16 * sg) = h;
            *reinterpret_cast<bf16x8 *>(Vt + PA_VPLANE + (4 * cg + d) * PA_VROW + 16 * sg) = l;
        }
    }
}

template <int NSPLIT, int HPW>
__global__ void __launch_bounds__(64 * HPW * NSPLIT)
vt_prefill_attention_kernel(float *out, uint16_t *out_hi, uint16_t *out_lo, const float *Q,
                            int q_stride, int q_planes, size_t q_plane_stride, const float *rope,
                            const unsigned char *img, int img_tiles, int S, int start_pos, float scale) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pa_lds[];
    constexpr int GT = 64 * HPW;                         /* threads of a residue group */
    constexpr int NCH = PA_TILE_BYTES / 16;              /* 16-byte chunks of a tile image */
    constexpr int NLD = (NCH + GT - 1) / GT;             /* chunks per thread and tile */
    const int kvh = (int)blockIdx.x / (4 / HPW), hsub = (int)blockIdx.x % (4 / HPW);
    /* The last query block has the most keys.  Workgroups are handed to the CUs in launch order, one per
     * CU and then a second one each: the first half of the launch takes the long blocks in descending
     * order, the second half the short ones in ascending order, so that every CU gets a long block and
     * the short one that makes up the same total. */
    const int ny = (int)gridDim.y, half = (ny + 1) / 2;
    const int qt = (int)blockIdx.y < half ? ny - 1 - (int)blockIdx.y : (int)blockIdx.y - half;
    const int t = (int)threadIdx.x, lane = t & 63, wave = t >> 6;
    const int hq = wave % HPW, pz = wave / HPW;
    const int tl = hq * 64 + lane;                       /* thread index inside the residue group */
    const int g = lane >> 4, li = lane & 15;
    const int q0 = qt * PA_QT;
    const int my_q = q0 + li;
    const int head = kvh * 4 + hsub * HPW + hq;
    unsigned char *Kt = pa_lds + (size_t)pz * PA_TILE_BYTES, *Vt = Kt + 2 * PA_KPLANE;   /* hi plane, then lo */

    /* this lane's query as the B operand of K Q^T: dims 8*g + 32*ks .. + 8 for K step ks, both planes */
    bf16x8 qhi[4], qlo[4];
    {
        /* Q as it is, or (rope != NULL) the raw product: the sum of q_planes split-K planes, rotated here
         * (adjacent pairs, voxtral_tts_kernels.c:616-634; the table holds (cos, sin) per pair).  All
         * requests of a plane go out before the first value is used: inside a prefill every one of them
         * goes to memory, and one after the other they were 7 us of a 27 us launch. */
        const int qrow = my_q < S ? my_q : S - 1;
        const float *qp = Q + (size_t)qrow * q_stride + head * VT_HEAD_DIM + 8 * g;
        f32x4 qa[4], qb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            qa[ks] = reinterpret_cast<const f32x4 *>(qp + 32 * ks)[0];
            qb[ks] = reinterpret_cast<const f32x4 *>(qp + 32 * ks)[1];
        }
        if (rope) {
            const float *cs = rope + (size_t)(start_pos + qrow) * VT_HEAD_DIM + 8 * g;
            f32x4 c0[4], c1[4];
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                c0[ks] = reinterpret_cast<const f32x4 *>(cs + 32 * ks)[0];
                c1[ks] = reinterpret_cast<const f32x4 *>(cs + 32 * ks)[1];
            }
            for (int p = 1; p < q_planes; p++) {
                f32x4 a2[4], b2[4];
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    a2[ks] = reinterpret_cast<const f32x4 *>(qp + p * q_plane_stride + 32 * ks)[0];
                    b2[ks] = reinterpret_cast<const f32x4 *>(qp + p * q_plane_stride + 32 * ks)[1];
                }
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    f32x4 &a = qa[ks], &b = qb[ks];
                    a.x = __fadd_rn(a.x, a2[ks].x); a.y = __fadd_rn(a.y, a2[ks].y); a.z = __fadd_rn(a.z, a2[ks].z); a.w = __fadd_rn(a.w, a2[ks].w);
                    b.x = __fadd_rn(b.x, b2[ks].x); b.y = __fadd_rn(b.y, b2[ks].y); b.z = __fadd_rn(b.z, b2[ks].z); b.w = __fadd_rn(b.w, b2[ks].w);
                }
            }
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const f32x4 a = qa[ks], b = qb[ks];
                qa[ks] = f32x4{__fsub_rn(__fmul_rn(a.x, c0[ks].x), __fmul_rn(a.y, c0[ks].y)), __fadd_rn(__fmul_rn(a.x, c0[ks].y), __fmul_rn(a.y, c0[ks].x)),
                               __fsub_rn(__fmul_rn(a.z, c0[ks].z), __fmul_rn(a.w, c0[ks].w)), __fadd_rn(__fmul_rn(a.z, c0[ks].w), __fmul_rn(a.w, c0[ks].z))};
                qb[ks] = f32x4{__fsub_rn(__fmul_rn(b.x, c1[ks].x), __fmul_rn(b.y, c1[ks].y)), __fadd_rn(__fmul_rn(b.x, c1[ks].y), __fmul_rn(b.y, c1[ks].x)),
                               __fsub_rn(__fmul_rn(b.z, c1[ks].z), __fmul_rn(b.w, c1[ks].w)), __fadd_rn(__fmul_rn(b.z, c1[ks].w), __fmul_rn(b.w, c1[ks].z))};
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) pa_planes8(qa[ks], qb[ks], qhi[ks], qlo[ks]);
    }
    f32x4 o[8];
#pragma unroll
    for (int b = 0; b < 8; b++) o[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -1e30f, lsum = 0.f;

    const int last_q = (q0 + PA_QT - 1 < S ? q0 + PA_QT - 1 : S - 1) + start_pos;
    const int ntiles = last_q / 32 + 1;                  /* key tiles 0 .. ntiles-1 are visible */
    const int nsteps = (ntiles + NSPLIT - 1) / NSPLIT;

    /* staging: a tile arrives as the image vt_kv_image_kernel made of it, which is what the LDS holds:
     * the threads of a residue group copy its 16-byte chunks tl, tl + GT, ...  Buffer loads: the tile as the
     * scalar offset, the thread's chunk as a vector offset that never changes (no 64-bit address arithmetic
     * per load); the chunks past the end of a tile belong to nobody and are never stored. */
    u32x4 rt[NLD];
    const __amdgpu_buffer_rsrc_t t_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(img + (size_t)kvh * img_tiles * PA_TILE_BYTES), 0, img_tiles * PA_TILE_BYTES, 0x00020000);
    int voff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) voff[i] = 16 * (tl + GT * i < NCH ? tl + GT * i : NCH - 1);
    /* A tile is requested in four parts, dealt out over the step: a wave's requests are accepted at the
     * pace at which the CU's address unit works them off (16 cycles per 1 KB request, all waves of the CU
     * together), and all of them in a row hold the wave's own matrix instructions up behind them. */
    auto fetch_part = [&](int tile, int part) {
        const int soff = __builtin_amdgcn_readfirstlane(tile) * PA_TILE_BYTES;
#pragma unroll
        for (int i = (part * NLD) / 4; i < ((part + 1) * NLD) / 4; i++)
            rt[i] = __builtin_amdgcn_raw_buffer_load_b128(t_rs, voff[i], soff, 0);
    };
    auto fetch = [&](int tile) {
#pragma unroll
        for (int part = 0; part < 4; part++) fetch_part(tile, part);
    };
    /* Every request of the loop below is unconditional (a tile index beyond the last visible one
     * is clamped: that tile is fetched again, out of the L2, and never stored): behind a
     * conditional request the compiler waits for all outstanding loads before the next use of
     * anything loaded, here the query registers, i.e. before the products of every step. */
    fetch(pz < ntiles ? pz : ntiles - 1);

    /* The workgroups of one blockIdx.x run on one XCD and walk the same K and V rows, tile by tile, at the
     * same pace: left alone, every tile is a miss in that XCD's L2 for all of them at the moment they need
     * it, and each step pays the full memory latency.  So they first touch all the rows between them, one
     * 128-byte line per lane and request (K and V rows are 4 lines each), which starts every line on its way
     * into the L2 at once.  The values are dropped at the end of the kernel. */
    unsigned warm[4];
    {   /* (behind the query and the first tile: a wave's loads return in order, and these go all the way to memory) */
        const int n_lines = ((start_pos + S + 31) / 32) * (PA_TILE_BYTES / 128), stride = (int)(gridDim.y * blockDim.x);
        const unsigned char *mine = img + (size_t)kvh * img_tiles * PA_TILE_BYTES;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int j = (int)blockIdx.y * (int)blockDim.x + t + k * stride;
            j = j < n_lines ? j : n_lines - 1;
            warm[k] = *reinterpret_cast<const unsigned *>(mine + (size_t)j * 128);
        }
    }

    for (int step = 0; step < nsteps; step++) {
        const int tile = step * NSPLIT + pz;
        const bool valid = tile < ntiles;
        __syncthreads();
        if (valid) {
#pragma unroll
            for (int i = 0; i < NLD; i++)
                if (GT * (i + 1) <= NCH || tl + GT * i < NCH) *reinterpret_cast<u32x4 *>(Kt + 16 * (tl + GT * i)) = rt[i];
        }
        __syncthreads();
        const int nxt = tile + NSPLIT < ntiles ? tile + NSPLIT : ntiles - 1;
        fetch_part(nxt, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (!valid) {
            fetch_part(nxt, 1); fetch_part(nxt, 2); fetch_part(nxt, 3);
            continue;
        }

        /* S^T = K Q^T: K step ks pairs the dims 8*g + 32*ks .. + 8 of key 16*kb + li and of the query */
        f32x4 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            s[kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const unsigned char *kp = Kt + (16 * kb + li) * PA_KROW + 16 * g + 64 * ks;
                const bf16x8 khi = *reinterpret_cast<const bf16x8 *>(kp);
                const bf16x8 klo = *reinterpret_cast<const bf16x8 *>(kp + PA_KPLANE);
                s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(klo, qhi[ks], s[kb], 0, 0, 0);
                s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(khi, qlo[ks], s[kb], 0, 0, 0);
                s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(khi, qhi[ks], s[kb], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        fetch_part(nxt, 1);
        __builtin_amdgcn_sched_barrier(0);
        /* online softmax for this lane's query; element v of block kb is key 16*kb + 4*g + v */
        const int qpos = start_pos + my_q;
        float mx = -1e30f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int kpos = tile * 32 + 16 * kb + 4 * g + v;
                s[kb][v] = kpos <= qpos ? __fmul_rn(s[kb][v], scale) : -3e38f;
                mx = fmaxf(mx, s[kb][v]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float mn = fmaxf(m, mx);
        const float corr = __expf(m - mn);
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                s[kb][v] = s[kb][v] > -1e38f ? __expf(s[kb][v] - mn) : 0.f;
                psum += s[kb][v];
            }
        lsum = fmaf(lsum, corr, psum);
        m = mn;
#pragma unroll
        for (int b = 0; b < 8; b++) o[b] = o[b] * corr;
        /* O^T += V^T P^T: slot j of this lane group is key 16*(j/4) + 4*g + j%4, whose probability is
         * s[j/4][j%4]; the A operand of dim block b is that key's column 16*b + li of V */
        bf16x8 phi, plo;
        pa_planes8(s[0], s[1], phi, plo);
        __builtin_amdgcn_sched_barrier(0);
        fetch_part(nxt, 2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const unsigned char *vp = Vt + (16 * b + li) * PA_VROW + 16 * g;
            const bf16x8 vhi = *reinterpret_cast<const bf16x8 *>(vp);
            const bf16x8 vlo = *reinterpret_cast<const bf16x8 *>(vp + PA_VPLANE);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vlo, phi, o[b], 0, 0, 0);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vhi, plo, o[b], 0, 0, 0);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vhi, phi, o[b], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        fetch_part(nxt, 3);
    }

    /* merge the residues: residue r > 0 parks (m, l, O) in LDS, residue 0 folds them in */
    if (NSPLIT > 1) {
        __syncthreads();
        float *park = reinterpret_cast<float *>(pa_lds);  /* [NSPLIT-1][HPW][34][64 lanes] */
        for (int r = 1; r < NSPLIT; r++) {
            float *slot = park + ((size_t)((r - 1) * HPW + hq) * 34) * 64 + lane;
            if (pz == r) {
                slot[0] = m;
                slot[64] = lsum;
#pragma unroll
                for (int b = 0; b < 8; b++)
#pragma unroll
                    for (int v = 0; v < 4; v++) slot[(2 + b * 4 + v) * 64] = o[b][v];
            }
            __syncthreads();
            if (pz == 0) {
                const float m2 = slot[0], l2 = slot[64];
                const float mn = fmaxf(m, m2);
                const float c1 = __expf(m - mn), c2 = __expf(m2 - mn);
                lsum = fmaf(lsum, c1, l2 * c2);
                m = mn;
#pragma unroll
                for (int b = 0; b < 8; b++)
#pragma unroll
                    for (int v = 0; v < 4; v++) o[b][v] = fmaf(o[b][v], c1, slot[(2 + b * 4 + v) * 64] * c2);
            }
            __syncthreads();
        }
    }
    asm volatile("" ::"v"(warm[0]), "v"(warm[1]), "v"(warm[2]), "v"(warm[3]));
    if (pz != 0 || my_q >= S) return;
    float L = lsum + __shfl_xor(lsum, 16);
    L += __shfl_xor(L, 32);
    const float inv = L > 0.f ? __fdiv_rn(1.0f, L) : 0.f;
    const size_t ob = (size_t)my_q * VT_Q_DIM + head * VT_HEAD_DIM;
#pragma unroll
    for (int b = 0; b < 8; b++) {
        const int d = 16 * b + 4 * g;
        f32x4 r;
        r.x = __fmul_rn(o[b][0], inv);
        r.y = __fmul_rn(o[b][1], inv);
        r.z = __fmul_rn(o[b][2], inv);
        r.w = __fmul_rn(o[b][3], inv);
        if (out) *reinterpret_cast<f32x4 *>(out + ob + d) = r;
        if (out_hi) {
            u32x2 sph, spl;
            vt_split_planes4(r.x, r.y, r.z, r.w, sph, spl);
            u32x2 ph = sph, pl = spl;
            *reinterpret_cast<u32x2 *>(out_hi + ob + d) = ph;
            *reinterpret_cast<u32x2 *>(out_lo + ob + d) = pl;
        }
    }
}

#ifndef PA_NSPLIT
#define PA_NSPLIT 2
#endif
#ifndef PA_HPW
#define PA_HPW 2
#endif

static size_t pa_lds_bytes(void) {
    size_t tiles = (size_t)PA_NSPLIT * PA_TILE_BYTES;
    size_t park = sizeof(float) * (size_t)(PA_NSPLIT - 1) * PA_HPW * 34 * 64;
    return tiles > park ? tiles : park;
}

/* Tiles of 32 keys that cover `rows` cache rows, and the tile images of one layer's K and V (a buffer of the
 * library's own that grows with the longest cache seen) */
static int pa_tiles(int rows) { return (rows + 31) / 32; }
unsigned char *vt_pa_image(int rows) {
    const size_t bytes = (size_t)VT_KV_HEADS * pa_tiles(rows) * PA_TILE_BYTES;
    if (bytes > g_vt.kv_img_bytes) {
        if (g_vt.d_kv_img) {
            (void)hipStreamSynchronize(g_vt.stream);
            (void)hipFree(g_vt.d_kv_img);
        }
        g_vt.d_kv_img = vt_dev_alloc(bytes);
        g_vt.kv_img_bytes = g_vt.d_kv_img ? bytes : 0;
    }
    return (unsigned char *)g_vt.d_kv_img;
}

/* d_qkv != NULL: rows start_pos .. start_pos + S - 1 are taken from the q|k|v product (summed, k rotated)
 * and appended to the cache d_K / d_V; otherwise all start_pos + S rows are in the cache already */
void vt_pa_launch_image(unsigned char *d_img, const float *d_qkv, int planes, size_t plane_stride, float *d_K,
                            float *d_V, int S, int start_pos) {
    const int rows = start_pos + S;
    hipLaunchKernelGGL(vt_kv_image_kernel, dim3(pa_tiles(rows), VT_KV_HEADS), dim3(256), 0, g_vt.stream, d_img,
                       pa_tiles(rows), d_qkv, planes, plane_stride, d_K, d_V, g_vt.d_rope, start_pos, rows);
}

/* Q rows are q_stride floats apart; out / (out_hi, out_lo) are [S,4096], each optional.  d_rope != NULL: d_Q
 * holds q_planes split-K planes (q_plane_stride floats apart) of the raw q product, to be summed and
 * rotated with the table rows start_pos .. by the kernel.  d_img: the tile images of the start_pos + S
 * cache rows (vt_kv_image_kernel). */
void vt_launch_prefill_attention_raw(float *d_out, uint16_t *d_hi, uint16_t *d_lo, const float *d_Q,
                                     int q_stride, int q_planes, size_t q_plane_stride, const float *d_rope,
                                     const unsigned char *d_img, int S, int start_pos, float scale) {
    static int attr_set = 0;
    if (!attr_set) {
        if (vt_check(hipFuncSetAttribute((const void *)vt_prefill_attention_kernel<PA_NSPLIT, PA_HPW>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)pa_lds_bytes()),
                     "attention LDS size"))
            return;
        attr_set = 1;
    }
    hipLaunchKernelGGL((vt_prefill_attention_kernel<PA_NSPLIT, PA_HPW>),
                       dim3(VT_KV_HEADS * (4 / PA_HPW), (S + PA_QT - 1) / PA_QT), dim3(64 * PA_HPW * PA_NSPLIT),
                       pa_lds_bytes(), g_vt.stream, d_out, d_hi, d_lo, d_Q, q_stride, q_planes, q_plane_stride, d_rope,
                       d_img, pa_tiles(start_pos + S), S, start_pos, scale);
}

void vt_launch_prefill_attention(float *d_out, uint16_t *d_hi, uint16_t *d_lo, const float *d_Q,
                                 int q_stride, const float *d_K, const float *d_V, int S, int start_pos,
                                 float scale) {
    unsigned char *img = vt_pa_image(start_pos + S);
    if (!img) return;
    /* (the image kernel only reads a cache that is complete) */
    vt_pa_launch_image(img, NULL, 0, 0, const_cast<float *>(d_K), const_cast<float *>(d_V), S, start_pos);
    vt_launch_prefill_attention_raw(d_out, d_hi, d_lo, d_Q, q_stride, 1, 0, NULL, img, S, start_pos, scale);
}

/* ---- backbone prefill ------------------------------------------------------------ */

/* K cuts of a product of `tiles` output tiles: one item per CU at most, `most` planes at most */
int vt_prefill_cuts(int tiles, int most) {
    const int c = g_vt.n_cu / tiles;
    return c < 1 ? 1 : c > most ? most : c;
}

/* The prefill with one persistent launch per layer for everything behind the attention
 * (vt_prefill_layer_kernel): per layer the k|v kernel, the attention and that launch, which also multiplies
 * the next layer's q|k|v.  Same arithmetic as the launch-per-product schedule below, bit for bit.
 * Measured slower than that schedule at every length (512 rows: 8.29 against 7.65 ms on the same box; 64 rows
 * 4.53 / 4.34; 2048 rows 29.96 / 29.77): a dependency wait costs about 5 us (results written through and
 * acknowledged, counter, poll, first operand loads from memory) against about 1.5 us for a launch boundary,
 * and with one item per workgroup and stage there is nothing to overlap it with (the same kernel with the
 * waits taken out, results wrong, takes 7.34 ms).  It is therefore the optional schedule, not the default. */
static void prefill_persistent(const float *embeds, int seq_len, int start_pos, float *out_x) {
    const size_t S = (size_t)seq_len;
    hipStream_t st = g_vt.stream;
    const int m_tiles = (seq_len + 127) / 128, n_layers = g_vt.n_dec_layers;
    const int fq = vt_prefill_cuts(m_tiles * (VT_QKV_DIM / 256), 4), fo = vt_prefill_cuts(m_tiles * (VT_DIM / 256), 8);
    /* work area: x | q|k|v planes | two sets of K-cut planes | gate|up tail planes | counters | bf16 planes */
    const size_t n_x = S * VT_DIM, n_wide = S * 4 * VT_QKV_DIM, n_part = 8 * S * VT_DIM, n_tail = (size_t)VT_W13_TAIL_CUT * S * 2048;
    const size_t cnt_bytes = vt_prefill_layer_counter_bytes() * n_layers;
    const size_t n_p3 = S * VT_DIM, n_p4 = S * VT_Q_DIM, n_p9 = S * VT_FFN;     /* bf16 elements per plane */
    const size_t bytes = sizeof(float) * (n_x + n_wide + 2 * n_part + n_tail) + cnt_bytes +
                         2 * sizeof(uint16_t) * (2 * n_p3 + n_p4 + n_p9);
    float *x = (float *)vt_scratch(bytes);
    unsigned char *img = vt_pa_image(start_pos + seq_len);
    if (!x || !img) return;
    float *wide = x + n_x, *part_a = wide + n_wide, *part_b = part_a + n_part, *tail = part_b + n_part;
    unsigned *cnt = (unsigned *)(tail + n_tail);
    uint16_t *n1_hi = (uint16_t *)((unsigned char *)cnt + cnt_bytes), *n1_lo = n1_hi + n_p3;
    uint16_t *n2_hi = n1_lo + n_p3, *n2_lo = n2_hi + n_p3;
    uint16_t *at_hi = n2_lo + n_p3, *at_lo = at_hi + n_p4;
    uint16_t *h_hi = at_lo + n_p4, *h_lo = h_hi + n_p9;
    int *abort_flag = g_vt.d_abort + 8;

    VT_TRYV(hipMemcpyAsync(x, embeds, sizeof(float) * n_x, hipMemcpyDefault, st));
    VT_TRYV(hipMemsetAsync(cnt, 0, cnt_bytes, st));
    vt_launch_residual_norm_split(x, NULL, 0, 0, g_vt.h_layers[0].attn_norm, n2_hi, n2_lo, seq_len);
    vt_launch_gemm_frag(wide, VT_QKV_DIM, S * VT_QKV_DIM, n2_hi, n2_lo, g_vt.h_frag[0].wqkv, seq_len, VT_QKV_DIM, VT_DIM, fq);
    for (int l = 0; l < n_layers; l++) {
        const vt_layer_dev *L = &g_vt.h_layers[l];
        const vt_layer_frag *F = &g_vt.h_frag[l];
        float *kc = g_hip.kv_cache_k_gpu + (size_t)l * g_vt.kv_max * VT_KV_DIM;
        float *vc = g_hip.kv_cache_v_gpu + (size_t)l * g_vt.kv_max * VT_KV_DIM;
        vt_pa_launch_image(img, wide, fq, S * VT_QKV_DIM, kc, vc, seq_len, start_pos);
        vt_launch_prefill_attention_raw(NULL, at_hi, at_lo, wide, VT_QKV_DIM, fq, S * VT_QKV_DIM, g_vt.d_rope, img,
                                        seq_len, start_pos, VT_ATT_SCALE);
        const bool more = l + 1 < n_layers;
        vt_prefill_layer_args a = {};
        a.M = seq_len;
        a.wo_f = F->wo; a.w13_f = F->w13; a.w2_f = F->w2;
        a.qkv_next_f = more ? g_vt.h_frag[l + 1].wqkv : NULL;
        a.ffn_norm = L->ffn_norm;
        a.next_norm = more ? g_vt.h_layers[l + 1].attn_norm : NULL;
        a.attn_hi = at_hi; a.attn_lo = at_lo;
        a.x = x; a.part_a = part_a; a.part_b = part_b;
        a.n1_hi = n1_hi; a.n1_lo = n1_lo; a.n2_hi = n2_hi; a.n2_lo = n2_lo;
        a.h_hi = h_hi; a.h_lo = h_lo; a.tail = tail; a.qkv = wide;
        a.fo = fo; a.fq = fq;
        a.cnt = cnt + (size_t)l * (vt_prefill_layer_counter_bytes() / sizeof(unsigned));
        a.abort_flag = abort_flag;
        a.timeout = g_vt.bar_timeout ? g_vt.bar_timeout : 200000000ull;      /* default 2 s of the 100 MHz wall clock */
        if (vt_launch_prefill_layer(a)) return;
    }
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    int gave_up = 0;
    VT_TRYV(hipMemcpy(&gave_up, abort_flag, sizeof gave_up, hipMemcpyDeviceToHost));
    if (gave_up) {
        (void)hipMemset(abort_flag, 0, sizeof(int));
        vt_set_error("tts_hip_llm_prefill: a dependency wait of the layer kernel timed out; the kernel left early, result invalid");
        return;
    }
    if (out_x) VT_TRYV(hipMemcpy(out_x, x, sizeof(float) * n_x, hipMemcpyDefault));
}

extern "C" void tts_hip_llm_prefill_out(const float *embeds, int seq_len, int start_pos, float *out_x) {
    if (!g_vt.initialized || g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_llm_prefill: no weights uploaded"); return; }
    if (seq_len < 1 || start_pos < 0 || start_pos + seq_len > g_vt.kv_max) {
        vt_set_error("tts_hip_llm_prefill: rows [%d, %d) outside the KV cache (max %d)", start_pos,
                     start_pos + seq_len, g_vt.kv_max);
        return;
    }
    const size_t S = (size_t)seq_len;
    hipStream_t st = g_vt.stream;
    {
        bool all_frag = true;
        for (int l = 0; l < g_vt.n_dec_layers; l++) {
            const vt_layer_frag *F = &g_vt.h_frag[l];
            all_frag = all_frag && F->wqkv && F->wo && F->w13 && F->w2;
        }
        if (g_vt.prefill_mode == 1 && all_frag && vt_prefill_layer_usable(seq_len)) {
            prefill_persistent(embeds, seq_len, start_pos, out_x);
            return;
        }
    }
    /* work area: x | wide f32 (qkv or gate/up) | q | partial planes | hi | lo */
    /* K is cut into as many ranges as give every CU at most one item (M tiles x N tiles x cuts; the cuts
     * need not divide K): 4 M tiles at 512 rows are 96 / 48 / 48 tiles for q|k|v / output / down, i.e.
     * 192 / 240 / 240 items */
    const int m_tiles = (seq_len + 127) / 128;
    const int fq = vt_prefill_cuts(m_tiles * (VT_QKV_DIM / 256), 4), fo = vt_prefill_cuts(m_tiles * (VT_DIM / 256), 8);
    /* the 128 x 128 kernel on row-major weights (layers without a fragment copy) wants cuts that divide K */
    const int rq = m_tiles >= 3 ? 2 : 4, ro = m_tiles >= 3 ? 4 : 8;
    const int tail_cols = m_tiles == 4 ? 16 * 128 : 0;      /* part holds 4 x S x 2048 <= 8 x S x 3072 */
    const size_t n_x = S * VT_DIM, n_wide = S * 4 * VT_QKV_DIM, n_part = 8 * S * VT_DIM;
    const size_t n_plane = S * VT_FFN;                            /* bf16 elements per plane */
    const size_t bytes = sizeof(float) * (n_x + n_wide + n_part) + 2 * sizeof(uint16_t) * n_plane;
    float *x = (float *)vt_scratch(bytes);
    unsigned char *img = vt_pa_image(start_pos + seq_len);
    if (!x || !img) return;
    float *wide = x + n_x, *part = wide + n_wide;
    uint16_t *hi = (uint16_t *)(part + n_part), *lo = hi + n_plane;
    const size_t ps = S * VT_DIM;

    VT_TRYV(hipMemcpyAsync(x, embeds, sizeof(float) * n_x, hipMemcpyDefault, st));
    vt_launch_residual_norm_split(x, NULL, 0, 0, g_vt.h_layers[0].attn_norm, hi, lo, seq_len);
    for (int l = 0; l < g_vt.n_dec_layers; l++) {
        const vt_layer_dev *L = &g_vt.h_layers[l];
        float *kc = g_hip.kv_cache_k_gpu + (size_t)l * g_vt.kv_max * VT_KV_DIM;
        float *vc = g_hip.kv_cache_v_gpu + (size_t)l * g_vt.kv_max * VT_KV_DIM;
        const vt_layer_frag *F = &g_vt.h_frag[l];
        const bool frag = F->wqkv && F->wo && F->w13 && F->w2;
        const int sp_qkv = frag ? fq : rq, sp_wo = frag ? fo : ro, sp_w2 = sp_wo;
        if (frag) vt_launch_gemm_frag(wide, VT_QKV_DIM, S * VT_QKV_DIM, hi, lo, F->wqkv, seq_len, VT_QKV_DIM, VT_DIM, sp_qkv);
        else vt_launch_gemm(wide, hi, lo, L->wqkv, seq_len, VT_QKV_DIM, VT_DIM, sp_qkv);
        /* k (rotated) and v into the cache and, with the earlier rows, into the attention's tile images; the
         * attention takes q from the product's planes itself */
        vt_pa_launch_image(img, wide, sp_qkv, S * VT_QKV_DIM, kc, vc, seq_len, start_pos);
        vt_launch_prefill_attention_raw(NULL, hi, lo, wide, VT_QKV_DIM, sp_qkv, S * VT_QKV_DIM, g_vt.d_rope, img,
                                        seq_len, start_pos, VT_ATT_SCALE);
        if (frag) vt_launch_gemm_frag(part, VT_DIM, ps, hi, lo, F->wo, seq_len, VT_DIM, VT_Q_DIM, sp_wo);
        else vt_launch_gemm(part, hi, lo, L->wo, seq_len, VT_DIM, VT_Q_DIM, sp_wo);
        vt_launch_residual_norm_split(x, part, sp_wo, ps, L->ffn_norm, hi, lo, seq_len);
        /* with the fragment copies the SiLU(gate) * up planes come out of the product itself, into the wide
         * area (free between q|k|v and the next layer), which the down projection then reads */
        uint16_t *h_hi = (uint16_t *)wide, *h_lo = h_hi + n_plane;
        if (frag && m_tiles != 4) {
            vt_launch_gemm_frag_swiglu(h_hi, h_lo, VT_FFN, NULL, hi, lo, F->w13, seq_len, 2 * VT_FFN, 0, VT_DIM, 1);
        } else if (frag) {
            /* 4 M tiles x 72 N tiles of 256 columns are 288 items for 256 CUs: the last 8 N tiles get their K cut
             * in VT_W13_TAIL_CUT and every workgroup takes one of those cuts after its whole tile, in the same
             * launch, instead of 32 workgroups running a second round alone */
            const int tail = 8 * 256, main_cols = 2 * VT_FFN - tail;
            vt_launch_gemm_frag_swiglu(h_hi, h_lo, VT_FFN, part, hi, lo, F->w13, seq_len, main_cols, tail, VT_DIM, VT_W13_TAIL_CUT);
            vt_launch_swiglu_pair_tail(h_hi, h_lo, VT_FFN, main_cols / 2, part, VT_W13_TAIL_CUT, S * tail, seq_len, tail);
        } else if (tail_cols) {
            /* 4 M tiles x 144 N tiles are 576 workgroups for 512 slots: the last 16 N tiles get their
             * K cut in 4 instead of running as a nearly empty second round */
            const int main_cols = 2 * VT_FFN - tail_cols;
            vt_launch_gemm_ex(wide, 2 * VT_FFN, 0, hi, lo, L->w13, seq_len, main_cols, VT_DIM, 1);
            vt_launch_gemm_ex(part, tail_cols, S * tail_cols, hi, lo, L->w13 + (size_t)main_cols * VT_DIM, seq_len,
                              tail_cols, VT_DIM, 4);
            vt_launch_swiglu_split(hi, lo, wide, S * VT_FFN, main_cols, part, 4, S * tail_cols);
        } else {
            vt_launch_gemm(wide, hi, lo, L->w13, seq_len, 2 * VT_FFN, VT_DIM, 1);
            vt_launch_swiglu_split(hi, lo, wide, S * VT_FFN, 0, NULL, 0, 0);
        }
        if (frag) vt_launch_gemm_frag(part, VT_DIM, ps, h_hi, h_lo, F->w2, seq_len, VT_DIM, VT_FFN, sp_w2);
        else vt_launch_gemm(part, hi, lo, L->w2, seq_len, VT_DIM, VT_FFN, sp_w2);
        const float *next_norm = l + 1 < g_vt.n_dec_layers ? g_vt.h_layers[l + 1].attn_norm : NULL;
        vt_launch_residual_norm_split(x, part, sp_w2, ps, next_norm, hi, lo, seq_len);
    }
    VT_TRYV(hipGetLastError());
    VT_TRYV(hipStreamSynchronize(st));
    if (out_x) VT_TRYV(hipMemcpy(out_x, x, sizeof(float) * n_x, hipMemcpyDefault));
}

extern "C" void tts_hip_llm_prefill(const float *embeds, int seq_len, int start_pos) {
    tts_hip_llm_prefill_out(embeds, seq_len, start_pos, NULL);
}
