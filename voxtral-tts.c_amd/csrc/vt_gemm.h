/*
 * vt_gemm.h - launchers of the bf16 MFMA matrix product on (hi, lo) activation
 * planes and of the row kernels that produce those planes.
 */
#ifndef VT_GEMM_H
#define VT_GEMM_H

#include <stddef.h>
#include <stdint.h>

/* N a multiple of 128, K/splits a multiple of 64 */
int vt_gemm_shape_ok(int M, int N, int K, int splits);
/* d_C: `splits` planes of [M, N] fp32, plane s holds the sum over K range s */
void vt_launch_gemm(float *d_C, const uint16_t *d_Ahi, const uint16_t *d_Alo, const uint16_t *d_W,
                    int M, int N, int K, int splits);
/* the same with the row pitch of C and the distance between planes given */
void vt_launch_gemm_ex(float *d_C, int ldc, size_t plane_stride, const uint16_t *d_Ahi, const uint16_t *d_Alo,
                       const uint16_t *d_W, int M, int N, int K, int splits);
/* The same product on the 128 x 256 tile kernel, which reads the weights in fragment order
 * (vt_launch_frag_layout): N % 256 == 0, K % 128 == 0, at most K / 128 cuts (they need not divide K). */
int vt_gemm_frag_shape_ok(int N, int K, int splits);
void vt_launch_gemm_frag(float *d_C, int ldc, size_t plane_stride, const uint16_t *d_Ahi, const uint16_t *d_Alo,
                         const uint16_t *d_Wf, int M, int N, int K, int splits);
/* row-major bf16 W[N, K] -> the fragment-order copy (same size); N % 32 == 0, K % 64 == 0.  pair: W holds
 * (gate, up) rows interleaved and every 64 fragment columns become 32 gates followed by their 32 ups
 * (N % 64 == 0), the order vt_launch_gemm_frag_swiglu expects. */
void vt_launch_frag_layout(uint16_t *d_Wf, const uint16_t *d_W, int N, int K, int pair);
/* gate|up product on paired weights with SiLU(gate) * up as its epilogue: the first n_main columns leave the
 * planes d_hhi / d_hlo [M, ldh] (n_main / 2 columns); the other n_tail columns (may be 0) have K cut in
 * tail_splits and leave fp32 planes d_tail [tail_splits][M, n_tail] for vt_launch_swiglu_pair_tail */
void vt_launch_gemm_frag_swiglu(uint16_t *d_hhi, uint16_t *d_hlo, int ldh, float *d_tail, const uint16_t *d_Ahi,
                                const uint16_t *d_Alo, const uint16_t *d_Wf, int M, int n_main, int n_tail, int K,
                                int tail_splits);
void vt_launch_swiglu_pair_tail(uint16_t *d_hi, uint16_t *d_lo, int ldh, int h_col0, const float *d_tail, int planes,
                                size_t stride, int rows, int tw);
/* n even */
void vt_launch_split(uint16_t *d_hi, uint16_t *d_lo, const float *d_x, size_t n);
/* rows of 3072: x += sum of planes (splits > 0), then planes of rmsnorm(x)*w (d_w != NULL) */
void vt_launch_residual_norm_split(float *d_x, const float *d_part, int splits, size_t part_stride,
                                   const float *d_w, uint16_t *d_hi, uint16_t *d_lo, int rows);
/* n_out a multiple of 4, tail_col0 of 8: planes of silu(gate)*up from interleaved (gate, up) pairs */
void vt_launch_swiglu_split(uint16_t *d_hi, uint16_t *d_lo, const float *d_gu, size_t n_out, int tail_col0,
                            const float *d_tail, int tail_planes, size_t tail_stride);
void vt_launch_sum_planes(float *d_out, const float *d_part, int splits, size_t stride, size_t n);

/* The products of one prefill layer behind its attention, with the row passes between them and the next
 * layer's q|k|v product, as one persistent launch (vt_prefill_layer_kernel).  All weights in fragment order;
 * every buffer distinct (each is written once per launch); cnt: vt_prefill_layer_counter_bytes() of zeros. */
struct vt_prefill_layer_args {
    int M;                                              /* rows */
    const uint16_t *wo_f, *w13_f, *w2_f, *qkv_next_f;   /* qkv_next_f NULL: the last layer */
    const float *ffn_norm, *next_norm;                  /* next_norm NULL: no planes behind the last residual add */
    const uint16_t *attn_hi, *attn_lo;                  /* [M, 4096] attention output planes (in) */
    float *x;                                           /* [M, 3072] residual stream (in place) */
    float *part_a, *part_b;                             /* [fo][M, 3072] K-cut planes of the output / down projection */
    uint16_t *n1_hi, *n1_lo, *n2_hi, *n2_lo;            /* [M, 3072] planes behind the two RMSNorms */
    uint16_t *h_hi, *h_lo;                              /* [M, 9216] SiLU(gate) * up */
    float *tail;                                        /* [VT_W13_TAIL_CUT][M, 2048] */
    float *qkv;                                         /* [fq][M, 6144] K-cut planes of the next layer's q|k|v (out) */
    int fo, fq;                                         /* K cuts of output / down, and of q|k|v */
    unsigned *cnt;
    int *abort_flag;
    unsigned long long timeout;                         /* spin budget of one dependency wait, 100 MHz ticks */
};
int vt_prefill_layer_usable(int M);
size_t vt_prefill_layer_counter_bytes(void);
int vt_launch_prefill_layer(const vt_prefill_layer_args &a);

#endif /* VT_GEMM_H */
