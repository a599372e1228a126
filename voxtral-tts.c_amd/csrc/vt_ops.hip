/*
 * vt_ops.hip - kernel-level operators of the C ABI on device pointers
 * (replace the standalone kernels of voxtral_tts_cuda.cu:331-704): generic
 * bf16-weight linear, RMSNorm, RoPE, SiLU*mul, residual add, attention
 * (decode / causal prefill / bidirectional) and embedding lookup.
 * Shapes are arbitrary here; the fixed-shape fused paths live in
 * vt_decode.hip, vt_prefill.hip and vt_acoustic.hip.
 */
#include "vt_state.h"
#include "vt_gemm.h"

#include <math.h>
#include <stdlib.h>

/* ---- linear: y[s,o] = bias[o] + sum_k W[o,k] x[s,k] ------------------------- */
/* One wave per output row; up to S rows of x share each weight load. */
template <int S>
__global__ void __launch_bounds__(256)
vt_linear_kernel(float *y, const float *x, const uint16_t *W, const float *bias,
                 int seq_len, int in_dim, int out_dim, int vec_ok) {
    const int row = (int)blockIdx.x * (int)(blockDim.x >> 6) + vt_wave();
    if (row >= out_dim) return;
    const int lane = vt_lane();
    const uint16_t *wr = W + (size_t)row * in_dim;
    for (int s0 = 0; s0 < seq_len; s0 += S) {
        float acc[S];
#pragma unroll
        for (int s = 0; s < S; s++) acc[s] = 0.f;
        if (vec_ok) {
            for (int k = lane * 8; k < in_dim; k += 512) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(wr + k);
#pragma unroll
                for (int s = 0; s < S; s++) {
                    if (s0 + s < seq_len) {
                        const f32x4 *xp = reinterpret_cast<const f32x4 *>(x + (size_t)(s0 + s) * in_dim + k);
                        acc[s] = vt_dot8(w, xp[0], xp[1], acc[s]);
                    }
                }
            }
        } else {
            for (int k = lane; k < in_dim; k += 64) {
                const float w = __uint_as_float((unsigned)wr[k] << 16);
#pragma unroll
                for (int s = 0; s < S; s++)
                    if (s0 + s < seq_len) acc[s] = fmaf(w, x[(size_t)(s0 + s) * in_dim + k], acc[s]);
            }
        }
#pragma unroll
        for (int s = 0; s < S; s++) {
            const float v = vt_wave_sum(acc[s]);
            if (lane == 0 && s0 + s < seq_len)
                y[(size_t)(s0 + s) * out_dim + row] = bias ? __fadd_rn(bias[row], v) : v;
        }
    }
}

/* Single-row product y = W x as one stream (the decode GEMV of bf16_matvec_fused,
 * voxtral_tts_kernels.c:152-185).  A workgroup owns `rows_per_wg` consecutive rows, i.e. one
 * contiguous piece of W, and cuts it into 8 equal runs of 1 KB chunks (512 weights: 16 bytes per
 * lane), one per wave, wherever the row boundaries fall: every wave streams the same number of
 * bytes whatever the shape.  A wave keeps MV_RING chunks requested ahead (non-temporal 16-byte
 * loads, the first ones before x is even staged), multiplies each against the matching slice of
 * x in LDS, and leaves one partial sum per row it touched in part[row][wave]; the partials of a
 * row are added in wave order, so the result does not depend on timing.  x sits in LDS as
 * [chunk][half][lane][4] so that the two 16-byte reads of a lane are contiguous over the wave. */
#define MV_RING 16
#define MV_THREADS 512
#define MV_MAX_ROWS 512          /* rows per workgroup: part[] is MV_MAX_ROWS x 8 floats */

__global__ void __launch_bounds__(MV_THREADS)
vt_matvec_kernel(float *y, const float *x, const uint16_t *W, const float *bias, int in_dim, int out_dim,
                 int rows_per_wg) {
    extern __shared__ __attribute__((aligned(16))) float mv_lds[];
    float *xs = mv_lds, *part = mv_lds + in_dim;
    const int tid = (int)threadIdx.x, lane = vt_lane(), nw = (int)(blockDim.x >> 6);
    const int wave = __builtin_amdgcn_readfirstlane(vt_wave());      /* uniform: the loop bounds below are scalars */
    const int row0 = (int)blockIdx.x * rows_per_wg;
    const int rows = min(rows_per_wg, out_dim - row0);
    if (rows <= 0) return;
    const int cpr = in_dim >> 9;                                     /* chunks per row */
    const int n_wg = rows * cpr;
    const int c_lo = (int)((long long)n_wg * wave / nw), c_hi = (int)((long long)n_wg * (wave + 1) / nw);
    const int n = c_hi - c_lo;
    const uint16_t *base = W + (size_t)row0 * in_dim + (size_t)c_lo * 512 + lane * 8;
    u32x4 ring[MV_RING];
    const bool steady = n >= 2 * MV_RING;        /* then the first round is requested without conditions, too */
    if (steady) {
#pragma unroll
        for (int i = 0; i < MV_RING; i++) ring[i] = vt_ldw(base + (size_t)i * 512);
    } else {
#pragma unroll
        for (int i = 0; i < MV_RING; i++)
            if (i < n) ring[i] = vt_ldw(base + (size_t)i * 512);
    }
    for (int g = tid; g < in_dim / 4; g += (int)blockDim.x) {
        const int kc = g >> 7, within = g & 127;
        *reinterpret_cast<f32x4 *>(xs + kc * 512 + (within & 1) * 256 + (within >> 1) * 4) =
            *reinterpret_cast<const f32x4 *>(x + 4 * g);
    }
    for (int i = tid; i < rows * nw; i += (int)blockDim.x) part[i] = 0.f;
    __syncthreads();
    int r = c_lo / cpr, kc = c_lo % cpr;
    float acc = 0.f;
    const int dummy = rows * nw + tid;                 /* behind the partial sums */
    /* steady state: every slot is requested again as soon as it has been multiplied, without a
     * condition, so that the wait for slot j + 1 lets the 15 younger requests stay in flight */
    int c0 = 0;
    for (; c0 + 2 * MV_RING <= n; c0 += MV_RING) {
#pragma unroll
        for (int j = 0; j < MV_RING; j++) {
            const float *xp = xs + kc * 512 + lane * 4;
            acc = vt_dot8(ring[j], *reinterpret_cast<const f32x4 *>(xp), *reinterpret_cast<const f32x4 *>(xp + 256), acc);
            /* the request stays behind the last use of the registers it overwrites: hoisted, it would
             * land in other registers and be copied back at the end of the round, behind a wait for all */
            __builtin_amdgcn_sched_barrier(0);
            ring[j] = vt_ldw(base + (size_t)(c0 + j + MV_RING) * 512);
            __builtin_amdgcn_sched_barrier(0);
            /* no branch in this loop (behind one the compiler waits for every outstanding load):
             * the row sum is formed after every chunk and stored to a dummy slot unless the row ends */
            const bool end = ++kc == cpr;
            const float sum = vt_wave_sum(acc);
            part[lane == 0 && end ? r * nw + wave : dummy] = sum;
            acc = end ? 0.f : acc;
            r += end ? 1 : 0;
            kc = end ? 0 : kc;
        }
    }
    /* the last one or two rounds: requests only while chunks are left */
    for (; c0 < n; c0 += MV_RING) {
#pragma unroll
        for (int j = 0; j < MV_RING; j++) {
            const int c = c0 + j;
            if (c < n) {
                const u32x4 w = ring[j];
                if (c + MV_RING < n) ring[j] = vt_ldw(base + (size_t)(c + MV_RING) * 512);
                const float *xp = xs + kc * 512 + lane * 4;
                acc = vt_dot8(w, *reinterpret_cast<const f32x4 *>(xp), *reinterpret_cast<const f32x4 *>(xp + 256), acc);
                if (++kc == cpr || c == n - 1) {
                    const float sum = vt_wave_sum(acc);
                    if (lane == 0) part[r * nw + wave] = sum;
                    r++;
                    kc = 0;
                    acc = 0.f;
                }
            }
        }
    }
    __syncthreads();
    for (int i = tid; i < rows; i += (int)blockDim.x) {
        float sum = 0.f;
        for (int w = 0; w < nw; w++) sum = __fadd_rn(sum, part[i * nw + w]);
        y[row0 + i] = bias ? __fadd_rn(bias[row0 + i], sum) : sum;
    }
}

/* Shapes the stream kernel takes: whole 1 KB chunks per row, 16-byte aligned operands, x and the
 * partial sums within the 64 KB of LDS a workgroup gets without asking. */
static int matvec_launch(float *d_y, const float *d_x, const uint16_t *d_W, const float *d_bias,
                         int in_dim, int out_dim) {
    if (in_dim % 512 != 0 || (((uintptr_t)d_W | (uintptr_t)d_x) & 15)) return 0;
    /* one workgroup per CU for matrices of a few rounds per wave; up to four (two resident, the
     * others queued behind them) where a wave would otherwise run more than three rounds of its
     * ring: measured 6.3 -> 6.7 TB/s on 131072 x 3072, while 9216 x 3072 is fastest with one */
    const int n_cu = g_vt.n_cu > 0 ? g_vt.n_cu : 256;
    const long long chunks = (long long)out_dim * (in_dim / 512);
    long long want = chunks / ((MV_THREADS / 64) * 3 * MV_RING);
    const int n_wg = (int)(want < n_cu ? n_cu : (want > 4 * n_cu ? 4 * n_cu : want));
    int rows_per_wg = (out_dim + n_wg - 1) / n_wg;
    if (rows_per_wg > MV_MAX_ROWS) rows_per_wg = MV_MAX_ROWS;
    const size_t lds = sizeof(float) * ((size_t)in_dim + (size_t)rows_per_wg * (MV_THREADS / 64) + MV_THREADS);
    if (lds > 65536) return 0;
    const int grid = (out_dim + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL(vt_matvec_kernel, dim3(grid), dim3(MV_THREADS), lds, g_vt.stream, d_y, d_x, d_W, d_bias,
                       in_dim, out_dim, rows_per_wg);
    return 1;
}

void vt_launch_linear(float *d_y, const float *d_x, const uint16_t *d_W, const float *d_bias,
                      int seq_len, int in_dim, int out_dim) {
    if (seq_len == 1 && matvec_launch(d_y, d_x, d_W, d_bias, in_dim, out_dim)) return;
    const int vec_ok = (in_dim % 8 == 0) && (((uintptr_t)d_W | (uintptr_t)d_x) % 16 == 0);
    const dim3 grid((out_dim + 3) / 4), block(256);
    if (seq_len == 1)
        hipLaunchKernelGGL(vt_linear_kernel<1>, grid, block, 0, g_vt.stream, d_y, d_x, d_W, d_bias,
                           seq_len, in_dim, out_dim, vec_ok);
    else if (seq_len <= 4)
        hipLaunchKernelGGL(vt_linear_kernel<4>, grid, block, 0, g_vt.stream, d_y, d_x, d_W, d_bias,
                           seq_len, in_dim, out_dim, vec_ok);
    else
        hipLaunchKernelGGL(vt_linear_kernel<8>, grid, block, 0, g_vt.stream, d_y, d_x, d_W, d_bias,
                           seq_len, in_dim, out_dim, vec_ok);
}

/* Rows of activations against an aligned weight matrix go to the matrix cores:
 * (hi, lo) planes of x, K cut into enough ranges to fill the device, partial
 * planes summed in a fixed order.  linear_mfma_plan says whether the shape qualifies, into how
 * many ranges K is cut and how many bytes of work area (partial planes, then the two activation
 * planes) the launches need; linear_mfma_run queues them on that work area. */
static int linear_mfma_plan(const float *d_y, const float *d_x, const uint16_t *d_W, int seq_len, int in_dim,
                            int out_dim, int *splits_out, size_t *bytes_out) {
    if (seq_len < 8 || !vt_gemm_shape_ok(seq_len, out_dim, in_dim, 1) ||
        (((uintptr_t)d_W | (uintptr_t)d_x | (uintptr_t)d_y) & 15))
        return 0;
    const int tiles = ((seq_len + 127) / 128) * (out_dim / 128);
    int splits = 1;
    static const int cand[] = {2, 3, 4, 6, 8};
    for (int i = 0; i < 5 && tiles * splits < 192; i++)
        if (vt_gemm_shape_ok(seq_len, out_dim, in_dim, cand[i])) splits = cand[i];
    const size_t n_in = (size_t)seq_len * in_dim, n_out = (size_t)seq_len * out_dim;
    const size_t part_bytes = splits > 1 ? sizeof(float) * n_out * splits : 0;
    *splits_out = splits;
    *bytes_out = part_bytes + 2 * sizeof(uint16_t) * n_in;
    return 1;
}

static void linear_mfma_run(unsigned char *base, float *d_y, const float *d_x, const uint16_t *d_W, int seq_len,
                            int in_dim, int out_dim, int splits) {
    const size_t n_in = (size_t)seq_len * in_dim, n_out = (size_t)seq_len * out_dim;
    const size_t part_bytes = splits > 1 ? sizeof(float) * n_out * splits : 0;
    float *part = splits > 1 ? (float *)base : d_y;
    uint16_t *hi = (uint16_t *)(base + part_bytes), *lo = hi + n_in;
    vt_launch_split(hi, lo, d_x, n_in);
    vt_launch_gemm(part, hi, lo, d_W, seq_len, out_dim, in_dim, splits);
    if (splits > 1) vt_launch_sum_planes(d_y, part, splits, n_out, n_out);
}

/* Returns 0 when the shape does not qualify, 1 when queued, -1 on error. */
static int linear_mfma(float *d_y, const float *d_x, const uint16_t *d_W, int seq_len, int in_dim, int out_dim) {
    int splits;
    size_t bytes;
    if (!linear_mfma_plan(d_y, d_x, d_W, seq_len, in_dim, out_dim, &splits, &bytes)) return 0;
    unsigned char *base = (unsigned char *)vt_scratch(bytes);
    if (!base) return -1;
    linear_mfma_run(base, d_y, d_x, d_W, seq_len, in_dim, out_dim, splits);
    return 1;
}

/* ---- the same product for callers that cannot allocate ----------------------------------
 * The work area of the matrix-core path lives in a fixed array in device memory instead of the
 * context's growing buffer, so this entry point reaches no hipMalloc / hipFree (nor any routine
 * that allocates) on any path.  Every device that loads the library holds its own copy of the
 * array at its own address for the life of the process; the address is looked up once per device,
 * with that device current, and only that pointer is ever handed to kernels.  The array keeps the
 * last call's contents; nothing in it has to start at zero (the activation planes and every
 * element of every partial plane that is read are written by the call itself).  Calls that overlap
 * on one device would share the array: the library has one stream and is not thread-safe. */
#define VT_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
#define VT_STATIC_MAX_DEVICES 16
static __device__ __align__(256) unsigned char vt_static_scratch[VT_STATIC_SCRATCH_BYTES];
static unsigned char *s_static_ptr[VT_STATIC_MAX_DEVICES];

static unsigned char *static_scratch(void) {
    int dev = -1;
    if (vt_check(hipGetDevice(&dev), "hipGetDevice")) return NULL;
    /* the kernels run on the library's stream, which belongs to the device the context was made on:
     * the array's copy on any other device is not the one they could reach */
    if (dev != g_vt.device) {
        vt_set_error("tts_hip_linear_bf16_noalloc: current device %d is not the device of the context (%d)", dev, g_vt.device);
        return NULL;
    }
    if (dev < 0 || dev >= VT_STATIC_MAX_DEVICES) {
        vt_set_error("tts_hip_linear_bf16_noalloc: device %d beyond the %d this build keeps an address for", dev,
                     VT_STATIC_MAX_DEVICES);
        return NULL;
    }
    if (!s_static_ptr[dev]) {
        void *p = NULL;
        if (vt_check(hipGetSymbolAddress(&p, HIP_SYMBOL(vt_static_scratch)), "hipGetSymbolAddress")) return NULL;
        s_static_ptr[dev] = (unsigned char *)p;
    }
    return s_static_ptr[dev];
}

extern "C" int tts_hip_linear_bf16_noalloc(float *d_y, const float *d_x, int seq_len, int in_dim, int out_dim,
                                           const void *d_W) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_linear_bf16_noalloc: backend not initialised"); return -1; }
    if (!d_y || !d_x || !d_W || seq_len < 1 || in_dim < 1 || out_dim < 1) {
        vt_set_error("tts_hip_linear_bf16_noalloc: bad arguments");
        return -1;
    }
    int splits;
    size_t bytes;
    if (!linear_mfma_plan(d_y, d_x, (const uint16_t *)d_W, seq_len, in_dim, out_dim, &splits, &bytes)) {
        /* few rows or an unaligned shape: the row kernels, which use no work area at all */
        vt_launch_linear(d_y, d_x, (const uint16_t *)d_W, NULL, seq_len, in_dim, out_dim);
        return vt_check(hipGetLastError(), "tts_hip_linear_bf16_noalloc") ? -1 : 0;
    }
    if (bytes > VT_STATIC_SCRATCH_BYTES) {
        vt_set_error("tts_hip_linear_bf16_noalloc: %d x %d x %d needs %zu bytes of work area, the fixed one has %zu; "
                     "use tts_hip_linear_bf16", seq_len, out_dim, in_dim, bytes, (size_t)VT_STATIC_SCRATCH_BYTES);
        return -1;
    }
    unsigned char *base = static_scratch();
    if (!base) return -1;
    linear_mfma_run(base, d_y, d_x, (const uint16_t *)d_W, seq_len, in_dim, out_dim, splits);
    return vt_check(hipGetLastError(), "tts_hip_linear_bf16_noalloc") ? -1 : 0;
}

extern "C" int tts_hip_split_planes(uint16_t *d_hi, uint16_t *d_lo, const float *d_x, size_t n) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_split_planes: backend not initialised"); return -1; }
    if (!d_hi || !d_lo || !d_x || (n & 1) || (((uintptr_t)d_x) & 7) || (((uintptr_t)d_hi | (uintptr_t)d_lo) & 3)) {
        vt_set_error("tts_hip_split_planes: needs an even count and aligned device pointers");
        return -1;
    }
    if (n == 0) return 0;
    vt_launch_split(d_hi, d_lo, d_x, n);
    return vt_check(hipGetLastError(), "tts_hip_split_planes") ? -1 : 0;
}

static int is_device_ptr(const void *p) {
    hipPointerAttribute_t at;
    if (hipPointerGetAttributes(&at, p) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return at.type == hipMemoryTypeDevice;
}

extern "C" void tts_hip_linear_bf16(float *y, const float *x, const uint16_t *W_bf16,
                                    int seq_len, int in_dim, int out_dim, const void *W_gpu) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_linear_bf16: backend not initialised"); return; }
    if (seq_len < 1 || in_dim < 1 || out_dim < 1) { vt_set_error("tts_hip_linear_bf16: bad shape"); return; }
    const size_t xb = sizeof(float) * (size_t)seq_len * in_dim, yb = sizeof(float) * (size_t)seq_len * out_dim;
    const size_t wb = 2 * (size_t)out_dim * in_dim;
    const int x_dev = is_device_ptr(x), y_dev = is_device_ptr(y);
    float *dx = (float *)x, *dy = y;
    void *dW = (void *)W_gpu, *tmp_x = NULL, *tmp_y = NULL, *tmp_W = NULL;
    if (!x_dev) {
        if (!(tmp_x = vt_dev_alloc(xb))) return;
        if (vt_check(hipMemcpy(tmp_x, x, xb, hipMemcpyHostToDevice), "linear x upload")) goto done;
        dx = (float *)tmp_x;
    }
    if (!dW) {
        if (!W_bf16) { vt_set_error("tts_hip_linear_bf16: no weights given"); goto done; }
        if (!(tmp_W = vt_dev_alloc(wb))) goto done;
        if (vt_check(hipMemcpy(tmp_W, W_bf16, wb, hipMemcpyHostToDevice), "linear W upload")) goto done;
        dW = tmp_W;
    }
    if (!y_dev) {
        if (!(tmp_y = vt_dev_alloc(yb))) goto done;
        dy = (float *)tmp_y;
    }
    {
        const int r = linear_mfma(dy, dx, (const uint16_t *)dW, seq_len, in_dim, out_dim);
        if (r < 0) goto done;
        if (r == 0) vt_launch_linear(dy, dx, (const uint16_t *)dW, NULL, seq_len, in_dim, out_dim);
    }
    if (!y_dev || tmp_x || tmp_W) {
        if (vt_check(hipStreamSynchronize(g_vt.stream), "linear sync")) goto done;
        if (!y_dev) (void)vt_check(hipMemcpy(y, dy, yb, hipMemcpyDeviceToHost), "linear y download");
    }
done:
    if (tmp_x) (void)hipFree(tmp_x);
    if (tmp_y) (void)hipFree(tmp_y);
    if (tmp_W) (void)hipFree(tmp_W);
}

/* ---- RMSNorm: one workgroup per row ------------------------------------------ */

__global__ void __launch_bounds__(256)
vt_rms_norm_kernel(float *out, const float *x, const float *w, int dim, float eps) {
    __shared__ float lds[VT_MAX_WAVES];
    vt_block_rmsnorm<false>(out + (size_t)blockIdx.x * dim, x + (size_t)blockIdx.x * dim, w, dim, eps, lds);
}

void vt_launch_rms_norm(float *d_out, const float *d_x, const float *d_w, int seq, int dim, float eps) {
    hipLaunchKernelGGL(vt_rms_norm_kernel, dim3(seq), dim3(256), 0, g_vt.stream, d_out, d_x, d_w, dim, eps);
}

extern "C" void tts_hip_rms_norm(float *d_out, const float *d_x, const float *d_weight,
                                 int seq_len, int dim, float eps) {
    if (!g_vt.initialized || seq_len < 1 || dim < 1) { vt_set_error("tts_hip_rms_norm: bad call"); return; }
    vt_launch_rms_norm(d_out, d_x, d_weight, seq_len, dim, eps);
}

/* ---- RoPE on adjacent pairs with a (cos, sin) table ---------------------------- */

__global__ void vt_rope_kernel(float *x, const float *freqs, int seq, int heads, int head_dim) {
    const int half = head_dim / 2;
    const size_t total = (size_t)seq * heads * half;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const int d = (int)(i % half);
        const size_t sh = i / half;
        const int s = (int)(sh / heads);
        const float c = freqs[((size_t)s * half + d) * 2], sn = freqs[((size_t)s * half + d) * 2 + 1];
        float *v = x + sh * head_dim + 2 * d;
        const float a = v[0], b = v[1];
        v[0] = __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, sn));
        v[1] = __fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, c));
    }
}

extern "C" void tts_hip_apply_rope(float *d_x, const float *d_freqs, int seq, int heads, int head_dim) {
    if (!g_vt.initialized || seq < 1 || heads < 1 || head_dim < 2 || (head_dim & 1)) {
        vt_set_error("tts_hip_apply_rope: bad call");
        return;
    }
    const size_t total = (size_t)seq * heads * (head_dim / 2);
    const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
    hipLaunchKernelGGL(vt_rope_kernel, dim3(blocks), dim3(256), 0, g_vt.stream, d_x, d_freqs, seq, heads, head_dim);
}

/* The table is evaluated on the host with libm in the operation order of
 * voxtral_tts_kernels.c:602-614, then copied: entries are bit-equal to the CPU path. */
extern "C" void tts_hip_compute_rope_freqs(float *d_freqs, int start_pos, int seq, int dim, float theta) {
    if (!g_vt.initialized || seq < 1 || dim < 2) { vt_set_error("tts_hip_compute_rope_freqs: bad call"); return; }
    const int half = dim / 2;
    float *t = (float *)malloc(sizeof(float) * (size_t)seq * half * 2);
    if (!t) { vt_set_error("tts_hip_compute_rope_freqs: out of host memory"); return; }
    for (int s = 0; s < seq; s++) {
        const float p = (float)(start_pos + s);
        for (int d = 0; d < half; d++) {
            const float f = 1.0f / powf(theta, (float)(2 * d) / (float)dim);
            volatile float ang = p * f;
            t[((size_t)s * half + d) * 2] = cosf(ang);
            t[((size_t)s * half + d) * 2 + 1] = sinf(ang);
        }
    }
    (void)hipStreamSynchronize(g_vt.stream);
    (void)vt_check(hipMemcpy(d_freqs, t, sizeof(float) * (size_t)seq * half * 2, hipMemcpyHostToDevice),
                   "rope table copy");
    free(t);
}

/* ---- SiLU(gate) * up, residual add --------------------------------------------- */

__global__ void vt_silu_mul_kernel(float *gate, const float *up, int n) {
    for (int i = (int)(blockIdx.x * blockDim.x + threadIdx.x); i < n; i += (int)(gridDim.x * blockDim.x)) {
        const float g = gate[i];
        gate[i] = __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, expf(-g))), up[i]);
    }
}

__global__ void vt_add_kernel(float *a, const float *b, int n) {
    for (int i = (int)(blockIdx.x * blockDim.x + threadIdx.x); i < n; i += (int)(gridDim.x * blockDim.x))
        a[i] = __fadd_rn(a[i], b[i]);
}

static int ew_blocks(int n) { int b = (n + 255) / 256; return b > 2048 ? 2048 : b; }

extern "C" void tts_hip_silu_mul(float *d_gate, const float *d_up, int n) {
    if (!g_vt.initialized || n < 1) { vt_set_error("tts_hip_silu_mul: bad call"); return; }
    hipLaunchKernelGGL(vt_silu_mul_kernel, dim3(ew_blocks(n)), dim3(256), 0, g_vt.stream, d_gate, d_up, n);
}

void vt_launch_add(float *d_a, const float *d_b, int n) {
    hipLaunchKernelGGL(vt_add_kernel, dim3(ew_blocks(n)), dim3(256), 0, g_vt.stream, d_a, d_b, n);
}

extern "C" void tts_hip_add_inplace(float *d_a, const float *d_b, int n) {
    if (!g_vt.initialized || n < 1) { vt_set_error("tts_hip_add_inplace: bad call"); return; }
    vt_launch_add(d_a, d_b, n);
}

/* ---- attention, any head geometry (head_dim <= 256, multiple of 64) ------------- */
/* Workgroup = (head, query).  Waves stride over the keys, each lane owns
 * head_dim/64 dims; per-wave online softmax, merged over the waves in LDS.
 * Keys visible to query i: [0, min(q_offset+i+1, seq_k)) when causal, else all. */
__global__ void __launch_bounds__(256)
vt_attention_kernel(float *out, const float *Q, const float *K, const float *V, int q_offset,
                    int seq_k, int causal, int n_heads, int n_kv_heads, int head_dim,
                    float scale, int kv_stride, int q_stride) {
    __shared__ float part[4][2 + 256];
    const int h = (int)blockIdx.x, i = (int)blockIdx.y;
    const int kvh = h / (n_heads / n_kv_heads);
    const int lane = vt_lane(), wave = vt_wave(), nw = (int)(blockDim.x >> 6);
    const int per = head_dim / 64;
    int kend = seq_k;
    if (causal) { kend = q_offset + i + 1; if (kend > seq_k) kend = seq_k; }
    const float *q = Q + (size_t)i * q_stride + (size_t)h * head_dim;
    float qv[4], o[4];
    for (int e = 0; e < 4; e++) { qv[e] = e < per ? q[lane + 64 * e] : 0.f; o[e] = 0.f; }
    float m = -1e30f, l = 0.f;
    for (int j = wave; j < kend; j += nw) {
        const float *kr = K + (size_t)j * kv_stride + kvh * head_dim;
        const float *vr = V + (size_t)j * kv_stride + kvh * head_dim;
        float s = 0.f;
        for (int e = 0; e < per; e++) s = fmaf(qv[e], kr[lane + 64 * e], s);
        s = __fmul_rn(vt_wave_sum(s), scale);
        const float mn = fmaxf(m, s);
        const float corr = expf(m - mn), p = expf(s - mn);
        l = fmaf(l, corr, p);
        for (int e = 0; e < per; e++) o[e] = fmaf(o[e], corr, p * vr[lane + 64 * e]);
        m = mn;
    }
    if (lane == 0) { part[wave][0] = m; part[wave][1] = l; }
    for (int e = 0; e < per; e++) part[wave][2 + lane + 64 * e] = o[e];
    __syncthreads();
    for (int d = (int)threadIdx.x; d < head_dim; d += (int)blockDim.x) {
        float M = -1e30f;
        for (int w = 0; w < nw; w++) M = fmaxf(M, part[w][0]);
        float L = 0.f, O = 0.f;
        for (int w = 0; w < nw; w++) {
            const float e = expf(part[w][0] - M);
            L = fmaf(part[w][1], e, L);
            O = fmaf(part[w][2 + d], e, O);
        }
        out[((size_t)i * n_heads + h) * head_dim + d] = L > 0.f ? __fmul_rn(O, __fdiv_rn(1.0f, L)) : 0.f;
    }
}

void vt_launch_attention(float *d_out, const float *d_Q, const float *d_K, const float *d_V,
                         int seq_q, int q_offset, int seq_k, int causal, int n_heads,
                         int n_kv_heads, int head_dim, float scale, int kv_stride, int q_stride) {
    hipLaunchKernelGGL(vt_attention_kernel, dim3(n_heads, seq_q), dim3(256), 0, g_vt.stream, d_out, d_Q,
                       d_K, d_V, q_offset, seq_k, causal, n_heads, n_kv_heads, head_dim, scale, kv_stride,
                       q_stride);
}

static int attn_args_ok(const char *who, int seq_q, int seq_k, int n_heads, int n_kv_heads, int head_dim) {
    if (g_vt.initialized && seq_q >= 1 && seq_k >= 1 && n_heads >= 1 && n_kv_heads >= 1 &&
        n_heads % n_kv_heads == 0 && head_dim >= 64 && head_dim <= 256 && head_dim % 64 == 0)
        return 1;
    vt_set_error("%s: unsupported arguments (heads %d/%d, head_dim %d, seq %d/%d)", who, n_heads,
                 n_kv_heads, head_dim, seq_q, seq_k);
    return 0;
}

extern "C" void tts_hip_causal_attention_decode(float *d_out, const float *d_Q, const float *d_K_cache,
                                                const float *d_V_cache, int seq_k, int n_heads,
                                                int n_kv_heads, int head_dim, float scale,
                                                int kv_cache_stride) {
    if (!attn_args_ok("tts_hip_causal_attention_decode", 1, seq_k, n_heads, n_kv_heads, head_dim)) return;
    const int stride = kv_cache_stride > 0 ? kv_cache_stride : n_kv_heads * head_dim;
    vt_launch_attention(d_out, d_Q, d_K_cache, d_V_cache, 1, seq_k - 1, seq_k, 1, n_heads, n_kv_heads,
                        head_dim, scale, stride, n_heads * head_dim);
}

extern "C" void tts_hip_causal_attention_prefill(float *d_out, const float *d_Q, const float *d_K,
                                                 const float *d_V, int seq_len, int start_pos,
                                                 int n_heads, int n_kv_heads, int head_dim, float scale) {
    if (!attn_args_ok("tts_hip_causal_attention_prefill", seq_len, start_pos + seq_len, n_heads,
                      n_kv_heads, head_dim)) return;
    if (start_pos < 0) { vt_set_error("tts_hip_causal_attention_prefill: negative start_pos"); return; }
    if (n_heads == VT_HEADS && n_kv_heads == VT_KV_HEADS && head_dim == VT_HEAD_DIM && seq_len >= 8 &&
        !(((uintptr_t)d_out | (uintptr_t)d_Q | (uintptr_t)d_K | (uintptr_t)d_V) & 15)) {
        vt_launch_prefill_attention(d_out, NULL, NULL, d_Q, VT_Q_DIM, d_K, d_V, seq_len, start_pos, scale);
        return;
    }
    vt_launch_attention(d_out, d_Q, d_K, d_V, seq_len, start_pos, start_pos + seq_len, 1, n_heads,
                        n_kv_heads, head_dim, scale, n_kv_heads * head_dim, n_heads * head_dim);
}

extern "C" void tts_hip_bidirectional_attention(float *d_out, const float *d_Q, const float *d_K,
                                                const float *d_V, int seq_len, int n_heads,
                                                int n_kv_heads, int head_dim, float scale) {
    if (!attn_args_ok("tts_hip_bidirectional_attention", seq_len, seq_len, n_heads, n_kv_heads, head_dim))
        return;
    vt_launch_attention(d_out, d_Q, d_K, d_V, seq_len, 0, seq_len, 0, n_heads, n_kv_heads, head_dim,
                        scale, n_kv_heads * head_dim, n_heads * head_dim);
}

/* ---- embedding lookup ------------------------------------------------------------ */

__global__ void vt_embed_kernel(float *out, const uint16_t *emb, int token_id, int dim) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i < dim) out[i] = __uint_as_float((unsigned)emb[(size_t)token_id * dim + i] << 16);
}

extern "C" void tts_hip_embed_token(float *d_out, const void *d_embeddings_bf16, int token_id, int dim) {
    if (!g_vt.initialized || token_id < 0 || dim < 1) { vt_set_error("tts_hip_embed_token: bad call"); return; }
    hipLaunchKernelGGL(vt_embed_kernel, dim3((dim + 255) / 256), dim3(256), 0, g_vt.stream, d_out,
                       (const uint16_t *)d_embeddings_bf16, token_id, dim);
}
