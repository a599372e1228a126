/*
 * vt_bench.hip - libvoxtral_tts_hip_bench.so: timing loops for benchmarks, kept out of the product
 * library.  Links against libvoxtral_tts_hip.so and shares its context (stream, events, weights):
 * every loop here queues the product's own launches (the functions the real passes call) between
 * two events on the library's stream.  Also a plain streaming kernel that measures what the memory
 * system delivers to a grid shaped like the whole-step decode kernel's, and fill kernels for
 * benchmark inputs.  Declared in include/voxtral_tts_hip_bench.h.
 */
#include "vt_state.h"
#include "vt_gemm.h"
#include "../../include/voxtral_tts_hip_bench.h"

/* ---- event timing on the library's stream ------------------------------------------- */

extern "C" void tts_hip_timer_start(void) {
    (void)vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "timer start");
}

extern "C" float tts_hip_timer_stop_ms(void) {
    float ms = -1.f;
    if (vt_check(hipEventRecord(g_vt.ev1, g_vt.stream), "timer stop")) return ms;
    if (vt_check(hipEventSynchronize(g_vt.ev1), "timer sync")) return ms;
    (void)vt_check(hipEventElapsedTime(&ms, g_vt.ev0, g_vt.ev1), "timer elapsed");
    if (vt_step_poll_abort()) return -1.f;      /* a step of the timed region was abandoned: no figure */
    return ms;
}

static float timed_stop(int iters) {
    float ms = -1.f;
    if (vt_check(hipEventRecord(g_vt.ev1, g_vt.stream), "bench stop")) return -1.f;
    if (vt_check(hipEventSynchronize(g_vt.ev1), "bench sync")) return -1.f;
    if (vt_check(hipGetLastError(), "bench launch")) return -1.f;
    if (vt_check(hipEventElapsedTime(&ms, g_vt.ev0, g_vt.ev1), "bench time")) return -1.f;
    return ms / (float)iters;
}

/* ---- benchmark inputs ------------------------------------------------------------------- */

static int bn_blocks(size_t n) { size_t b = (n + 255) / 256; return (int)(b > 8192 ? 8192 : b); }

/* Pseudo-random bf16 values of the size of normalised activations, hi in +-(2^-7 .. 2) and
 * (d_lo != NULL) lo 2^-9 of that with a mantissa of its own.  Written over a float array as 2 n halves it
 * gives floats of the same range. */
__global__ void vt_bench_fill_kernel(uint16_t *hi, uint16_t *lo, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        unsigned h = (unsigned)i * 2654435761u + 12345u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        /* sign, an exponent in 120..127 (2^-7 .. 1, times 1.x), 7 mantissa bits */
        hi[i] = (uint16_t)(((h & 1u) << 15) | ((120u + ((h >> 1) & 7u)) << 7) | ((h >> 4) & 127u));
        if (lo) lo[i] = (uint16_t)((((h >> 11) & 1u) << 15) | ((111u + ((h >> 1) & 7u)) << 7) | ((h >> 12) & 127u));
    }
}

static void bench_fill(uint16_t *d_hi, uint16_t *d_lo, size_t n) {
    hipLaunchKernelGGL(vt_bench_fill_kernel, dim3(bn_blocks(n)), dim3(256), 0, g_vt.stream, d_hi, d_lo, n);
}

extern "C" int tts_hip_bench_fill_f32(float *d_ptr, size_t n) {
    if (!g_vt.initialized || !d_ptr) { vt_set_error("tts_hip_bench_fill_f32: bad call"); return -1; }
    bench_fill((uint16_t *)d_ptr, NULL, 2 * n);
    return vt_check(hipGetLastError(), "tts_hip_bench_fill_f32") ? -1 : 0;
}

/* ---- single kernels of the prefill, the acoustic transformer and the codec -------------------- */

static float bench_prefill_kernel(int which, int iters) {
    if (which < 0 || which > 4 || g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_bench_kernel: unknown kernel %d", which); return -1.f; }
    const int S = 512;
    if (which == 4 && g_vt.kv_max < S) { vt_set_error("tts_hip_bench_kernel: KV cache shorter than 512"); return -1.f; }
    static const int NN[4] = {VT_QKV_DIM, VT_DIM, 2 * VT_FFN, VT_DIM}, KK[4] = {VT_DIM, VT_Q_DIM, VT_DIM, VT_FFN};
    const int SP[4] = {vt_prefill_cuts(4 * (VT_QKV_DIM / 256), 4), vt_prefill_cuts(4 * (VT_DIM / 256), 8), 1,
                       vt_prefill_cuts(4 * (VT_DIM / 256), 8)};
    static const int RP[4] = {2, 4, 1, 4};            /* row-major weights: cuts that divide K */
    const size_t n_out = (size_t)S * 2 * VT_FFN * 4, n_plane = (size_t)S * VT_FFN, n_q = (size_t)S * VT_Q_DIM;
    const size_t bytes = sizeof(float) * (n_out + n_q) + 2 * sizeof(uint16_t) * n_plane;
    unsigned char *base = (unsigned char *)vt_scratch(bytes);
    if (!base) return -1.f;
    float *out = (float *)base, *q = out + n_out;
    uint16_t *hi = (uint16_t *)(q + n_q), *lo = hi + n_plane;
    /* The kernels do the same work on any data, but not at the same clock: on planes of zeros the matrix
     * cores draw less power and the products measure 5-15 % faster than inside a prefill.  The planes get
     * values of the size a normalised activation has. */
    if (which < 4)
        bench_fill(hi, lo, n_plane);
    else                                              /* q: floats whose upper halves are such bf16 values */
        bench_fill((uint16_t *)q, NULL, 2 * n_q);
    /* the attention alone: the tile images of layer 0's cache are made once, in front of the loop (in a
     * prefill the kernel that appends the new rows to the cache writes them) */
    unsigned char *img = NULL;
    if (which == 4) {
        if (!(img = vt_pa_image(S))) return -1.f;
        vt_pa_launch_image(img, NULL, 0, 0, g_hip.kv_cache_k_gpu, g_hip.kv_cache_v_gpu, S, 0);
    }
    for (int it = -2; it < iters; it++) {
        if (it == 0 && vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "bench start")) return -1.f;
        /* every launch takes the next layer's weights, as in a prefill: launched again and again on
         * one layer they would be served from the memory-side cache */
        const vt_layer_dev *L = &g_vt.h_layers[(it + 2) % g_vt.n_dec_layers];
        const uint16_t *W[4] = {L->wqkv, L->wo, L->w13, L->w2};
        const vt_layer_frag *F = &g_vt.h_frag[(it + 2) % g_vt.n_dec_layers];
        const uint16_t *Wf[4] = {F->wqkv, F->wo, F->w13, F->w2};
        const bool frag = F->wqkv && F->wo && F->w13 && F->w2;
        if (which == 2 && frag) {                       /* as in the prefill: main part + K-cut tail */
            const int tail = 8 * 256, main_cols = 2 * VT_FFN - tail;
            uint16_t *h_hi = (uint16_t *)out, *h_lo = h_hi + n_plane;
            vt_launch_gemm_frag_swiglu(h_hi, h_lo, VT_FFN, out + (size_t)S * 2 * VT_FFN, hi, lo, Wf[2], S, main_cols, tail, VT_DIM,
                                       VT_W13_TAIL_CUT);
        } else if (which == 2) {
            const int tail = 16 * 128, main_cols = 2 * VT_FFN - tail;
            vt_launch_gemm_ex(out, 2 * VT_FFN, 0, hi, lo, W[2], S, main_cols, VT_DIM, 1);
            vt_launch_gemm_ex(out + (size_t)S * 2 * VT_FFN, tail, (size_t)S * tail, hi, lo,
                              W[2] + (size_t)main_cols * VT_DIM, S, tail, VT_DIM, 4);
        } else if (which < 4 && frag) vt_launch_gemm_frag(out, NN[which], (size_t)S * NN[which], hi, lo, Wf[which], S, NN[which], KK[which], SP[which]);
        else if (which < 4) vt_launch_gemm(out, hi, lo, W[which], S, NN[which], KK[which], RP[which]);
        else vt_launch_prefill_attention_raw(out, NULL, NULL, q, VT_Q_DIM, 1, 0, NULL, img, S, 0, VT_ATT_SCALE);
    }
    return timed_stop(iters);
}

static float bench_acoustic_phase(int phase, int iters) {
    size_t n = 0;
    float *base = vt_ac_work_area(&n);
    if (!base) return -1.f;
    if (vt_check(hipMemsetAsync(base, 0, sizeof(float) * n, g_vt.stream), "bench clear")) return -1.f;
    for (int it = -2; it < iters; it++) {
        if (it == 0 && vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "bench start")) return -1.f;
        /* phase 4: the four launches of one layer in order, every iteration on the next layer, as
         * inside a frame (700 MB of weights per turn: none of them is still cached when it comes
         * round again).  A single phase launched again and again re-reads weights that partly sit
         * in the memory-side cache and comes out faster than inside a frame. */
        if (vt_ac_launch_layer_phase((it + 2) % TTS_HIP_AC_LAYERS, phase)) return -1.f;
    }
    return timed_stop(iters);
}

static float bench_codec(int which, int iters) {
    float *xn, *att, *h;
    int *codes;
    if (vt_codec_probe_buffers(&xn, &att, &h, &codes)) return -1.f;
    const int frames = 200, T = frames * 8;
    if (which == 4) {
        if (vt_check(hipMemsetAsync(codes, 0, (size_t)frames * 37 * sizeof(int), g_vt.stream), "bench clear")) return -1.f;
    } else {
        /* non-zero operands: on zeros the matrix cores draw less power and run at a higher clock */
        bench_fill((uint16_t *)xn, NULL, (size_t)T * 1024 * 2);
        bench_fill((uint16_t *)att, NULL, (size_t)T * 1024 * 2);
        bench_fill((uint16_t *)h, NULL, (size_t)T * 4096 * 2);
    }
    for (int it = -2; it < iters; it++) {
        if (it == 0 && vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "bench start")) return -1.f;
        if (vt_codec_probe_launch(which)) return -1.f;
    }
    return timed_stop(iters);
}

extern "C" float tts_hip_bench_kernel(int which, int iters) {
    if (!g_vt.initialized || iters < 1) { vt_set_error("tts_hip_bench_kernel: bad call"); return -1.f; }
    if (which >= 10 && which <= 14) return bench_acoustic_phase(which - 10, iters);
    if (which >= 20 && which <= 24) return bench_codec(which - 20, iters);
    return bench_prefill_kernel(which, iters);
}

extern "C" float tts_hip_bench_matvec(float *d_y, const float *d_x, const uint16_t *d_W, size_t copy_stride,
                                      int n_copies, int in_dim, int out_dim, int iters) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_bench_matvec: backend not initialised"); return -1.f; }
    if (!d_y || !d_x || !d_W || n_copies < 1 || in_dim < 1 || out_dim < 1 || iters < 1) {
        vt_set_error("tts_hip_bench_matvec: bad arguments");
        return -1.f;
    }
    for (int i = 0; i < n_copies; i++)                                  /* warm-up: one pass over every copy */
        vt_launch_linear(d_y, d_x, d_W + (size_t)i * copy_stride, NULL, 1, in_dim, out_dim);
    if (vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "bench record")) return -1.f;
    for (int i = 0; i < iters; i++)
        vt_launch_linear(d_y, d_x, d_W + (size_t)(i % n_copies) * copy_stride, NULL, 1, in_dim, out_dim);
    return timed_stop(iters);
}

/* ---- what a grid of the decode kernel's shape can stream ---------------------------------------
 * One workgroup of 512 threads per CU, as the whole-step decode kernel; a wave owns the same contiguous
 * share of every matrix as there (1/2048 of it: 18, 12, 54 and 27 KB of q|k|v, output, gate|up and down
 * projection per layer), reads it with the same 16-byte non-temporal loads, 1 KB per wave instruction, and
 * keeps the same 18 of them in flight (the row ring of vt_decode_phases.h).  No arithmetic beyond an
 * exclusive-or that keeps the loads alive, no staging, no hand-overs: what is left is the memory system
 * and the load path of a CU.  One launch walks the uploaded backbone layers once (6.05 GB at 26). */
#define SC_RING 18

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_stream_ceiling_kernel(const vt_layer_dev *layers, int n_layers, unsigned *sink) {
    const int lane = vt_lane();
    const size_t wave = (size_t)blockIdx.x * (blockDim.x >> 6) + vt_wave();
    const size_t n_waves = (size_t)gridDim.x * (blockDim.x >> 6);
    u32x4 ring[SC_RING];
    u32x4 acc = {0u, 0u, 0u, 0u};
    static const size_t ELEMS[4] = {(size_t)VT_QKV_DIM * VT_DIM, (size_t)VT_DIM * VT_Q_DIM, (size_t)2 * VT_FFN * VT_DIM,
                                    (size_t)VT_DIM * VT_FFN};
    /* the whole walk as one sequence of 1 KB chunks: the wave's share of matrix m of layer l, m and l ascending;
     * past the end the last chunk is read again (requests stay unconditional, so the compiler's wait counts
     * stay exact) */
    int l = 0, m = 0, c = 0;
    int per = (int)(ELEMS[0] / 512 / n_waves);
    const uint16_t *p = layers[0].wqkv + wave * (size_t)per * 512 + (size_t)lane * 8;
    auto next = [&]() -> const uint16_t * {
        const uint16_t *q = p;
        if (c + 1 < per) { c++; p += 512; return q; }
        if (m == 3 && l + 1 == n_layers) return q;                 /* the end: stay on the last chunk */
        c = 0;
        if (++m == 4) { m = 0; l++; }
        per = (int)(ELEMS[m] / 512 / n_waves);
        const vt_layer_dev &L = layers[l];
        const uint16_t *W = m == 0 ? L.wqkv : m == 1 ? L.wo : m == 2 ? L.w13 : L.w2;
        p = W + wave * (size_t)per * 512 + (size_t)lane * 8;
        return q;
    };
    int total = 0;
    for (int k = 0; k < 4; k++) total += (int)(ELEMS[k] / 512 / n_waves);
    total *= n_layers;
#pragma unroll
    for (int j = 0; j < SC_RING; j++) ring[j] = vt_ldw(next());
    for (int t0 = 0; t0 < total; t0 += SC_RING) {
#pragma unroll
        for (int j = 0; j < SC_RING; j++) {
            acc ^= ring[j];
            __builtin_amdgcn_sched_barrier(0);
            ring[j] = vt_ldw(next());
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int j = 0; j < SC_RING; j++) acc ^= ring[j];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;      /* keeps the loads alive */
}

extern "C" float tts_hip_bench_stream_ceiling(int iters, double *bytes_per_launch) {
    if (!g_vt.initialized || iters < 1 || g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_bench_stream_ceiling: bad call"); return -1.f; }
    const int grid = g_vt.grid;
    if ((size_t)VT_QKV_DIM * VT_DIM / 512 % ((size_t)grid * 8) || (size_t)VT_DIM * VT_Q_DIM / 512 % ((size_t)grid * 8) ||
        (size_t)2 * VT_FFN * VT_DIM / 512 % ((size_t)grid * 8) || (size_t)VT_DIM * VT_FFN / 512 % ((size_t)grid * 8)) {
        vt_set_error("tts_hip_bench_stream_ceiling: grid %d does not divide the matrices evenly", grid);
        return -1.f;
    }
    if (bytes_per_launch)
        *bytes_per_launch = 2.0 * ((double)VT_QKV_DIM * VT_DIM + (double)VT_DIM * VT_Q_DIM + 2.0 * VT_FFN * VT_DIM + (double)VT_DIM * VT_FFN) *
                            g_vt.n_dec_layers;
    for (int it = -2; it < iters; it++) {
        if (it == 0 && vt_check(hipEventRecord(g_vt.ev0, g_vt.stream), "bench start")) return -1.f;
        hipLaunchKernelGGL(vt_stream_ceiling_kernel, dim3(grid), dim3(VT_STEP_THREADS), 0, g_vt.stream, g_vt.d_layers,
                           g_vt.n_dec_layers, (unsigned *)g_vt.d_abort + 16);
    }
    return timed_stop(iters);
}
