/*
 * voxtral_tts_hip_bench.h - C ABI of libvoxtral_tts_hip_bench.so, the benchmark companion of
 * libvoxtral_tts_hip.so (include/voxtral_tts_hip.h).  Timing loops and benchmark inputs only: nothing
 * here is needed to run the model, and none of it has a counterpart in the reference.  The companion
 * links against the product library and shares its one global context, so tts_hip_init and the uploads
 * come first; every figure is taken with events on the library's stream around the product's own launches.
 */
#ifndef VOXTRAL_TTS_HIP_BENCH_H
#define VOXTRAL_TTS_HIP_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Event timing on the library's stream: start records an event, stop records a second one, waits for
 * it and returns the milliseconds between them (negative on error, or when a whole-step decode kernel
 * of the timed region left early on a timed-out barrier). */
void tts_hip_timer_start(void);
float tts_hip_timer_stop_ms(void);

/* Average duration in ms of one launch of a single kernel over `iters` launches on pseudo-random
 * activations of normal size (on zeros the matrix cores draw less power and the products measure
 * 5-15 % faster than in a real pass; needs the weights uploaded; launch i takes the weights of uploaded
 * layer i modulo their number, so that they come from HBM as in a real pass): which 0..3 = sequence-level
 * product at M = 512 with the q|k|v, output, gate/up and down projection; 4 = causal attention at 512
 * queries (KV cache of at least 512 rows); 10..13 = the four acoustic phase kernels, 14 = the four of them
 * in order on one layer (the value is the duration of all four); 20..23 = the codec's fp32 product at 1600
 * rows with the q|k|v, output, gate|up and down matrices, 24 = the whole codec decoder on 200 frames
 * (codec weights uploaded).  Negative on error. */
float tts_hip_bench_kernel(int which, int iters);

/* Average duration in ms of one single-row product y[out_dim] = W[out_dim, in_dim] x (the kernel
 * behind tts_hip_linear_bf16 with seq_len 1) over `iters` launches.  Launch i reads copy i % n_copies
 * of W, `copy_stride` elements apart, so that a matrix smaller than the memory-side cache is streamed
 * from HBM every time.  Device pointers.  Negative on error. */
float tts_hip_bench_matvec(float *d_y, const float *d_x, const uint16_t *d_W, size_t copy_stride,
                           int n_copies, int in_dim, int out_dim, int iters);

/* What a grid shaped like the whole-step decode kernel's can stream: one launch reads every matrix of
 * the uploaded backbone layers once (6.05 GB at 26 layers) with that kernel's grid (one workgroup of 8
 * waves per CU), per-wave shares, load type (16-byte non-temporal, 1 KB per wave instruction) and ring
 * depth (18 loads in flight per wave), and does nothing else: no arithmetic, no staging, no hand-overs.
 * Returns the average ms per launch over `iters` launches and, through bytes_per_launch (may be NULL),
 * the bytes one launch reads.  Negative on error. */
float tts_hip_bench_stream_ceiling(int iters, double *bytes_per_launch);

/* Fills n floats of device memory with pseudo-random values of magnitude 2^-7 .. 2 (a fill kernel on the
 * library's stream, no memset), e.g. rows of the KV cache for a decode benchmark at a long position.
 * 0 / -1. */
int tts_hip_bench_fill_f32(float *d_ptr, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* VOXTRAL_TTS_HIP_BENCH_H */
