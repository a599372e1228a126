/*
 * vt_device.h - device-side building blocks shared by the gfx950 kernels:
 * wave64 reductions over DPP, bf16 widening, streaming 16-byte weight loads
 * and the bounded grid barrier used by the persistent kernels.
 */
#ifndef VT_DEVICE_H
#define VT_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vt_rowsplit.h"

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define VT_WAVE 64

#define VT_EPS      1e-5f

/* The thread index goes through an empty asm: what a phase of a persistent kernel derives from
 * it (lane offsets, row pointers) is then recomputed where it is used instead of being hoisted
 * out of the layer loop and kept in registers, or in scratch, for the whole kernel. */
__device__ __forceinline__ int vt_tid() { int t = (int)threadIdx.x; asm volatile("" : "+v"(t)); return t; }
__device__ __forceinline__ int vt_lane() { return vt_tid() & (VT_WAVE - 1); }
__device__ __forceinline__ int vt_wave() { return vt_tid() >> 6; }

/* bf16 pair packed in a dword: element 0 in the low half. Widening is exact. */
__device__ __forceinline__ float vt_bf16_lo(unsigned int w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float vt_bf16_hi(unsigned int w) { return __uint_as_float(w & 0xffff0000u); }

/* 16-byte streaming load of 8 bf16 weights: weights are read once per step,
 * so they are marked non-temporal to keep the small activation vectors and
 * the KV cache resident in L2. */
typedef __attribute__((address_space(1))) const u32x4 vt_global_u32x4;
__device__ __forceinline__ u32x4 vt_ldw(const uint16_t *p) {
    /* weights live in device memory: say so, or pointers read from a struct in
     * memory are treated as generic and become FLAT loads, which also occupy
     * the LDS counter */
    return __builtin_nontemporal_load((vt_global_u32x4 *)p);
}

template <int CTRL>
__device__ __forceinline__ float vt_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

/* Sum over each row of 16 lanes; every lane of the row receives the row sum.
 * quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141,
 * row_mirror = 0x140. */
__device__ __forceinline__ float vt_row16_sum(float v) {
    v += vt_dpp<0xB1>(v);
    v += vt_dpp<0x4E>(v);
    v += vt_dpp<0x141>(v);
    v += vt_dpp<0x140>(v);
    return v;
}

__device__ __forceinline__ float vt_row16_max(float v) {
    v = fmaxf(v, vt_dpp<0xB1>(v));
    v = fmaxf(v, vt_dpp<0x4E>(v));
    v = fmaxf(v, vt_dpp<0x141>(v));
    v = fmaxf(v, vt_dpp<0x140>(v));
    return v;
}

__device__ __forceinline__ float vt_readlane(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

/* Full wave64 sum in a fixed order; the result is wave-uniform. */
__device__ __forceinline__ float vt_wave_sum(float v) {
    v = vt_row16_sum(v);
    float a = vt_readlane(v, 0) + vt_readlane(v, 16);
    float b = vt_readlane(v, 32) + vt_readlane(v, 48);
    return a + b;
}

/* Full wave64 sum that ends in lane 63 only (other lanes hold partial sums):
 * 4 steps inside each row of 16, then row_bcast:15 into rows 1 and 3 and
 * row_bcast:31 into rows 2 and 3.  No scalar round trip. */
__device__ __forceinline__ float vt_wave_sum_lane63(float v) {
    v = vt_row16_sum(v);
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xc, 0xf, false));
    return v;
}

/* 8 weights (one 16-byte load) times 8 activations, accumulated with FMA. */
__device__ __forceinline__ float vt_dot8(u32x4 w, f32x4 xa, f32x4 xb, float acc) {
    acc = fmaf(vt_bf16_lo(w.x), xa.x, acc);
    acc = fmaf(vt_bf16_hi(w.x), xa.y, acc);
    acc = fmaf(vt_bf16_lo(w.y), xa.z, acc);
    acc = fmaf(vt_bf16_hi(w.y), xa.w, acc);
    acc = fmaf(vt_bf16_lo(w.z), xb.x, acc);
    acc = fmaf(vt_bf16_hi(w.z), xb.y, acc);
    acc = fmaf(vt_bf16_lo(w.w), xb.z, acc);
    acc = fmaf(vt_bf16_hi(w.w), xb.w, acc);
    return acc;
}

/* fp32 -> two bf16 planes: hi = bf16(x) (round to nearest even) and
 * lo = bf16(x - hi); x - hi is exact in fp32, so hi + lo carries x to about
 * 2^-17 relative.  Finite inputs only. */
__device__ __forceinline__ unsigned vt_bf16_rne(float x) {
    const unsigned u = __float_as_uint(x);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
/* Two values at a time, packed (first value in the low half): the vector conversion compiles to
 * gfx950's v_cvt_pk_bf16_f32, one instruction per pair where the integer form above takes four
 * per value; the kernels that build planes are bound by exactly these instructions. */
typedef __bf16 vt_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void vt_split_planes2(float a, float b, unsigned &hi, unsigned &lo) {
    const f32x2 v = {a, b};
    hi = __builtin_bit_cast(unsigned, __builtin_convertvector(v, vt_bf16x2));
    const f32x2 r = {__fsub_rn(a, __uint_as_float(hi << 16)), __fsub_rn(b, __uint_as_float(hi & 0xffff0000u))};
    lo = __builtin_bit_cast(unsigned, __builtin_convertvector(r, vt_bf16x2));
}
__device__ __forceinline__ void vt_split_planes4(float a, float b, float c, float d, u32x2 &hi, u32x2 &lo) {
    unsigned h0, l0, h1, l1;
    vt_split_planes2(a, b, h0, l0);
    vt_split_planes2(c, d, h1, l1);
    hi = u32x2{h0, h1};
    lo = u32x2{l0, l1};
}

/* Device-scope coherent accesses for the small vectors that workgroups hand
 * to each other inside one kernel.  Each XCD has its own L2, so such data is
 * written through to memory and read past the L2 (relaxed agent-scope
 * atomics); no cache-wide write-back or invalidate is ever issued. */
__device__ __forceinline__ float vt_ldc(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void vt_stc(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned vt_ldc_u32(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void vt_stc_u32(unsigned *p, unsigned v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* ---- bounded grid barrier over per-workgroup flags -------------------------
 * All workgroups of a persistent kernel are co-resident (the grid is sized to
 * the device, one workgroup per CU).  Workgroup w announces barrier number e
 * by writing e to flags[w]; the first wave of every workgroup polls all flags
 * (one coherent load per lane and 64 flags) until each has reached e.  No
 * read-modify-write is involved, so arrivals do not serialise.  Epochs only
 * grow, across launches too (the host passes the first epoch of a launch).
 * The spin is bounded by a wall-clock budget; on expiry, or when another
 * workgroup has raised `abort_flag`, the barrier returns false and the caller
 * leaves the kernel, so every wave always reaches the end of the grid.
 *
 * Data handed over a barrier must be written with vt_stc and read with
 * vt_ldc: __syncthreads() makes every wave wait for its own stores to be
 * acknowledged before the flag is written. */
struct vt_grid_sync {
    unsigned *flags;                /* [gridDim.x] */
    int *abort_flag;
    unsigned epoch;                 /* epoch of the next barrier */
    unsigned long long timeout;     /* wall_clock64 ticks (100 MHz) */
};

/* The flags exist in VT_FLAG_COPIES copies, VT_FLAG_STRIDE words apart (so in different memory
 * channels); a workgroup writes all copies and polls copy blockIdx % VT_FLAG_COPIES: the polls
 * of 256 workgroups are coherent loads served by the memory side, and spread over the copies
 * they do not queue on one channel. */
#ifndef VT_FLAG_COPIES
#define VT_FLAG_COPIES 4          /* 1 / 2 / 4 / 8 / 16 copies: 1.180 / 1.182 / 1.179 / 1.185 / 1.193 ms per launch (every copy is one more flag store per barrier) */
#endif
#define VT_FLAG_STRIDE 16384
/* Words between the flags of two workgroups: partial writes to one 64-byte line are served one
 * after another by the memory side (about 60 ns each, measured: 256 workgroups writing 16 flags to
 * a line see their stores acknowledged after 0.9 us, one flag to a line after 0.3 us), so the flags
 * are spread out; a poll then touches VT_FLAG_PAD times as many lines. */
#ifndef VT_FLAG_PAD
#define VT_FLAG_PAD 8             /* with 4 copies, 4 / 6 / 8 / 12 / 16 words: 1.1805 / 1.179 / 1.1746 / 1.178 / 1.180 ms per launch */
#endif
#define VT_FLAG_LOADS 4           /* flags a lane polls: grids of up to 256 workgroups */
#define VT_FLAG_ABORT_AT 8192     /* word of a copy that says "a workgroup has given up" (one word read by 256
                                   * workgroups at every poll would be a queue of its own) */
/* Polls in flight per workgroup, and the pause (in units of 64 clocks) in front of a repeated poll.
 * The polls of 256 workgroups are traffic on the memory side themselves: measured on the whole-step
 * kernel, ms/frame with 4 / 3 / 2 / 1 polls in flight: 1.219 / 1.209 / 1.205 / 1.195, and 1.190
 * with one poll and a pause of 2-12 units. */
#ifndef VT_POLL_DEPTH
#define VT_POLL_DEPTH 1
#endif
#ifndef VT_POLL_SLEEP
#define VT_POLL_SLEEP 4
#endif

/* A fence for the compiler only (no instruction): memory accesses written on one side of it are not
 * moved to the other.  The hardware order comes from the wait for the store acknowledgements; this
 * keeps the compiler from placing a hand-over store behind that wait, or a load of handed-over data
 * in front of the poll that releases it. */
__device__ __forceinline__ void vt_compiler_fence() { __atomic_signal_fence(__ATOMIC_SEQ_CST); }

__device__ __forceinline__ void vt_barrier_arrive(vt_grid_sync &gs) {
    vt_compiler_fence();
    __builtin_amdgcn_s_waitcnt(0x0F70);          /* vmcnt(0): this wave's stores are acknowledged */
    vt_compiler_fence();
    __syncthreads();
    if (threadIdx.x < VT_FLAG_COPIES) vt_stc_u32(gs.flags + threadIdx.x * VT_FLAG_STRIDE + blockIdx.x * VT_FLAG_PAD, gs.epoch);
}

/* Wait until the workgroups idx(0) .. idx(nloads - 1) of every lane have announced the current
 * barrier (the first wave polls; a lane with fewer workgroups to watch names one of them again).
 * A hand-over that only some workgroups feed needs only their flags: fewer lines per poll, and
 * nobody waits for a straggler whose results it does not read. */
template <class IDX>
__device__ __forceinline__ bool vt_barrier_wait_on(vt_grid_sync &gs, int *lds_flag, int nloads, IDX idx) {
    if (threadIdx.x < VT_WAVE) {
        const unsigned *mine = gs.flags + (blockIdx.x % VT_FLAG_COPIES) * VT_FLAG_STRIDE;
        const unsigned long long t0 = wall_clock64();
        int ok = 1;
        unsigned f[VT_POLL_DEPTH][VT_FLAG_LOADS];
        int at[VT_FLAG_LOADS];
#pragma unroll
        for (int k = 0; k < VT_FLAG_LOADS; k++) at[k] = idx(k < nloads ? k : 0) * VT_FLAG_PAD;
#pragma unroll
        for (int d = 0; d < VT_POLL_DEPTH; d++)
#pragma unroll
            for (int k = 0; k < VT_FLAG_LOADS; k++) f[d][k] = k < nloads ? vt_ldc_u32(mine + at[k]) : gs.epoch;
        bool released = false;
        while (!released) {
            /* the abort flag travels with the flags: one round trip per poll, not two */
            const int aborted = (int)vt_ldc_u32(mine + VT_FLAG_ABORT_AT);
#pragma unroll
            for (int d = 0; d < VT_POLL_DEPTH; d++) {
                if (!released) {
                    int done = 1;
#pragma unroll
                    for (int k = 0; k < VT_FLAG_LOADS; k++) done &= (int)(f[d][k] - gs.epoch) >= 0;
                    released = __all(done);
                    if (!released) {
                        if (VT_POLL_SLEEP > 0) __builtin_amdgcn_s_sleep(VT_POLL_SLEEP);
#pragma unroll
                        for (int k = 0; k < VT_FLAG_LOADS; k++)
                            if (k < nloads) f[d][k] = vt_ldc_u32(mine + at[k]);
                    }
                }
            }
            if (!released && (aborted != 0 || wall_clock64() - t0 > gs.timeout)) {
                ok = 0;
                break;
            }
        }
        ok = __all(ok);
        if (!ok) {
            /* the host reads abort_flag; the other workgroups read the copy that travels with their flags */
            if (threadIdx.x == 0) __hip_atomic_store(gs.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (threadIdx.x < VT_FLAG_COPIES) vt_stc_u32(gs.flags + threadIdx.x * VT_FLAG_STRIDE + VT_FLAG_ABORT_AT, 1u);
        }
        if (threadIdx.x == 0) *lds_flag = ok;
    }
    __syncthreads();
    vt_compiler_fence();                         /* loads of handed-over data stay behind the release */
    gs.epoch += 1u;
    return *lds_flag != 0;
}

/* every workgroup: a lane reads the flags lane, lane + 64, ... (the last one again where the grid has fewer) */
__device__ __forceinline__ bool vt_barrier_wait(vt_grid_sync &gs, int *lds_flag) {
    const int G = (int)gridDim.x, lane = (int)threadIdx.x & (VT_WAVE - 1);
    return vt_barrier_wait_on(gs, lds_flag, VT_FLAG_LOADS, [&](int k) { return min(lane + VT_WAVE * k, G - 1); });
}

/* the workgroups 0 .. n - 1 */
__device__ __forceinline__ bool vt_barrier_wait_first(vt_grid_sync &gs, int *lds_flag, int n) {
    const int lane = (int)threadIdx.x & (VT_WAVE - 1);
    return vt_barrier_wait_on(gs, lds_flag, (n + VT_WAVE - 1) / VT_WAVE, [&](int k) { return min(lane + VT_WAVE * k, n - 1); });
}

/* A workgroup that reads nothing of what this hand-over passes on: it has announced itself and goes on. */
__device__ __forceinline__ void vt_barrier_pass(vt_grid_sync &gs) { gs.epoch += 1u; }

#endif /* VT_DEVICE_H */
