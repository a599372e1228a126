/*
 * vt_device.h - device-side building blocks shared by the gfx950 kernels:
 * wave64 reductions over DPP, bf16 widening, streaming 16-byte weight loads
 * and the bounded grid barrier used by the persistent kernels.
 */
#ifndef VT_DEVICE_H
#define VT_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define VT_WAVE 64

/* Model dimensions of the backbone / acoustic transformer layer. */
#define VT_DIM      3072
#define VT_HEADS    32
#define VT_KV_HEADS 8
#define VT_HEAD_DIM 128
#define VT_Q_DIM    4096
#define VT_KV_DIM   1024
#define VT_QKV_DIM  6144
#define VT_FFN      9216
#define VT_EPS      1e-5f

__device__ __forceinline__ int vt_lane() { return (int)(threadIdx.x & (VT_WAVE - 1)); }
__device__ __forceinline__ int vt_wave() { return (int)(threadIdx.x >> 6); }

/* bf16 pair packed in a dword: element 0 in the low half. Widening is exact. */
__device__ __forceinline__ float vt_bf16_lo(unsigned int w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float vt_bf16_hi(unsigned int w) { return __uint_as_float(w & 0xffff0000u); }

/* 16-byte streaming load of 8 bf16 weights: weights are read once per step,
 * so they are marked non-temporal to keep the small activation vectors and
 * the KV cache resident in L2. */
__device__ __forceinline__ u32x4 vt_ldw(const uint16_t *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
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

/* Coherent (device-scope) scalar accesses for data exchanged between
 * workgroups inside one kernel. */
__device__ __forceinline__ float vt_ld_coherent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* ---- bounded grid barrier -------------------------------------------------
 * All workgroups of a persistent kernel are co-resident (the launch is
 * cooperative and sized to the device).  `counter` only grows: barrier number
 * b of a launch is passed once the counter reaches base + (b+1)*gridDim.x.
 * The spin is bounded by a wall-clock budget; on expiry (or when another
 * workgroup has raised `abort_flag`) the barrier returns false and the caller
 * leaves the kernel, so every wave always reaches the end of the grid. */
struct vt_grid_sync {
    unsigned long long *counter;
    int *abort_flag;
    unsigned long long target;      /* value that releases the next barrier */
    unsigned long long timeout;     /* wall_clock64 ticks (100 MHz) */
};

__device__ __forceinline__ bool vt_grid_barrier(vt_grid_sync &gs, int *lds_flag) {
    __syncthreads();
    if (threadIdx.x == 0) {
        int ok = 1;
        __threadfence();                                   /* release this workgroup's stores */
        __hip_atomic_fetch_add(gs.counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned long long t0 = wall_clock64();
        while (__hip_atomic_load(gs.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gs.target) {
            __builtin_amdgcn_s_sleep(2);
            if (__hip_atomic_load(gs.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
                wall_clock64() - t0 > gs.timeout) {
                __hip_atomic_store(gs.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
        }
        __threadfence();                                   /* acquire the other workgroups' stores */
        *lds_flag = ok;
    }
    __syncthreads();
    gs.target += gridDim.x;
    return *lds_flag != 0;
}

#endif /* VT_DEVICE_H */
