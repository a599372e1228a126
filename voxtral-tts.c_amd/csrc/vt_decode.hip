/*
 * vt_decode.hip - batch-1 backbone decode step (replaces tts_cuda_llm_forward,
 * voxtral_tts_cuda.cu:710-797, whose schedule is ~24 launches per layer with a
 * bf16->f32 conversion of every weight matrix before each cublasSgemm).
 *
 * Two schedules over the same phase code (vt_decode_phases.h):
 *   mode 0  one persistent kernel for the whole step: 5 phases per layer
 *           separated by grid barriers; the weight rows of the next phase are
 *           requested between arriving at a barrier and waiting on it, so the
 *           HBM stream does not stop while the tiny activation vectors are
 *           exchanged between workgroups.
 *   mode 1  one kernel per phase (5 launches per layer), same numerics; also the
 *           schedule a device falls to when the whole grid of mode 0 cannot be
 *           resident at once.
 *
 * A barrier of mode 0 that runs out of its spin budget raises a flag on the device
 * and every workgroup leaves the kernel.  The host learns of it at its next
 * synchronising call (vt_step_poll_abort): the failed step is counted as an error,
 * the flag and the barrier epochs are reset, and the next launch starts clean.
 */
#include "vt_state.h"

#include <stdlib.h>
#include <string.h>

/* ---- persistent whole-step kernel -------------------------------------------- */

/* Arrive at the grid barrier, request the next phase's first weight rows while
 * the other workgroups arrive, then wait. */
template <class F, class W>
__device__ __forceinline__ bool vt_barrier_then(vt_grid_sync &gs, int *flag, F between, W wait) {
    vt_barrier_arrive(gs);
    between();
    return wait();
}

template <class F>
__device__ __forceinline__ bool vt_barrier_then(vt_grid_sync &gs, int *flag, F between) {
    return vt_barrier_then(gs, flag, between, [&] { return vt_barrier_wait(gs, flag); });
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_decode_step_kernel(vt_step_args a, vt_grid_sync gs) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    __shared__ int s_flag;
    u32x4 ring[VT_RING];

    if (blockIdx.x == 0)
        for (int t = (int)threadIdx.x; t < a.n_layers * VT_KV_HEADS; t += (int)blockDim.x)
            vt_stc_u32(a.att_cnt + t, 0u);

    const float *x_in = a.in_embed;
    vt_qkv_prefetch(ring, a.layers[0]);
    /* scalars of the whole step: who runs the attention, and whether enough workgroups are left over */
    const int att_busy = __builtin_amdgcn_readfirstlane(vt_attn_busy(a));
    const bool l2_prefetch = 4 * att_busy <= 3 * (int)gridDim.x;
    /* The two hand-overs around the attention are narrow.  Into it: a workgroup of the direct schedule
     * reads the q rows of one head and the new K and V rows of one kv head, which some 20 workgroups
     * wrote, and the workgroups without a share of the attention read nothing.  Out of it: everybody
     * reads what the att_busy attention workgroups wrote.  Those have, between them, waited for every
     * workgroup that owns q|k|v rows, so behind the second hand-over nobody still reads the residual
     * stream that the output projection is about to overwrite. */
    const bool att_direct = vt_attn_is_direct(a);
    auto wait_qkv = [&]() -> bool {
        if (!att_direct) return vt_barrier_wait(gs, &s_flag);
        if ((int)blockIdx.x >= att_busy) { vt_barrier_pass(gs); return true; }
        const int lane = (int)threadIdx.x & (VT_WAVE - 1);
        return vt_barrier_wait_on(gs, &s_flag, 1, [&](int) { return vt_attn_producer((int)blockIdx.x, lane); });
    };
    auto wait_attn = [&]() -> bool { return vt_barrier_wait_first(gs, &s_flag, att_busy); };
    for (int l = 0; l < a.n_layers; l++) {
        const vt_layer_dev L = a.layers[l];
        /* the next phase's first row is requested as soon as the ring is free, the other rows
         * between arriving at the barrier and waiting on it: together they keep the HBM pipe
         * busy from the end of one phase's arithmetic to the start of the next one's */
        const bool more = l + 1 < a.n_layers;
        vt_qkv_body(ring, L, a, l, x_in, lds, [&] { vt_wo_prefetch(ring, L, VT_PART_HEAD); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_wo_prefetch(ring, L, VT_PART_TAIL); }, wait_qkv)) return;
        vt_attn_phase(a, l, lds);
        /* with 3 rows per wave the output projection leaves the ring slots from VT_WO_SLOTS on
         * free: the gate|up rows that go there are requested a phase early */
        const int wo_slots = vt_wo_rows().nr * 4 <= VT_WO_SLOTS ? VT_WO_SLOTS : VT_RING;
        if (!vt_barrier_then(gs, &s_flag, [&] {
                vt_w13_prefetch(ring, L, VT_PART_ALL, wo_slots, VT_RING);
                /* the workgroups without a share of the attention prefetch into their L2: gate|up rows
                 * when at least a quarter of the grid is free, the next layer's K/V rows while the
                 * cache is short enough to leave room for them */
                if (l2_prefetch) {
                    vt_w13_l2_prefetch(L, att_busy);
                    if (more && vt_attn_is_direct(a)) vt_kv_l2_prefetch(a, l + 1, att_busy);
                }
            }, wait_attn))
            return;
        vt_wo_body(ring, L, a, x_in, lds, [&] { vt_w13_prefetch(ring, L, VT_PART_HEAD, 0, wo_slots); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_w13_prefetch(ring, L, VT_PART_TAIL, 0, wo_slots); }))
            return;
        vt_w13_body(ring, L, a, lds, [&] { vt_w2_prefetch(ring, L, VT_PART_HEAD); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_w2_prefetch(ring, L, VT_PART_TAIL); })) return;
        /* without a final norm the last layer's rows are the output: every workgroup writes its own and the
         * kernel ends without a last hand-over (in place is fine: the input was last read two phases ago) */
        const bool last_direct = !more && !a.final_norm;
        vt_w2_body(ring, L, a, lds, [&] { if (more) vt_qkv_prefetch(ring, a.layers[l + 1], VT_PART_HEAD); }, last_direct);
        if (last_direct) return;
        if (!vt_barrier_then(gs, &s_flag, [&] { if (more) vt_qkv_prefetch(ring, a.layers[l + 1], VT_PART_TAIL); }))
            return;
        x_in = a.x;
    }
    if (blockIdx.x == 0) vt_block_rmsnorm<true>(a.out_hidden, a.x, a.final_norm, VT_DIM, VT_EPS, lds);
}

/* ---- one kernel per phase ------------------------------------------------------ */

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_qkv_kernel(vt_step_args a, int l, const float *x_in) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    u32x4 ring[VT_RING];
    const vt_layer_dev L = a.layers[l];
    vt_qkv_prefetch(ring, L);
    vt_qkv_body(ring, L, a, l, x_in, lds);
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_attn_kernel(vt_step_args a, int l) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    vt_attn_phase(a, l, lds);
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_wo_kernel(vt_step_args a, int l, const float *x_in) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    u32x4 ring[VT_RING];
    const vt_layer_dev L = a.layers[l];
    vt_wo_prefetch(ring, L);
    vt_wo_body(ring, L, a, x_in, lds);
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_w13_kernel(vt_step_args a, int l) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    u32x4 ring[VT_RING];
    const vt_layer_dev L = a.layers[l];
    vt_w13_prefetch(ring, L);
    vt_w13_body(ring, L, a, lds);
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_w2_kernel(vt_step_args a, int l) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    u32x4 ring[VT_RING];
    const vt_layer_dev L = a.layers[l];
    vt_w2_prefetch(ring, L);
    vt_w2_body(ring, L, a, lds);
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_final_kernel(vt_step_args a) {
    __shared__ float lds[VT_MAX_WAVES];
    if (a.final_norm) {
        vt_block_rmsnorm<false>(a.out_hidden, a.x, a.final_norm, VT_DIM, VT_EPS, lds);
    } else {
        for (int i = (int)threadIdx.x; i < VT_DIM; i += (int)blockDim.x) a.out_hidden[i] = a.x[i];
    }
}

/* ---- host side ------------------------------------------------------------------- */

/* Rows per workgroup of every phase must fit the 256-float LDS row buffer, and a lane of the
 * barrier polls VT_FLAG_LOADS flags. */
static int grid_fits(int grid) {
    const int per = vt_rows_per_wg(2 * VT_FFN, 2, grid);
    return per <= 256 && grid % VT_KV_HEADS == 0 && grid >= VT_KV_HEADS && grid <= VT_WAVE * VT_FLAG_LOADS;
}

int vt_run_step(const vt_layer_dev *d_layers, int n_layers, int first_layer,
                const float *d_final_norm, const float *d_in, float *d_out, int pos) {
    if (!g_vt.initialized) { vt_set_error("decode step: backend not initialised"); return -1; }
    if (n_layers < 1 || first_layer < 0 || first_layer + n_layers > TTS_HIP_DEC_LAYERS) {
        vt_set_error("decode step: bad layer range [%d, %d)", first_layer, first_layer + n_layers);
        return -1;
    }
    if (pos < 0 || pos >= g_vt.kv_max) {
        vt_set_error("decode step: position %d outside the KV cache (max %d)", pos, g_vt.kv_max);
        return -1;
    }
    if (!grid_fits(g_vt.grid)) { vt_set_error("decode step: grid %d unsupported", g_vt.grid); return -1; }

    vt_step_args a;
    a.layers = d_layers;
    a.n_layers = n_layers;
    a.first_layer = first_layer;
    a.final_norm = d_final_norm;
    a.kv_k = g_hip.kv_cache_k_gpu;
    a.kv_v = g_hip.kv_cache_v_gpu;
    a.kv_max = g_vt.kv_max;
    a.pos = pos;
    a.rope = g_vt.d_rope;
    a.in_embed = d_in;
    a.out_hidden = d_out;
    a.x = g_vt.d_x;
    a.q = g_vt.d_q;
    a.attn = g_vt.d_attn;
    a.h = g_vt.d_h;
    a.att_part = g_vt.d_att_part;
    a.att_cnt = g_vt.d_att_cnt;

    const dim3 grid(g_vt.grid), block(VT_STEP_THREADS);
    hipStream_t st = g_vt.stream;
    if (g_vt.decode_mode != 0 && g_vt.decode_mode != 1) {
        vt_set_error("decode step: unknown schedule %d (0 = whole-step kernel, 1 = one kernel per phase)",
                     g_vt.decode_mode);
        return -1;
    }
    if (g_vt.decode_mode == 0 && vt_step_resident()) {
        vt_grid_sync gs;
        gs.flags = g_vt.d_bar_flags;
        gs.abort_flag = g_vt.d_abort;
        gs.epoch = g_vt.bar_epoch + 1u;
        gs.timeout = g_vt.bar_timeout ? g_vt.bar_timeout : 20000000ull;   /* default 0.2 s of the 100 MHz wall clock */
        g_vt.bar_epoch += 5u * (unsigned)n_layers;
        g_vt.step_pending = 1;
        hipLaunchKernelGGL(vt_decode_step_kernel, grid, block, g_vt.step_dyn_lds, st, a, gs);
    } else {
        if (vt_check(hipMemsetAsync(g_vt.d_att_cnt, 0, sizeof(unsigned) * n_layers * VT_KV_HEADS, st),
                     "att_cnt clear")) return -1;
        const float *x_in = d_in;
        for (int l = 0; l < n_layers; l++) {
            hipLaunchKernelGGL(vt_qkv_kernel, grid, block, 0, st, a, l, x_in);
            hipLaunchKernelGGL(vt_attn_kernel, grid, block, 0, st, a, l);
            hipLaunchKernelGGL(vt_wo_kernel, grid, block, 0, st, a, l, x_in);
            hipLaunchKernelGGL(vt_w13_kernel, grid, block, 0, st, a, l);
            hipLaunchKernelGGL(vt_w2_kernel, grid, block, 0, st, a, l);
            x_in = g_vt.d_x;
        }
        hipLaunchKernelGGL(vt_final_kernel, dim3(1), block, 0, st, a);
    }
    return vt_check(hipGetLastError(), "decode step launch");
}

/* Whether every workgroup of the whole-step kernel can be resident at once, which its grid
 * barrier needs: asked of the runtime once per context, for the kernel as built (registers, static
 * LDS) with the dynamic LDS it is launched with.  The dynamic LDS is sized from the kernel's real
 * static LDS so that static + dynamic exceeds half a CU's LDS, i.e. so that a CU never takes a
 * second workgroup of this kernel whatever its register count; where a workgroup may not ask for
 * that much the pin is left out (the registers of 8 waves of this kernel fill more than half a
 * CU's file, which has the same effect).  Not resident: the step runs as one kernel per phase. */
int vt_step_resident(void) {
    if (g_vt.step_checked) return g_vt.step_fits;
    g_vt.step_checked = 1;
    g_vt.step_fits = 0;
    hipFuncAttributes fa;
    if (vt_check(hipFuncGetAttributes(&fa, (const void *)vt_decode_step_kernel), "hipFuncGetAttributes")) return 0;
    hipDeviceProp_t prop;
    if (vt_check(hipGetDeviceProperties(&prop, g_vt.device), "hipGetDeviceProperties")) return 0;
    const size_t lds_cu = prop.maxSharedMemoryPerMultiProcessor;
    size_t dyn = 0;
    if (fa.sharedSizeBytes <= lds_cu / 2) {
        dyn = lds_cu / 2 + 1024 - fa.sharedSizeBytes;
        dyn = (dyn + 1023) / 1024 * 1024;
        if (fa.sharedSizeBytes + dyn > (size_t)prop.sharedMemPerBlockOptin && fa.sharedSizeBytes + dyn > prop.sharedMemPerBlock) dyn = 0;
        if (dyn && hipFuncSetAttribute((const void *)vt_decode_step_kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn) != hipSuccess) {
            (void)hipGetLastError();
            dyn = 0;
        }
    }
    int per_cu = 0;
    if (vt_check(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, vt_decode_step_kernel, VT_STEP_THREADS, dyn),
                 "hipOccupancyMaxActiveBlocksPerMultiprocessor")) return 0;
    if (per_cu < 1 && dyn) {            /* the pin itself does not fit: without it */
        dyn = 0;
        if (vt_check(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, vt_decode_step_kernel, VT_STEP_THREADS, dyn),
                     "hipOccupancyMaxActiveBlocksPerMultiprocessor")) return 0;
    }
    g_vt.step_dyn_lds = dyn;
    g_vt.step_fits = (long long)per_cu * g_vt.n_cu >= g_vt.grid;
    if (getenv("TTS_HIP_VERBOSE"))
        fprintf(stderr, "  HIP: whole-step kernel: %d VGPRs, %zu B static + %zu B dynamic LDS, %d workgroup(s) per CU, grid %d %s\n",
                fa.numRegs, (size_t)fa.sharedSizeBytes, dyn, per_cu, g_vt.grid,
                g_vt.step_fits ? "resident" : "NOT resident: one kernel per phase instead");
    if (!g_vt.step_fits)
        fprintf(stderr, "tts_hip: the whole-step decode kernel cannot be resident on this device "
                        "(%d workgroups per CU x %d CUs < grid %d): running one kernel per phase\n",
                per_cu, g_vt.n_cu, g_vt.grid);
    return g_vt.step_fits;
}

/* After a timed-out barrier: count the failure, clear the flag and the epochs. */
static int step_aborted(int flag) {
    if (!flag) return 0;
    vt_set_error("decode step: grid barrier timed out; kernel left early, result invalid");
    (void)hipMemsetAsync(g_vt.d_abort, 0, sizeof(int), g_vt.stream);
    (void)hipMemsetAsync(g_vt.d_bar_flags, 0, sizeof(unsigned) * VT_FLAG_COPIES * VT_FLAG_STRIDE, g_vt.stream);
    (void)hipStreamSynchronize(g_vt.stream);
    g_vt.bar_epoch = 0;
    return -1;
}

/* Workgroups of the whole-step kernel: 0 = the default (the CU count rounded down to a multiple of the
 * KV heads), else a multiple of 8 between 72 and that default.  The barrier's flags start from zero
 * again, so workgroups that sat out a few steps do not come back with an old epoch. */
extern "C" void tts_hip_set_decode_grid(int workgroups) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_set_decode_grid: backend not initialised"); return; }
    const int full = g_vt.n_cu / VT_KV_HEADS * VT_KV_HEADS;
    const int grid = workgroups == 0 ? full : workgroups;
    if (grid > full || !grid_fits(grid)) {
        vt_set_error("tts_hip_set_decode_grid: %d workgroups (0, or a multiple of %d in 72..%d)", workgroups,
                     VT_KV_HEADS, full);
        return;
    }
    if (vt_check(hipStreamSynchronize(g_vt.stream), "decode grid: sync")) return;
    (void)vt_step_poll_abort();
    if (vt_check(hipMemset(g_vt.d_bar_flags, 0, sizeof(unsigned) * VT_FLAG_COPIES * VT_FLAG_STRIDE), "decode grid: flags")) return;
    g_vt.bar_epoch = 0;
    g_vt.grid = grid;
}

/* Called by every entry point right after it has synchronised with the library's stream: if a
 * whole-step kernel ran since the last look, reads its abort flag (a 4-byte copy) and reports a
 * timed-out barrier like any other failed call.  Returns -1 if a step had been abandoned. */
int vt_step_poll_abort(void) {
    if (!g_vt.initialized || !g_vt.step_pending) return 0;
    g_vt.step_pending = 0;
    int flag = 0;
    if (vt_check(hipMemcpy(&flag, g_vt.d_abort, sizeof flag, hipMemcpyDeviceToHost), "abort flag read")) return -1;
    return step_aborted(flag);
}

/* The same for a caller that has already read the abort flag and found it set. */
int vt_step_poll_abort_now(void) { return step_aborted(1); }

extern "C" void tts_hip_llm_forward_device(float *d_out_hidden, const float *d_input_embed, int pos) {
    if (g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_llm_forward: no weights uploaded"); return; }
    (void)vt_run_step(g_vt.d_layers, g_vt.n_dec_layers, 0, g_vt.d_dec_norm, d_input_embed,
                      d_out_hidden, pos);
}

extern "C" void tts_hip_llm_forward(float *out_hidden, const float *input_embed, int pos) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_llm_forward: backend not initialised"); return; }
    if (g_vt.n_dec_layers < 1) { vt_set_error("tts_hip_llm_forward: no weights uploaded"); return; }
    hipStream_t st = g_vt.stream;
    float *pin_in = g_vt.h_pin, *pin_out = g_vt.h_pin + VT_DIM;
    memcpy(pin_in, input_embed, sizeof(float) * VT_DIM);
    VT_TRYV(hipMemcpyAsync(g_vt.d_embed, pin_in, sizeof(float) * VT_DIM, hipMemcpyHostToDevice, st));
    if (vt_run_step(g_vt.d_layers, g_vt.n_dec_layers, 0, g_vt.d_dec_norm, g_vt.d_embed,
                    g_vt.d_hidden, pos)) return;
    VT_TRYV(hipMemcpyAsync(pin_out, g_vt.d_hidden, sizeof(float) * VT_DIM, hipMemcpyDeviceToHost, st));
    VT_TRYV(hipMemcpyAsync(pin_out + VT_DIM, g_vt.d_abort, sizeof(int), hipMemcpyDeviceToHost, st));
    VT_TRYV(hipStreamSynchronize(st));
    int flag;
    memcpy(&flag, pin_out + VT_DIM, sizeof flag);
    g_vt.step_pending = 0;
    if (step_aborted(flag)) return;
    memcpy(out_hidden, pin_out, sizeof(float) * VT_DIM);
}

extern "C" void tts_hip_layer_decode(int layer, float *d_hidden, int pos) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_layer_decode: backend not initialised"); return; }
    if (layer < 0 || layer >= g_vt.n_dec_layers) {
        vt_set_error("tts_hip_layer_decode: layer %d not uploaded", layer);
        return;
    }
    /* in place is safe: without a final norm every workgroup writes its own rows of the output in the
     * down projection's epilogue, and the input was last read two phases earlier (by the output
     * projection's residual add), behind two grid-wide hand-overs */
    (void)vt_run_step(g_vt.d_layers + layer, 1, layer, NULL, d_hidden, d_hidden, pos);
}
