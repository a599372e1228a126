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
 *   mode 1  one kernel per phase (5 launches per layer), same numerics.
 *   mode 2  the streaming kernel of vt_decode_stream.hip (256-CU devices only):
 *           weight streaming decoupled from synchronisation, 6 stream waves + 1
 *           control wave per CU.  Correct and reproducible, but not yet faster
 *           than mode 0 (its control path pays the CU's shared memory queue on
 *           every hand-over); opt-in.
 */
#include "vt_state.h"

#include <string.h>

/* ---- persistent whole-step kernel -------------------------------------------- */

/* Arrive at the grid barrier, request the next phase's first weight rows while
 * the other workgroups arrive, then wait. */
#ifdef VT_TRACE
/* Build-time instrumentation (never in the shipped library): workgroups 0 and
 * gridDim.x-1 record the 100 MHz wall clock at the points of every phase. */
__device__ unsigned long long vt_trace_buf[2 * 4096];
__device__ __forceinline__ void vt_tr(int &n) {
    if (threadIdx.x == 0 && (blockIdx.x == 0 || blockIdx.x == gridDim.x - 1) && n < 4096)
        vt_trace_buf[(blockIdx.x ? 4096 : 0) + n] = wall_clock64();
    n++;
}
#define VT_TR(n) vt_tr(n)
#else
#define VT_TR(n) ((void)0)
#endif

template <class F>
__device__ __forceinline__ bool vt_barrier_then(vt_grid_sync &gs, int *flag, F between, int &tn) {
    VT_TR(tn);                      /* body done */
    vt_barrier_arrive(gs);
    VT_TR(tn);                      /* arrived */
    between();
    VT_TR(tn);                      /* prefetch requested */
    const bool ok = vt_barrier_wait(gs, flag);
    VT_TR(tn);                      /* released */
    return ok;
}

__global__ void __launch_bounds__(VT_STEP_THREADS)
vt_decode_step_kernel(vt_step_args a, vt_grid_sync gs) {
    __shared__ __attribute__((aligned(16))) float lds[VT_LDS_FLOATS];
    __shared__ int s_flag;
    u32x4 ring[VT_RING];
    int tn = 0;

    if (blockIdx.x == 0)
        for (int t = (int)threadIdx.x; t < a.n_layers * VT_KV_HEADS; t += (int)blockDim.x)
            vt_stc_u32(a.att_cnt + t, 0u);

    const float *x_in = a.in_embed;
    vt_qkv_prefetch(ring, a.layers[0]);
    /* scalars of the whole step: who runs the attention, and whether enough workgroups are left over */
    const int att_busy = __builtin_amdgcn_readfirstlane(vt_attn_busy(a));
    const bool l2_prefetch = 4 * att_busy <= 3 * (int)gridDim.x;
    for (int l = 0; l < a.n_layers; l++) {
        const vt_layer_dev L = a.layers[l];
        /* the next phase's first row is requested as soon as the ring is free, the other rows
         * between arriving at the barrier and waiting on it: together they keep the HBM pipe
         * busy from the end of one phase's arithmetic to the start of the next one's */
        const bool more = l + 1 < a.n_layers;
        vt_qkv_body(ring, L, a, l, x_in, lds, [&] { vt_wo_prefetch(ring, L, VT_PART_HEAD); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_wo_prefetch(ring, L, VT_PART_TAIL); }, tn)) return;
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
            }, tn))
            return;
        vt_wo_body(ring, L, a, x_in, lds, [&] { vt_w13_prefetch(ring, L, VT_PART_HEAD, 0, wo_slots); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_w13_prefetch(ring, L, VT_PART_TAIL, 0, wo_slots); }, tn))
            return;
        vt_w13_body(ring, L, a, lds, [&] { vt_w2_prefetch(ring, L, VT_PART_HEAD); });
        if (!vt_barrier_then(gs, &s_flag, [&] { vt_w2_prefetch(ring, L, VT_PART_TAIL); }, tn)) return;
        vt_w2_body(ring, L, a, lds, [&] { if (more) vt_qkv_prefetch(ring, a.layers[l + 1], VT_PART_HEAD); });
        if (!vt_barrier_then(gs, &s_flag, [&] { if (more) vt_qkv_prefetch(ring, a.layers[l + 1], VT_PART_TAIL); }, tn))
            return;
        x_in = a.x;
    }
    if (blockIdx.x == 0) {
        if (a.final_norm) {
            vt_block_rmsnorm<true>(a.out_hidden, a.x, a.final_norm, VT_DIM, VT_EPS, lds);
        } else {
            for (int i = (int)threadIdx.x; i < VT_DIM; i += (int)blockDim.x) a.out_hidden[i] = vt_ldc(a.x + i);
        }
    }
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
    int per = (2 * VT_FFN + grid - 1) / grid;
    per = (per + 1) / 2 * 2;
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
    if (g_vt.decode_mode == 2) {
        if (!vt_stream_supported()) { vt_set_error("decode step: the streaming schedule needs a 256-CU device"); return -1; }
        return vt_run_step_stream(a);
    } else if (g_vt.decode_mode == 0) {
        vt_grid_sync gs;
        gs.flags = g_vt.d_bar_flags;
        gs.abort_flag = g_vt.d_abort;
        gs.epoch = g_vt.bar_epoch + 1u;
        gs.timeout = g_vt.bar_timeout ? g_vt.bar_timeout : 20000000ull;   /* default 0.2 s of the 100 MHz wall clock */
        g_vt.bar_epoch += 5u * (unsigned)n_layers;
        static int attr_set = 0;
        if (!attr_set && g_vt.step_dyn_lds) {
            if (vt_check(hipFuncSetAttribute((const void *)vt_decode_step_kernel,
                                             hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)g_vt.step_dyn_lds), "hipFuncSetAttribute"))
                g_vt.step_dyn_lds = 0;
            attr_set = 1;
        }
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

/* Reads the abort flag of the persistent kernel after a synchronisation. */
static int step_aborted(int flag) {
    if (!flag) return 0;
    vt_set_error("decode step: grid barrier timed out; kernel left early, result invalid");
    (void)hipMemsetAsync(g_vt.d_abort, 0, sizeof(int), g_vt.stream);
    (void)hipMemsetAsync(g_vt.d_bar_flags, 0, sizeof(unsigned) * VT_FLAG_COPIES * VT_FLAG_STRIDE, g_vt.stream);
    (void)hipStreamSynchronize(g_vt.stream);
    g_vt.bar_epoch = 0;
    return -1;
}

#ifdef VT_TRACE
extern "C" void tts_hip_trace_read(unsigned long long *out) {
    (void)hipDeviceSynchronize();
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(vt_trace_buf), sizeof(unsigned long long) * 2 * 4096);
}
#endif

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
    if (step_aborted(flag)) return;
    memcpy(out_hidden, pin_out, sizeof(float) * VT_DIM);
}

extern "C" void tts_hip_layer_decode(int layer, float *d_hidden, int pos) {
    if (!g_vt.initialized) { vt_set_error("tts_hip_layer_decode: backend not initialised"); return; }
    if (layer < 0 || layer >= g_vt.n_dec_layers) {
        vt_set_error("tts_hip_layer_decode: layer %d not uploaded", layer);
        return;
    }
    /* the step reads its input while it writes the output only at the very end,
     * from workgroup 0, after the last barrier: in-place is safe */
    (void)vt_run_step(g_vt.d_layers + layer, 1, layer, NULL, d_hidden, d_hidden, pos);
}
