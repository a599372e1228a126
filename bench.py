#!/usr/bin/env python3
"""Benchmark of the backbone decode hot path on one MI355X.

Workload (BASELINE.json config "Full 26-layer backbone autoregressive decode"):
26 layers of seeded random-init bf16 weights (~N(0,0.02)), a 64-token prompt of
random ids < 131072 (rows of a lazily evaluated random embedding table),
prefill on the GPU, then decode steps that feed each output hidden back through
a random 3072x3072 bf16 projection.  A "step" is one such decode step (one
audio frame's backbone forward).  Everything is resident in HBM when the timed
region starts; the timed region is bracketed by events on the library's stream.

Prints ONE JSON line: ms/frame as `value`, the roofline of the dominant kernel
(the persistent whole-step kernel, algorithmic bytes / its own average launch
duration) and the reference CPU path timed on this host's cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

import hipsupport as H  # noqa: E402
import vtsupport as S  # noqa: E402

HBM_PEAK_GBPS = 8000.0
N_LAYERS = 26
PROMPT = 64
LAYER_WEIGHT_BYTES = 2 * (S.Q_DIM * S.DIM + 2 * S.KV_DIM * S.DIM + S.DIM * S.Q_DIM + 3 * S.FFN * S.DIM)


def step_bytes(pos):
    """Algorithmic HBM bytes of one 26-layer decode step at cache position pos:
    every bf16 weight once, the norm gains, the K and V rows 0..pos of every
    layer once (f32, 1024 wide), the appended rows, input and output vectors."""
    w = N_LAYERS * LAYER_WEIGHT_BYTES
    norms = (2 * N_LAYERS + 1) * S.DIM * 4
    kv_read = N_LAYERS * 2 * (pos + 1) * S.KV_DIM * 4
    kv_write = N_LAYERS * 2 * S.KV_DIM * 4
    io = 2 * S.DIM * 4
    return w + norms + kv_read + kv_write + io


def emb_row(token_id):
    """Row `token_id` of the synthetic [131072, 3072] bf16 embedding table."""
    return S.bf16_to_f32(S.bf16_normal(S.DIM, 7_000_000 + int(token_id), 1.0))


def make_layers(n, workers):
    with ThreadPoolExecutor(workers) as ex:
        return list(ex.map(lambda i: S.Layer(1000 + i), range(n)))


def cpu_baseline(layers, final_norm, kv_k, kv_v, kv_max, embeds, gpu_hidden, budget_s):
    """Times the reference CPU decode step (single thread: the reference has no
    threads and its decode matvec never reaches BLAS) on the same weights, from
    the same cache state, for as many steps as fit the budget.  Uses the compiled
    reference (oracle/_ref) when it travelled with the tree, else our port."""
    import cases
    n_cached = PROMPT
    if S.have_ref():
        kind = "reference"
        b = cases.RefBackend()
        b.llm_open(layers, final_norm, kv_max)
        nbytes = N_LAYERS * kv_max * S.KV_DIM * 4
        C.memmove(b.lib.ref_kv_k(b.ctx), kv_k.ctypes.data, nbytes)
        C.memmove(b.lib.ref_kv_v(b.ctx), kv_v.ctypes.data, nbytes)
        b.lib.ref_set_kv_len(b.ctx, n_cached)
    else:
        kind = "port"
        b = cases.OracleBackend(threads=1)
        b.llm_open(layers, final_norm, kv_max, n_layers=N_LAYERS)
        b.kv_k[:] = kv_k
        b.kv_v[:] = kv_v
        b.pos = n_cached
    times, errs = [], []
    t_start = time.time()
    for i in range(len(embeds)):
        t0 = time.time()
        h = b.llm_forward(embeds[i])
        times.append(time.time() - t0)
        errs.append(S.rel_errors(h, gpu_hidden[i]))
        if time.time() - t_start + times[-1] > budget_s:
            break
    b.llm_close()
    ms = 1000.0 * float(np.mean(times))
    return {
        "value": round(ms, 1), "unit": "ms/frame", "cores": 1, "kind": kind,
        "sample": f"{len(times)} decode steps (pos {n_cached}..{n_cached + len(times) - 1}) of the same "
                  f"26-layer weights, KV prefix copied from the GPU prefill, teacher-forced inputs",
        "gbps": round(step_bytes(n_cached) / (ms * 1e-3) / 1e9, 2),
    }, {"max_abs_over_rms": max(e[0] for e in errs), "rel_l2": max(e[1] for e in errs),
        "steps_checked": len(errs), "against": kind}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--mode", type=int, default=0, help="0 persistent kernel, 1 per-phase kernels, 2 streaming kernel")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain elementwise kernel (vt_add_kernel, a += b over 64 Mi floats: "
                         "512 MiB read, 256 MiB written) so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "can be scaled by a kernel of known traffic")
    ap.add_argument("--traffic-kib", type=float, default=None,
                    help="HBM bytes per launch measured with rocprofv3 --pmc (KiB), if known")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus above 1 is not supported "
                 "(the decode chain is not sharded; see DESIGN.md)")
    K, W = args.steps, args.warmup
    workers = min(16, os.cpu_count() or 8)

    t0 = time.time()
    layers = make_layers(N_LAYERS, workers)
    final_norm = S.norm_weight(S.DIM, 99)
    proj = S.bf16_normal((S.DIM, S.DIM), 31337)
    ids = np.random.default_rng(7).integers(0, 131072, PROMPT)
    prompt = np.stack([emb_row(t) for t in ids]).astype(np.float32)
    t_gen = time.time() - t0

    n_cpu = 6 if args.cpu_seconds > 0 else 0
    kv_max = PROMPT + n_cpu + 2 * (W + K) + 8
    hip = H.Hip(kv_max=kv_max)
    lib = hip.lib
    lib.tts_hip_set_decode_mode(args.mode)
    t0 = time.time()
    hip.upload_decoder(layers, final_norm, N_LAYERS)
    d_proj = H.DevBuf.from_numpy(lib, proj)
    t_up = time.time() - t0

    if args.calibrate:
        n_cal = 64 << 20
        ca, cb = H.DevBuf(lib, 4 * n_cal), H.DevBuf(lib, 4 * n_cal)
        lib.tts_hip_memset(ca.ptr, 0, 4 * n_cal)
        lib.tts_hip_memset(cb.ptr, 0, 4 * n_cal)
        lib.tts_hip_add_inplace(ca.ptr, cb.ptr, n_cal)
        lib.tts_hip_sync()
        ca.free()
        cb.free()

    # prefill the prompt on the GPU; the first decode input is the last residual row
    # pushed through the feedback projection (any O(1) vector would do)
    x_last = hip.llm_prefill(prompt, want_x=True)[-1]
    d_e = H.DevBuf.from_numpy(lib, x_last / np.sqrt(np.mean(x_last ** 2)))
    d_h = H.DevBuf(lib, S.DIM * 4)
    pos = PROMPT

    # a few recorded steps for the CPU leg / parity (inputs and outputs kept)
    rec_e, rec_h = [], []
    kv_k = kv_v = None
    if n_cpu:
        kv_k, kv_v = hip.kv()
        for _ in range(n_cpu):
            rec_e.append(d_e.to_numpy(np.float32, S.DIM))
            lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, pos)
            lib.tts_hip_linear_bf16(d_e.ptr, d_h.ptr, None, 1, S.DIM, S.DIM, d_proj.ptr)
            lib.tts_hip_sync()
            rec_h.append(d_h.to_numpy(np.float32, S.DIM))
            pos += 1
    hip.check()

    def run(n, with_proj):
        nonlocal pos
        for _ in range(n):
            lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, pos)
            if with_proj:
                lib.tts_hip_linear_bf16(d_e.ptr, d_h.ptr, None, 1, S.DIM, S.DIM, d_proj.ptr)
            pos += 1

    # headline: W warm-up steps, then exactly K timed steps (decode + feedback projection)
    run(W, True)
    lib.tts_hip_sync()
    pos0 = pos
    lib.tts_hip_timer_start()
    run(K, True)
    ms_total = lib.tts_hip_timer_stop_ms()
    lib.tts_hip_sync()
    hip.check()
    ms_step = ms_total / K
    h_final = d_h.to_numpy(np.float32, S.DIM)
    assert np.all(np.isfinite(h_final)), "non-finite hidden state"

    # dominant kernel alone: K launches of the whole-step kernel over the same positions
    pos = pos0
    run(min(W, 5), False)
    pos = pos0
    lib.tts_hip_sync()
    lib.tts_hip_timer_start()
    run(K, False)
    ms_kernel = lib.tts_hip_timer_stop_ms() / K
    lib.tts_hip_sync()
    hip.check()

    avg_pos = pos0 + (K - 1) / 2.0
    bytes_launch = step_bytes(avg_pos)
    achieved = bytes_launch / (ms_kernel * 1e-3) / 1e9
    traffic = None if args.traffic_kib is None else args.traffic_kib * 1024.0
    out = {
        "metric": "backbone decode ms/frame",
        "value": round(ms_step, 4),
        "unit": "ms/frame",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "26-layer backbone autoregressive decode, batch 1, 64-token prompt, "
                        "hidden fed back through a 3072x3072 bf16 projection (BASELINE.json configs[2])",
            "layers": N_LAYERS, "prompt": PROMPT, "positions": [pos0, pos0 + K - 1],
            "weights": "bf16 N(0,0.02) seeded, truncated", "activations": "f32",
            "schedule": ("persistent whole-step kernel", "one kernel per phase", "streaming whole-step kernel")[args.mode],
        },
        "frames_per_s": round(1000.0 / ms_step, 1),
        "hbm_gbps": round((bytes_launch + 2 * S.DIM * S.DIM) / (ms_step * 1e-3) / 1e9, 1),
        "hbm_frac_of_peak": round((bytes_launch + 2 * S.DIM * S.DIM) / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "ms_per_frame_normalised_6p8GB": round(ms_kernel * 6.8e9 / bytes_launch, 4),
        "roofline": {
            "kernel": ("vt_decode_step_kernel", "5 phase kernels per layer", "vt_decode_stream_kernel")[args.mode],
            "bound": "hbm",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "bytes_per_launch": int(bytes_launch),
            "ms_per_launch": round(ms_kernel, 4),
        },
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
    }
    if n_cpu:
        base, parity = cpu_baseline(layers, final_norm, kv_k, kv_v, kv_max, rec_e, rec_h, args.cpu_seconds)
        out["cpu_baseline"] = base
        out["parity"] = {k: (float(f"{v:.3e}") if isinstance(v, float) else v) for k, v in parity.items()}
        assert parity["max_abs_over_rms"] < 1e-3 and parity["rel_l2"] < 1e-3, parity
    else:
        out["cpu_baseline"] = None
    hip.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
