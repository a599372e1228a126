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


def _package():
    """The package directory (its name is not a Python identifier): the ctypes mirror of the C ABI,
    the seeded synthetic weights and the device session."""
    import importlib.util
    name = "voxtral_tts_c_amd"
    if name not in sys.modules:
        pkg_dir = os.path.join(ROOT, "voxtral-tts.c_amd")
        spec = importlib.util.spec_from_file_location(name, os.path.join(pkg_dir, "__init__.py"),
                                                      submodule_search_locations=[pkg_dir])
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
    return sys.modules[name]


PKG = _package()
from voxtral_tts_c_amd import session as H  # noqa: E402
from voxtral_tts_c_amd import synth as S  # noqa: E402


class _Checkers:
    """The CPU checkers: ctypes bindings of oracle/liboracle.so and oracle/_ref/libvoxtral_ref.so and the
    backends over them, which live with the tests.  Only the cpu_baseline and parity legs below (and the
    set-up of --workload codec, whose weight-norm reconstruction is the checker's) load them; nothing that
    is timed on the GPU does."""
    _mods = None

    def __getattr__(self, name):
        if _Checkers._mods is None:
            for d in (os.path.join(ROOT, "tests"), os.path.join(ROOT, "tests", "golden")):
                if d not in sys.path:
                    sys.path.insert(0, d)
            import cases
            import codec_cases
            import codecsupport
            import vtsupport
            _Checkers._mods = {"cases": cases, "codec_cases": codec_cases, "codecsupport": codecsupport, "vt": vtsupport}
        return _Checkers._mods[name]


CHK = _Checkers()


def BL():
    """The benchmark companion library (event timing and single-kernel loops on the library's stream)."""
    return PKG.bench_lib()

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


def measured_traffic(workload):
    """HBM bytes per launch (or per layer) of the dominant kernel as measured with rocprofv3
    --pmc and recorded under profiles/; None when no measurement is on file."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            e = json.load(f)[workload]
        return 1024.0 * (e["fetch_kib"] * e["fetch_factor"] + e["write_kib"] * e["write_factor"])
    except (OSError, KeyError, ValueError):
        return None


def live_decode_traffic(budget_s=150.0):
    """HBM bytes per launch of the whole-step kernel, measured now: two child runs of this command under
    rocprofv3 --pmc (FETCH_SIZE, then WRITE_SIZE; one counter per run), each with one launch of a plain
    elementwise kernel of known traffic (--calibrate) that scales the counter.  Runs before this process
    touches the GPU.  Returns (bytes, description) or (None, reason); never raises."""
    import csv
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof):
        return None, "rocprofv3 not found"
    steps, warmup = 6, 2
    known_kib = {"FETCH_SIZE": 524288.0, "WRITE_SIZE": 262144.0}      # vt_add_kernel over 64 Mi floats
    kib = {}
    try:
        out = tempfile.mkdtemp(prefix="vt_traffic_", dir="/tmp")
    except OSError as e:
        return None, "no scratch directory: %s" % e
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            cmd = [rocprof, "--pmc", counter, "--output-format", "csv", "-d", os.path.join(out, counter), "-o", "t", "--",
                   sys.executable, os.path.abspath(__file__), "--steps", str(steps), "--warmup", str(warmup),
                   "--cpu-seconds", "0", "--calibrate", "--no-workloads", "--no-traffic"]
            p = subprocess.Popen(cmd, cwd="/tmp", env=dict(os.environ, TMPDIR="/tmp"), stdout=subprocess.DEVNULL,
                                 stderr=subprocess.DEVNULL, start_new_session=True)
            try:
                rc = p.wait(timeout=budget_s / 2)
            except subprocess.TimeoutExpired:
                os.killpg(p.pid, signal.SIGKILL)          # the process group this call started, nothing else
                p.wait()
                return None, "rocprofv3 --pmc %s did not finish in %.0f s" % (counter, budget_s / 2)
            if rc != 0:
                return None, "rocprofv3 --pmc %s exited with %d" % (counter, rc)
            step, add = [], []
            for path in glob.glob(os.path.join(out, counter, "**", "*counter_collection.csv"), recursive=True):
                with open(path, newline="") as f:
                    for row in csv.DictReader(f):
                        if row.get("Counter_Name") != counter:
                            continue
                        name = row.get("Kernel_Name", "")
                        if name.startswith("vt_decode_step_kernel"):
                            step.append(float(row["Counter_Value"]))
                        elif name.startswith("vt_add_kernel"):
                            add.append(float(row["Counter_Value"]))
            if not step or not add or min(add) <= 0:
                return None, "no %s rows for the step kernel and the calibration kernel" % counter
            kib[counter] = (sum(step) / len(step), known_kib[counter] / (sum(add) / len(add)), len(step))
    except (OSError, ValueError, KeyError) as e:
        return None, "traffic measurement failed: %s" % e
    finally:
        shutil.rmtree(out, ignore_errors=True)
    (fk, ff, n), (wk, wf, _) = kib["FETCH_SIZE"], kib["WRITE_SIZE"]
    desc = ("measured by this run: two child runs of this command under rocprofv3 --pmc (FETCH_SIZE %.1f KiB x %.3f, "
            "WRITE_SIZE %.1f KiB x %.3f per launch, mean of %d launches at positions %d..%d; factors from a kernel of "
            "known traffic in the same runs)" % (fk, ff, wk, wf, n, PROMPT, PROMPT + 2 * (warmup + steps)))
    return 1024.0 * (fk * ff + wk * wf), desc


TRAFFIC_SOURCE = "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command, scaled by a copy kernel; not measured by this run)"


def find_cblas():
    """A CBLAS sgemm found at run time, as (callable, description, threads), or (None, reason, 0).
    Looks for a system OpenBLAS, the OpenBLAS that scipy bundles (exported with a scipy_ prefix) and
    MKL, in that order; nothing is installed or built for it."""
    import ctypes.util
    import glob
    tries = []
    for name in ("openblas", "mkl_rt"):
        path = ctypes.util.find_library(name)
        if path:
            tries.append((path, "cblas_sgemm", "openblas_get_config", "openblas_get_num_threads"))
    try:
        import scipy
        libs = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs")
        for path in sorted(glob.glob(os.path.join(libs, "libscipy_openblas*.so*"))):
            tries.append((path, "scipy_cblas_sgemm", "scipy_openblas_get_config", "scipy_openblas_get_num_threads"))
    except ImportError:
        pass
    for path, sym, cfg, nthr in tries:
        try:
            lib = C.CDLL(path)
            fn = getattr(lib, sym)
        except (OSError, AttributeError):
            continue
        fn.restype = None
        fn.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_int,
                       C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_int]
        desc, threads = os.path.basename(path), 0
        try:
            g = getattr(lib, cfg)
            g.restype = C.c_char_p
            desc += ": " + g().decode()
            t = getattr(lib, nthr)
            t.restype = C.c_int
            threads = int(t())
        except AttributeError:
            pass
        return fn, desc, threads
    return None, "no CBLAS library found (libopenblas, scipy's bundled OpenBLAS, libmkl_rt)", 0


def cpu_blas_linears(sgemm, shapes, weights, m, budget_s):
    """The reference's seq_len > 1 linear in its BLAS build (voxtral_tts_kernels.c:187-198 and
    112-140): widen the whole bf16 matrix to fp32 (tts_bf16_to_f32_buf, :49-53), then
    cblas_sgemm(RowMajor, NoTrans, Trans, seq, out, in, 1, x, in, W, in, 0, y, out).  Times that pair
    for every (out, in) of `shapes` once (twice if the budget allows) on m rows of N(0,1) activations;
    returns the seconds per shape."""
    orc = CHK.vt.oracle()
    orc.orc_bf16_to_f32_buf.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    out = {}
    t_start = time.time()
    for (name, n, k), W in zip(shapes, weights):
        x = S.f32_normal((m, k), 77 + k)
        y = np.zeros((m, n), np.float32)
        wf = np.empty((n, k), np.float32)
        best = None
        for rep in range(2):
            t0 = time.time()
            orc.orc_bf16_to_f32_buf(wf.ctypes.data, W.ctypes.data, n * k)
            sgemm(101, 111, 112, m, n, k, 1.0, x.ctypes.data, k, wf.ctypes.data, k, 0.0, y.ctypes.data, n)
            dt = time.time() - t0
            best = dt if best is None else min(best, dt)
            if time.time() - t_start > budget_s:
                break
        out[name] = best
    return out


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
    n_cached = PROMPT
    if CHK.vt.have_ref():
        kind = "reference"
        b = CHK.cases.RefBackend()
        b.llm_open(layers, final_norm, kv_max)
        nbytes = N_LAYERS * kv_max * S.KV_DIM * 4
        C.memmove(b.lib.ref_kv_k(b.ctx), kv_k.ctypes.data, nbytes)
        C.memmove(b.lib.ref_kv_v(b.ctx), kv_v.ctypes.data, nbytes)
        b.lib.ref_set_kv_len(b.ctx, n_cached)
    else:
        kind = "port"
        b = CHK.cases.OracleBackend(threads=1)
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


MFMA_BF16_PEAK_TFLOPS = 2500.0
LAYER_WEIGHT_ELEMS = LAYER_WEIGHT_BYTES // 2
PREFILL_LEN = 512
GEMM_SHAPES = (("q|k|v", 6144, 3072), ("output", 3072, 4096), ("gate|up", 18432, 3072), ("down", 3072, 9216))


def prefill_flops(seq):
    """Algorithmic flops of a 26-layer prefill: 2 M N K per projection plus the causal
    attention (QK^T and PV over the visible keys of each query, 32 heads of 128)."""
    gemm = 2 * seq * LAYER_WEIGHT_ELEMS * N_LAYERS
    attn = 4 * S.HEAD_DIM * S.HEADS * (seq * (seq + 1) // 2) * N_LAYERS
    return gemm, attn


REF_LINEARS = (("wq", S.Q_DIM, S.DIM), ("wk", S.KV_DIM, S.DIM), ("wv", S.KV_DIM, S.DIM), ("wo", S.DIM, S.Q_DIM),
               ("w1", S.FFN, S.DIM), ("w3", S.FFN, S.DIM), ("w2", S.DIM, S.FFN))


def prefill_cpu_baseline(layers, budget_s, m=PREFILL_LEN, calls=N_LAYERS):
    """The seq_len > 1 products of the reference's BLAS build on this host: the seven linears of one
    layer at m rows (widen + sgemm each), times `calls` layer passes.  Attention, norms and RoPE
    (under 2 % of the reference's prefill) are left out and the figure says so."""
    sgemm, desc, threads = find_cblas()
    if sgemm is None:
        return {"value": None, "unit": "ms", "cores": 0, "kind": "reference-noblas", "sample": desc}
    # layer after layer (distinct weights, so nothing is served from a cache) until the budget is used
    t0, per, n_done = time.time(), {}, 0
    for l in layers:
        one = cpu_blas_linears(sgemm, REF_LINEARS, [getattr(l, n) for n, _, _ in REF_LINEARS], m, budget_s)
        for k, v in one.items():
            per[k] = per.get(k, 0.0) + v
        n_done += 1
        if time.time() - t0 > 0.7 * budget_s:
            break
    per = {k: v / n_done for k, v in per.items()}
    layer_s = sum(per.values())
    return {
        "value": round(layer_s * calls * 1e3, 1), "unit": "ms", "cores": threads or (os.cpu_count() or 1),
        "kind": "port", "library": desc,
        "sample": f"the seven linears of one layer at {m} rows as the reference's BLAS build runs them "
                  f"(tts_bf16_to_f32_buf of the whole matrix + cblas_sgemm, voxtral_tts_kernels.c:187-198, 112-140): "
                  f"{layer_s * 1e3:.0f} ms per layer (mean over {n_done} layers), x {calls}; attention / norms / RoPE "
                  f"not included",
        "per_linear_ms": {k: round(v * 1e3, 1) for k, v in per.items()},
    }


def bench_prefill(args):
    """BASELINE.json config "Backbone prefill": 26 layers, 512 random token ids, causal GQA
    attention.  A step is one whole prefill into an empty cache; inputs are resident in HBM."""
    K, W = args.steps, args.warmup
    workers = min(16, os.cpu_count() or 8)
    t0 = time.time()
    layers = make_layers(N_LAYERS, workers)
    final_norm = S.norm_weight(S.DIM, 99)
    ids = np.random.default_rng(11).integers(0, 131072, PREFILL_LEN)
    with ThreadPoolExecutor(workers) as ex:
        embeds = np.stack(list(ex.map(emb_row, ids))).astype(np.float32)
    t_gen = time.time() - t0
    hip = H.Hip(kv_max=PREFILL_LEN + 8)
    lib = hip.lib
    t0 = time.time()
    hip.upload_decoder(layers, final_norm, N_LAYERS)
    t_up = time.time() - t0
    d_e = H.DevBuf.from_numpy(lib, embeds)
    lib.tts_hip_set_prefill_mode(args.prefill_mode)
    for _ in range(W):
        lib.tts_hip_llm_prefill(d_e.ptr, PREFILL_LEN, 0)
    lib.tts_hip_sync()
    BL().tts_hip_timer_start()
    for _ in range(K):
        lib.tts_hip_llm_prefill(d_e.ptr, PREFILL_LEN, 0)
    ms_step = BL().tts_hip_timer_stop_ms() / K
    lib.tts_hip_sync()
    hip.check()
    gemm_fl, attn_fl = prefill_flops(PREFILL_LEN)
    # the dominant kernel alone, per projection shape, timed by the library with events
    per_shape = {}
    for i, (name, n, k) in enumerate(GEMM_SHAPES):
        ms = BL().tts_hip_bench_kernel(i, 50)
        fl = 2.0 * PREFILL_LEN * n * k
        per_shape[name] = {"N": n, "K": k, "us": round(ms * 1e3, 1), "tflops": round(fl / ms / 1e9, 1)}
    ms_attn = BL().tts_hip_bench_kernel(4, 50)
    hip.check()
    ms_gemm_layer = sum(v["us"] for v in per_shape.values()) / 1e3
    achieved = 2.0 * PREFILL_LEN * LAYER_WEIGHT_ELEMS / ms_gemm_layer / 1e9
    out = {
        "metric": "backbone prefill ms (512 tokens, 26 layers)",
        "value": round(ms_step, 4), "unit": "ms/prefill",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 weights x (hi, lo) bf16 activation planes, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "26-layer backbone prefill of 512 random token ids, causal GQA attention "
                               "(BASELINE.json configs[3])",
                   "layers": N_LAYERS, "seq_len": PREFILL_LEN, "weights": "bf16 N(0,0.02) seeded, truncated",
                   "schedule": ("one launch per product and row pass", "one persistent launch per layer behind the attention")[args.prefill_mode]},
        "tokens_per_s": round(PREFILL_LEN / (ms_step * 1e-3), 1),
        "tflops": round((gemm_fl + attn_fl) / ms_step / 1e9, 1),
        "roofline": {
            "kernel": "vt_gemm_wide_kernel (the four projection launches of one layer at M = 512)",
            "bound": "mfma",
            "achieved": round(achieved, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": measured_traffic("prefill"), "traffic_source": TRAFFIC_SOURCE,
            "flops_per_layer": 2 * PREFILL_LEN * LAYER_WEIGHT_ELEMS,
            "ms_per_layer": round(ms_gemm_layer, 4),
            "executed_over_algorithmic": 2.0,
            "per_shape": per_shape,
            "attention_us": round(ms_attn * 1e3, 1),
        },
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
        "cpu_baseline": None,
    }
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = prefill_cpu_baseline(layers, args.cpu_seconds)
    if args.cpu_seconds > 0 and CHK.vt.have_ref():
        # parity of the GPU prefill against the reference's own tts_llm_prefill on the first tokens
        n_cpu = 2
        b = CHK.cases.RefBackend()
        b.llm_open(layers, final_norm, 16)
        t0 = time.time()
        b.llm_prefill(embeds[:n_cpu])
        dt = time.time() - t0
        rk, rv = b.llm_kv()
        b.llm_close()
        lib.tts_hip_llm_prefill(embeds[:n_cpu].ctypes.data, n_cpu, 0)
        gk, gv = hip.kv()
        errs = [S.rel_errors(rk[l, r], gk[l, r]) for l in (0, N_LAYERS - 1) for r in range(n_cpu)]
        errs += [S.rel_errors(rv[l, r], gv[l, r]) for l in (0, N_LAYERS - 1) for r in range(n_cpu)]
        out["cpu_reference_noblas"] = {
            "value": round(dt / n_cpu * PREFILL_LEN * 1e3, 1), "unit": "ms/prefill", "cores": 1, "kind": "reference-noblas",
            "sample": f"tts_llm_prefill of the first {n_cpu} tokens through all 26 layers ({dt:.1f} s), scaled "
                      f"linearly to 512 tokens; no-BLAS build of the reference (its BLAS build needs <cblas.h>)",
        }
        out["parity"] = {"max_abs_over_rms": float(f"{max(e[0] for e in errs):.3e}"),
                         "rel_l2": float(f"{max(e[1] for e in errs):.3e}"),
                         "checked": f"K and V rows 0..{n_cpu - 1} of layers 0 and 25", "against": "reference",
                         "full_size": "tests/test_gpu_fullsize.py holds all 512 rows x 26 layers to 1e-3 against the CPU port"}
        assert out["parity"]["max_abs_over_rms"] < 1e-3, out["parity"]
    hip.close()
    print(json.dumps(out))


AC_LAYER_BYTES = LAYER_WEIGHT_BYTES
AC_PHASES = (("q|k|v", 10, 2 * 6144 * 3072), ("attention+output", 11, 2 * 3072 * 4096),
             ("gate|up", 12, 2 * 18432 * 3072), ("down", 13, 2 * 3072 * 9216))


def acoustic_frame_bytes():
    """Algorithmic HBM bytes of one frame: 7 Euler steps x 3 layers of bf16 weights (each streamed
    once per step for both guidance branches), the 36-wide in/out projections per step, the semantic
    head and the LLM-token projection once per frame.  Time tokens are cached per upload."""
    per_step = 3 * AC_LAYER_BYTES + 2 * (S.DIM * S.ACOUSTIC_DIM * 2) + 6 * S.DIM * 4
    return 7 * per_step + 8320 * S.DIM * 2 + S.DIM * S.DIM * 2


def bench_acoustic(args):
    """BASELINE.json config "Flow-matching acoustic transformer per frame": 3 layers, batch 2
    (conditional + unconditional, guidance 1.2), 7 Euler steps, FSQ.  A step is one frame."""
    K, W = args.steps, args.warmup
    t0 = time.time()
    ac = S.Acoustic(50)
    t_gen = time.time() - t0
    hip = H.Hip(kv_max=8)
    lib = hip.lib
    t0 = time.time()
    hip.upload_acoustic(ac)
    t_up = time.time() - t0
    hs = [S.f32_normal(S.DIM, 20 + f) for f in range(8)]
    xs = [S.f32_normal(S.ACOUSTIC_DIM, 4200 + f) for f in range(8)]      # the frames' noise: any N(0,1) draw
    codes = np.zeros(S.CODES, np.int32)
    d_h = [H.DevBuf.from_numpy(lib, h) for h in hs]
    d_x = [H.DevBuf.from_numpy(lib, x) for x in xs]
    for i in range(W):
        lib.tts_hip_acoustic_frame(codes.ctypes.data, d_h[i % 8].ptr, d_x[i % 8].ptr, None)
    lib.tts_hip_sync()
    t0 = time.time()
    for i in range(K):
        lib.tts_hip_acoustic_frame(codes.ctypes.data, d_h[i % 8].ptr, d_x[i % 8].ptr, None)
    lib.tts_hip_sync()
    ms_step = (time.time() - t0) * 1e3 / K          # host clock: every frame ends in a device->host copy
    hip.check()
    per_phase = {}
    for name, which, nbytes in AC_PHASES:
        ms = BL().tts_hip_bench_kernel(which, 50)
        per_phase[name] = {"us": round(ms * 1e3, 1), "gbps": round(nbytes / ms / 1e6, 1)}
    # the four launches of a layer in order, each turn on the next layer's weights, as inside a frame
    ms_layer = BL().tts_hip_bench_kernel(14, 60)
    hip.check()
    achieved = AC_LAYER_BYTES / ms_layer / 1e6
    fb = acoustic_frame_bytes()
    out = {
        "metric": "acoustic transformer ms/frame",
        "value": round(ms_step, 4), "unit": "ms/frame",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 weights x (hi, lo) bf16 activation planes, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "flow-matching acoustic transformer, one frame: semantic head + 7 Euler steps of "
                               "3 layers at batch 2 x 3 tokens, guidance 1.2, FSQ (BASELINE.json configs[4])",
                   "weights": "bf16 N(0,0.02) seeded, truncated", "timed": "host clock over whole frames, "
                   "inputs resident in HBM, 37 codes copied back per frame"},
        "frames_per_s": round(1000.0 / ms_step, 1),
        "hbm_gbps": round(fb / (ms_step * 1e-3) / 1e9, 1),
        "hbm_frac_of_peak": round(fb / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "roofline": {
            "kernel": "vt_ac_phase_kernel (the four launches of one layer, 6 activation rows)",
            "bound": "hbm",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("acoustic"), "traffic_source": TRAFFIC_SOURCE,
            "bytes_per_layer": AC_LAYER_BYTES, "ms_per_layer": round(ms_layer, 4),
            "per_phase_alone": per_phase,
            "note": "ms_per_layer: the four launches in order, rotating over the 3 layers; per_phase_alone: one "
                    "phase launched back to back (its weights partly stay in the memory-side cache)",
        },
        "bytes_per_frame": fb,
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
        "cpu_baseline": None,
    }
    if args.cpu_seconds > 0:
        # 14 velocity evaluations per frame (7 Euler steps x 2 guidance branches), each 3 layers at 3 rows
        base = prefill_cpu_baseline(ac.layers, args.cpu_seconds, m=3, calls=14 * 3)
        base["unit"] = "ms/frame"
        out["cpu_baseline"] = base
    if args.cpu_seconds > 0:
        # parity: as many frames as fit the budget against the CPU port on all host threads (bit-identical
        # to one thread), noise from the restated host RNG at seed 42
        orc = CHK.cases.OracleBackend(threads=min(16, os.cpu_count() or 1))
        orc.ac_open(ac)
        st2 = C.c_uint64(0)
        T = CHK.vt
        T.oracle().orc_rng_seed(C.byref(st2), 42)
        equal = total = 0
        worst = 0.0
        t0 = time.time()
        f = 0
        while f < 200 and time.time() - t0 < args.cpu_seconds:
            h = S.f32_normal(S.DIM, 20 + f)
            rc, _, rx = orc.acoustic_forward(h, seed=42 if f == 0 else None, want_x=True)
            x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
            if rc[0] != 1:
                T.oracle().orc_randn_fill(C.byref(st2), T.fp(x0), S.ACOUSTIC_DIM)
            g, gx = hip.acoustic_frame(h, x0)
            equal += int(np.sum(g == rc))
            total += S.CODES
            if rc[0] != 1:
                worst = max(worst, float(np.max(np.abs(gx.astype(np.float64) - rx))))
            f += 1
        out["parity"] = {"codes_equal": equal, "codes": total, "frames": f, "max_latent_diff": float(f"{worst:.3e}"),
                         "against": "port", "full_size": "tests/test_gpu_fullsize.py runs all 200 frames (7,400 codes)"}
        assert worst < 1e-4, worst
    if args.cpu_seconds > 0 and CHK.vt.have_ref():
        # one frame of the reference's tts_acoustic_forward (14 velocity evaluations), single thread, no BLAS
        b = CHK.cases.RefBackend()
        b.ac_open(ac)
        t0 = time.time()
        rc, _ = b.acoustic_forward(hs[0], seed=42)
        dt = time.time() - t0
        b.ac_close()
        st3 = C.c_uint64(0)
        CHK.vt.oracle().orc_rng_seed(C.byref(st3), 42)
        x42 = np.zeros(S.ACOUSTIC_DIM, np.float32)
        CHK.vt.oracle().orc_randn_fill(C.byref(st3), CHK.vt.fp(x42), S.ACOUSTIC_DIM)     # the noise the reference drew
        g, _ = hip.acoustic_frame(hs[0], x42)
        out["cpu_reference_noblas"] = {"value": round(dt * 1e3, 1), "unit": "ms/frame", "cores": 1, "kind": "reference-noblas",
                                       "sample": "one frame of tts_acoustic_forward at seed 42 (same hidden state and noise)"}
        assert np.array_equal(g, rc), (g, rc)
    hip.close()
    print(json.dumps(out))


MFMA_F32_PEAK_TFLOPS = 157.3
CODEC_FRAMES = 200


def codec_flops(frames):
    """Algorithmic flops of one codec decode: the 8 transformer layers at 1x, 2x, 4x, 8x the frame
    count (7 products each), the three transposed convolutions, the input and output convolutions
    (unpadded sizes) and the windowed attention."""
    d, hid = 1024, 4096
    total = frames * 2 * (292 * 3) * d
    for stage, window in enumerate((2, 4, 8, 16)):
        t = frames << stage
        total += 2 * t * 2 * (4 * d * d + 3 * d * hid)
        total += 2 * t * 8 * window * 128 * 4
        if stage < 3:
            total += t * 2 * d * d * 4
    total += (frames * 8) * 2 * d * 240 * 7
    return total


def bench_codec(args):
    """Codec decoder: 200 frames of 37 codes (16 s of audio) -> 384,000 samples.  A step is one such
    decode with codes and waveform resident in HBM."""
    K, CC = CHK.codecsupport, CHK.codec_cases      # weight-norm reconstruction of the synthetic weights: the checker's
    Kk, W = args.steps, args.warmup
    t0 = time.time()
    hc = K.HostCodec(5)
    t_gen = time.time() - t0
    hip = H.Hip(kv_max=8)
    lib = hip.lib
    t0 = time.time()
    cs = hc.struct()
    assert lib.tts_hip_upload_codec_weights(C.addressof(cs)) == 0, lib.tts_hip_last_error()
    t_up = time.time() - t0
    codes = K.random_codes(CODEC_FRAMES, 77)
    d_codes = H.DevBuf.from_numpy(lib, codes)
    d_wave = H.DevBuf(lib, CODEC_FRAMES * 1920 * 4)
    for _ in range(W):
        assert lib.tts_hip_codec_decode_device(d_codes.ptr, CODEC_FRAMES, d_wave.ptr) == 0
    lib.tts_hip_sync()
    BL().tts_hip_timer_start()
    for _ in range(Kk):
        lib.tts_hip_codec_decode_device(d_codes.ptr, CODEC_FRAMES, d_wave.ptr)
    ms_step = BL().tts_hip_timer_stop_ms() / Kk
    hip.check()
    wave = d_wave.to_numpy(np.float32, (CODEC_FRAMES * 1920,))
    shapes = (("qkv 1600x3072x1024", 20, 1600 * 3072 * 1024 * 2), ("wo 1600x1024x1024", 21, 1600 * 1024 * 1024 * 2),
              ("gate|up 1600x8192x1024", 22, 1600 * 8192 * 1024 * 2), ("down 1600x1024x4096", 23, 1600 * 1024 * 4096 * 2))
    per_shape = {}
    for name, which, fl in shapes:
        ms = BL().tts_hip_bench_kernel(which, 30)
        per_shape[name] = {"us": round(ms * 1e3, 1), "tflops": round(fl / ms / 1e9, 1)}
    hip.check()
    layer_fl = sum(fl for _, _, fl in shapes)
    layer_ms = sum(v["us"] for v in per_shape.values()) / 1e3
    achieved = layer_fl / layer_ms / 1e9
    fl = codec_flops(CODEC_FRAMES)
    audio_s = CODEC_FRAMES * FRAME_SECONDS
    out = {
        "metric": "codec decode ms per 200-frame utterance",
        "value": round(ms_step, 4), "unit": "ms/utterance",
        "n_gpus": 1, "steps": Kk, "warmup": W, "ms_per_step": round(ms_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "audio codec decoder: 200 frames x 37 codes -> 384,000 samples at 24 kHz (16 s): "
                               "conv 292->1024, 4 stages of 2 ALiBi sliding-window transformer layers (dim 1024, "
                               "hidden 4096, windows 2/4/8/16) with 2x transposed convolutions between, conv 1024->240",
                   "weights": "f32 seeded, weight norm folded", "timed": "events on the library's stream, codes and "
                   "waveform resident in HBM"},
        "tflops": round(fl / ms_step / 1e9, 1),
        "times_real_time": round(audio_s * 1e3 / ms_step, 1),
        "roofline": {
            "kernel": "vt_codec_gemm_kernel (the four products of a last-stage layer, 1600 rows)",
            "bound": "mfma",
            "achieved": round(achieved, 1), "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_F32_PEAK_TFLOPS, 4),
            "traffic": measured_traffic("codec"), "traffic_source": TRAFFIC_SOURCE,
            "flops_per_layer": layer_fl, "ms_per_layer": round(layer_ms, 4), "per_shape": per_shape,
        },
        "flops_per_utterance": fl,
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
        "cpu_baseline": None,
    }
    if args.cpu_seconds > 0 and CHK.vt.have_ref():
        n = 8
        b = CC.RefCodecBackend()
        b.open(hc)
        t0 = time.time()
        ref = b.decode(codes[:n])
        dt = time.time() - t0
        b.close()
        got = wave[:n * 1920]
        # the decoder is causal: the first 8 frames of the long decode equal a decode of 8 frames
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        out["cpu_baseline"] = {"value": round(dt * 1e3 * CODEC_FRAMES / n, 1), "unit": "ms/utterance", "cores": 1,
                               "kind": "reference",
                               "sample": f"tts_codec_decode on the first {n} frames ({dt:.1f} s), scaled by {CODEC_FRAMES // n} "
                                         "(the cost is linear in the frame count: windowed attention)"}
        out["parity"] = {"max_abs_over_rms": float(f"{np.abs(ref - got).max() / rms:.3e}"),
                         "samples_checked": int(ref.size), "against": "reference"}
        assert np.abs(ref - got).max() / rms < 1e-3
    hip.close()
    print(json.dumps(out))


AUDIO_ROWS = 8194 + 36 * 23
FRAME_SECONDS = 0.08                      # one frame of codes is 80 ms of audio (12.5 Hz)


def bench_frame(args):
    """The whole per-frame loop of voxtral_tts.c:301-321 on the device: 26-layer backbone step,
    acoustic frame (semantic head, 7 guided Euler steps, FSQ) and the audio-code embedding that
    becomes the next backbone input.  A step is one frame; 64-token prompt prefilled first."""
    K, W = args.steps, args.warmup
    workers = min(16, os.cpu_count() or 8)
    t0 = time.time()
    layers = make_layers(N_LAYERS, workers)
    final_norm = S.norm_weight(S.DIM, 99)
    ac = S.Acoustic(50)
    table = S.bf16_normal((AUDIO_ROWS, S.DIM), 4242, 0.05)
    offs = np.zeros(S.CODES, np.int32)
    offs[1] = 8194
    for i in range(2, S.CODES):
        offs[i] = offs[i - 1] + 23
    ids = np.random.default_rng(7).integers(0, 131072, PROMPT)
    prompt = np.stack([emb_row(t) for t in ids]).astype(np.float32)
    t_gen = time.time() - t0
    hip = H.Hip(kv_max=PROMPT + W + K + 8)
    lib = hip.lib
    t0 = time.time()
    hip.upload_decoder(layers, final_norm, N_LAYERS)
    hip.upload_acoustic(ac)
    assert lib.tts_hip_upload_audio_embeddings(table.ctypes.data, AUDIO_ROWS, offs.ctypes.data) == 0
    t_up = time.time() - t0
    hip.llm_prefill(prompt)
    noise = S.f32_normal((W + K, S.ACOUSTIC_DIM), 4200)      # the frames' noise: any N(0,1) draw
    d_e = H.DevBuf.from_numpy(lib, emb_row(24))          # the audio start token's stand-in
    codes = np.zeros(S.CODES, np.int32)
    pos = PROMPT
    n_end = 0
    for f in range(W):
        lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, noise[f].ctypes.data, pos)
        pos += 1
    lib.tts_hip_sync()
    t0 = time.time()
    for f in range(W, W + K):
        lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, noise[f].ctypes.data, pos)
        n_end += int(codes[0] == 1)
        pos += 1
    lib.tts_hip_sync()
    ms_step = (time.time() - t0) * 1e3 / K
    hip.check()
    fb = step_bytes(PROMPT + W + (K - 1) / 2.0) + acoustic_frame_bytes() + S.CODES * S.DIM * 2
    out = {
        "metric": "generation loop ms/frame (backbone step + acoustic frame + code embedding)",
        "value": round(ms_step, 4), "unit": "ms/frame",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 activations, bf16 weights", "data": "synthetic",
        "config": {"workload": "per-frame generation loop on the device (configs[2] + configs[4] chained through the "
                               "audio-code embedding), 64-token prompt", "layers": N_LAYERS,
                   "timed": "host clock over whole frames; per frame 36 floats of noise go in, 37 codes come back"},
        "frames_per_s": round(1000.0 / ms_step, 1),
        "realtime_factor": round(FRAME_SECONDS * 1000.0 / ms_step, 1),
        "end_audio_frames": n_end,
        "roofline": {"kernel": "whole frame (vt_decode_step_kernel + 84 vt_ac_phase_kernel launches)", "bound": "hbm",
                     "achieved": round(fb / (ms_step * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(fb / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_frame": int(fb)},
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
        "cpu_baseline": None,
    }
    hip.close()
    print(json.dumps(out))


MATVEC_SHAPES = ((9216, 3072, "FFN up/gate"), (3072, 9216, "FFN down"), (131072, 3072, "LM-head sized"))


def bench_matvec(args):
    """The single bf16 matvec of configs[0]: y = W x, W bf16 ~N(0,0.02), x f32 ~N(0,1), the three
    shapes of the reference's CPU kernel.  A step is one product; launches rotate through copies of
    the two small matrices (8 x 56.6 MB) so that every one streams from HBM, not the memory-side cache."""
    K, W = args.steps, args.warmup
    hip = H.Hip(kv_max=8)
    lib = hip.lib
    cpu_lib = kind = None
    if args.cpu_seconds > 0:
        cpu_lib = CHK.cases.RefBackend() if CHK.vt.have_ref() else CHK.cases.OracleBackend(threads=1)
        kind = "reference" if CHK.vt.have_ref() else "port"
    per_shape, t_gen, t_up = {}, 0.0, 0.0
    cpu_ms, parity = {}, {}
    for n, k, what in MATVEC_SHAPES:
        t0 = time.time()
        Wm = S.bf16_normal((n, k), 1000 + n % 97 + k)
        x = S.f32_normal((1, k), 42)
        t_gen += time.time() - t0
        nbytes = 2 * n * k + 4 * k + 4 * n
        copies = 8 if 2 * n * k < (512 << 20) else 1
        t0 = time.time()
        d_W = H.DevBuf(lib, copies * 2 * n * k)
        for c in range(copies):
            lib.tts_hip_to_device(d_W.at(c * 2 * n * k), Wm.ctypes.data, 2 * n * k)
        d_x = H.DevBuf.from_numpy(lib, x)
        d_y = H.DevBuf(lib, 4 * n)
        t_up += time.time() - t0
        ms = BL().tts_hip_bench_matvec(d_y.ptr, d_x.ptr, d_W.ptr, n * k, copies, k, n, max(K, copies))
        hip.check()
        got = d_y.to_numpy(np.float32, (1, n))
        name = f"{n}x{k}"
        per_shape[name] = {"what": what, "us": round(ms * 1e3, 2), "bytes": nbytes,
                           "gbps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
                           "copies": copies}
        if args.cpu_seconds > 0:
            reps = 3 if n * k < (1 << 28) else 1
            t0 = time.time()
            for _ in range(reps):
                ref = cpu_lib.linear(x, Wm, None, 1)
            cpu_ms[name] = round((time.time() - t0) / reps * 1e3, 1)
            mx, l2 = S.rel_errors(ref, got)
            parity[name] = {"max_abs_over_rms": float(f"{mx:.3g}"), "l2_rel": float(f"{l2:.3g}")}
            assert mx < 1e-3 and l2 < 1e-3, (name, mx, l2)
        for b in (d_W, d_x, d_y):
            b.free()
    big = per_shape["131072x3072"]
    out = {
        "metric": "bf16 matvec achieved HBM GB/s (131072x3072)",
        "value": big["gbps"], "unit": "GB/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(big["us"] / 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "single bf16 matvec y = W x, batch 1, fp32 accumulate (BASELINE.json configs[0]): "
                               "9216x3072, 3072x9216 and 131072x3072",
                   "weights": "bf16 N(0,0.02) seeded, truncated", "activations": "f32 N(0,1)",
                   "timed": "events on the library's stream, operands resident in HBM"},
        "per_shape": per_shape,
        "roofline": {"kernel": "vt_matvec_kernel (131072x3072)", "bound": "hbm", "achieved": big["gbps"],
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": big["frac"], "traffic": measured_traffic("matvec"), "traffic_source": TRAFFIC_SOURCE,
                     "bytes_per_launch": big["bytes"], "ms_per_launch": round(big["us"] / 1e3, 5)},
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
        "cpu_baseline": None,
    }
    if cpu_ms:
        name = "131072x3072"
        out["cpu_baseline"] = {"value": round(per_shape[name]["bytes"] / cpu_ms[name] / 1e6, 2), "unit": "GB/s",
                               "cores": 1, "kind": kind, "ms": cpu_ms,
                               "sample": "the same three products through the reference's tts_linear_bf16 "
                                         "(bf16_matvec_fused), one thread, 3 / 3 / 1 repetitions"}
        out["parity"] = parity
    hip.close()
    print(json.dumps(out))


def bench_layer(args):
    """configs[1]: one decoder layer, decode step at batch 1 over a KV cache of 512 positions
    ~N(0,1).  A step is one tts_hip_layer_decode on a device-resident hidden state (the whole-step
    kernel run over a single layer, final norm off)."""
    K, W = args.steps, args.warmup
    pos, kv_max = 512, 520
    layer = S.Layer(3)
    ones = np.ones(S.DIM, np.float32)
    k = np.zeros((N_LAYERS, kv_max, S.KV_DIM), np.float32)
    v = np.zeros((N_LAYERS, kv_max, S.KV_DIM), np.float32)
    k[0, :pos] = S.f32_normal((pos, S.KV_DIM), 200)
    v[0, :pos] = S.f32_normal((pos, S.KV_DIM), 300)
    x = S.f32_normal(S.DIM, 42)
    hip = H.Hip(kv_max=kv_max)
    lib = hip.lib
    hip.upload_decoder([layer], ones, 1)
    hip.set_kv(k, v)
    lib.tts_hip_set_decode_mode(args.mode)
    d_x = H.DevBuf.from_numpy(lib, x)
    lib.tts_hip_layer_decode(0, d_x.ptr, pos)
    lib.tts_hip_sync()
    hip.check()
    got = d_x.to_numpy(np.float32, (S.DIM,))
    d_in = H.DevBuf.from_numpy(lib, x)
    for _ in range(W):
        lib.tts_hip_to_device(d_x.ptr, x.ctypes.data, x.nbytes)
        lib.tts_hip_layer_decode(0, d_x.ptr, pos)
    lib.tts_hip_sync()
    # the hidden state is fed back in place: values drift but the bytes moved do not depend on them
    lib.tts_hip_to_device(d_x.ptr, x.ctypes.data, x.nbytes)
    BL().tts_hip_timer_start()
    for _ in range(K):
        lib.tts_hip_layer_decode(0, d_x.ptr, pos)
    ms = BL().tts_hip_timer_stop_ms() / K
    hip.check()
    nbytes = LAYER_WEIGHT_BYTES + 2 * S.DIM * 4 + 2 * (pos + 1) * S.KV_DIM * 4 + 2 * S.KV_DIM * 4 + 2 * S.DIM * 4
    gbps = nbytes / ms / 1e6
    out = {
        "metric": "one decoder layer, decode step ms (512 cached positions)",
        "value": round(ms * 1e3, 2), "unit": "us/step",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "one Mistral decoder layer, decode step at batch 1, KV cache of 512 positions ~N(0,1), "
                               "hidden ~N(0,1) (BASELINE.json configs[1])",
                   "weights": "bf16 N(0,0.02) seeded, truncated", "activations": "f32",
                   "schedule": {0: "persistent whole-step kernel over one layer",
                                1: "one kernel per phase"}.get(args.mode, str(args.mode)),
                   "timed": "events on the library's stream, back-to-back launches, operands resident in HBM"},
        "hbm_gbps": round(gbps, 1),
        "roofline": {"kernel": "vt_decode_step_kernel (one layer)", "bound": "hbm", "achieved": round(gbps, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": nbytes, "ms_per_launch": round(ms, 5)},
        "cpu_baseline": None,
    }
    if args.cpu_seconds > 0:
        kind = "reference" if CHK.vt.have_ref() else "port"
        if CHK.vt.have_ref():
            b = CHK.cases.RefBackend()
            b.llm_open([layer] * N_LAYERS, ones, kv_max)
            nb = N_LAYERS * kv_max * S.KV_DIM * 4
            C.memmove(b.lib.ref_kv_k(b.ctx), k.ctypes.data, nb)
            C.memmove(b.lib.ref_kv_v(b.ctx), v.ctypes.data, nb)
            b.lib.ref_set_kv_len(b.ctx, pos)
            t0 = time.time()
            b.llm_forward(x)                                   # 26 layers: the reference has no per-layer entry
            cpu_ms = (time.time() - t0) * 1e3 / N_LAYERS
            b.llm_close()
            sample = "one tts_llm_forward over 26 copies of the layer at pos 512, divided by 26"
        else:
            b = CHK.cases.OracleBackend(threads=1)
            b.llm_open([layer], ones, kv_max, n_layers=1)
            b.kv_k[0], b.kv_v[0] = k[0], v[0]
            b.pos = pos
            t0 = time.time()
            b.llm_forward(x)
            cpu_ms = (time.time() - t0) * 1e3
            sample = "one layer step of the CPU port at pos 512"
        out["cpu_baseline"] = {"value": round(cpu_ms * 1e3, 0), "unit": "us/step", "cores": 1, "kind": kind,
                               "sample": sample, "gbps": round(nbytes / cpu_ms / 1e6, 2)}
        # parity of the timed entry point against the CPU port: the port's hidden state is the final
        # norm (unit gains) of the residual stream that tts_hip_layer_decode leaves
        o = CHK.cases.OracleBackend(threads=8)
        o.llm_open([layer], ones, kv_max, n_layers=1)
        o.kv_k[0], o.kv_v[0] = k[0], v[0]
        o.pos = pos
        ref_h = o.llm_forward(x)
        renorm = o.rms_norm(got.reshape(1, -1), ones, 1)[0]
        mx, l2 = S.rel_errors(ref_h, renorm)
        out["parity"] = {"max_abs_over_rms": float(f"{mx:.3g}"), "rel_l2": float(f"{l2:.3g}"), "against": "port"}
        assert mx < 1e-3 and l2 < 1e-3, (mx, l2)
    hip.close()
    print(json.dumps(out))


def other_workloads(hip, kv_max):
    """Short runs of the other BASELINE.json configurations inside the default line, so that one
    command shows every kernel's rate: the three single products (configs[0]), one decoder layer at
    512 cached positions (configs[1]), the 512-token prefill (configs[3]) and the acoustic frame
    (configs[4]).  Weights of the single products are a constant fill (timing only; their parity is
    in tests/); the backbone runs use the 26 uploaded layers, each launch on the next layer so that
    weights come from HBM.  The full lines, with CPU baseline and parity, are --workload <name>."""
    lib = hip.lib
    w = {}
    # configs[0]
    for n, k, what in MATVEC_SHAPES:
        copies = 8 if 2 * n * k < (512 << 20) else 1
        d_W = H.DevBuf(lib, copies * 2 * n * k)
        lib.tts_hip_memset(d_W.ptr, 0x3c, copies * 2 * n * k)          # bf16 0x3c3c = 0.0115
        d_x = H.DevBuf.from_numpy(lib, S.f32_normal((1, k), 42))
        d_y = H.DevBuf(lib, 4 * n)
        ms = BL().tts_hip_bench_matvec(d_y.ptr, d_x.ptr, d_W.ptr, n * k, copies, k, n, 24)
        nbytes = 2 * n * k + 4 * k + 4 * n
        w[f"matvec {n}x{k}"] = {"config": 0, "kernel": "vt_matvec_kernel", "us": round(ms * 1e3, 2), "launches": 24,
                                "achieved": round(nbytes / ms / 1e6, 1), "unit": "GB/s",
                                "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        for b in (d_W, d_x, d_y):
            b.free()
    # configs[1]: one layer per launch at position 512, walking through the 26 layers
    pos = PREFILL_LEN
    d_x = H.DevBuf.from_numpy(lib, S.f32_normal(S.DIM, 42))
    for l in range(N_LAYERS):
        lib.tts_hip_layer_decode(l, d_x.ptr, pos)
    lib.tts_hip_sync()
    BL().tts_hip_timer_start()
    n_l = 2 * N_LAYERS
    for i in range(n_l):
        lib.tts_hip_layer_decode(i % N_LAYERS, d_x.ptr, pos)
    ms = BL().tts_hip_timer_stop_ms() / n_l
    nbytes = LAYER_WEIGHT_BYTES + 2 * S.DIM * 4 + 2 * (pos + 1) * S.KV_DIM * 4 + 2 * S.KV_DIM * 4 + 2 * S.DIM * 4
    w["layer decode, 512 cached positions"] = {
        "config": 1, "kernel": "vt_decode_step_kernel (one layer per launch)", "us": round(ms * 1e3, 2), "launches": n_l,
        "achieved": round(nbytes / ms / 1e6, 1), "unit": "GB/s", "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    d_x.free()
    # configs[3]: whole prefills, then the product kernel per projection shape
    d_e = H.DevBuf.from_numpy(lib, S.f32_normal((PREFILL_LEN, S.DIM), 11))
    for _ in range(3):
        lib.tts_hip_llm_prefill(d_e.ptr, PREFILL_LEN, 0)
    lib.tts_hip_sync()
    BL().tts_hip_timer_start()
    for _ in range(8):
        lib.tts_hip_llm_prefill(d_e.ptr, PREFILL_LEN, 0)
    ms = BL().tts_hip_timer_stop_ms() / 8
    gemm_fl, attn_fl = prefill_flops(PREFILL_LEN)
    ms_layer = sum(BL().tts_hip_bench_kernel(i, 26) for i in range(4))
    achieved = 2.0 * PREFILL_LEN * LAYER_WEIGHT_ELEMS / ms_layer / 1e9
    w["prefill, 512 tokens x 26 layers"] = {
        "config": 3, "kernel": "vt_gemm_wide_kernel (the projection launches of one layer)", "ms": round(ms, 3), "launches": 8,
        "tokens_per_s": round(PREFILL_LEN / (ms * 1e-3), 1), "tflops_whole_prefill": round((gemm_fl + attn_fl) / ms / 1e9, 1),
        "us_products_per_layer": round(ms_layer * 1e3, 1), "achieved": round(achieved, 1), "unit": "TFLOP/s",
        "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "attention_us_per_layer": round(BL().tts_hip_bench_kernel(4, 26) * 1e3, 1)}
    d_e.free()
    # configs[4]
    ac = S.Acoustic(50)
    hip.upload_acoustic(ac)
    x0 = S.f32_normal(S.ACOUSTIC_DIM, 4200)
    d_h, d_x0 = H.DevBuf.from_numpy(lib, S.f32_normal(S.DIM, 20)), H.DevBuf.from_numpy(lib, x0)
    codes = np.zeros(S.CODES, np.int32)
    for _ in range(2):
        lib.tts_hip_acoustic_frame(codes.ctypes.data, d_h.ptr, d_x0.ptr, None)
    t0 = time.perf_counter()
    for _ in range(10):
        lib.tts_hip_acoustic_frame(codes.ctypes.data, d_h.ptr, d_x0.ptr, None)
    ms = (time.perf_counter() - t0) * 1e3 / 10
    ms_layer = BL().tts_hip_bench_kernel(14, 30)
    achieved = AC_LAYER_BYTES / ms_layer / 1e6
    w["acoustic frame"] = {
        "config": 4, "kernel": "vt_ac_phase_kernel (the launches of one layer, in order)", "ms": round(ms, 4), "launches": 10,
        "frame_gbps": round(acoustic_frame_bytes() / ms / 1e6, 1), "us_per_layer": round(ms_layer * 1e3, 1),
        "achieved": round(achieved, 1), "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4)}
    # configs[2] at the cache lengths of a real utterance (~250 prompt rows + up to 2000 frames): the whole-step
    # kernel at a fixed position over K and V rows filled by a kernel with pseudo-random values
    ctx = PKG.ctx()
    d_e, d_hid = H.DevBuf.from_numpy(lib, S.f32_normal(S.DIM, 43)), H.DevBuf(lib, S.DIM * 4)
    for pos in (1024, 2000):
        if pos + 1 > kv_max:
            continue
        for base in (ctx.kv_cache_k_gpu, ctx.kv_cache_v_gpu):
            for l in range(N_LAYERS):
                BL().tts_hip_bench_fill_f32(base + l * kv_max * S.KV_DIM * 4, pos * S.KV_DIM)
        for _ in range(3):
            lib.tts_hip_llm_forward_device(d_hid.ptr, d_e.ptr, pos)
        lib.tts_hip_sync()
        BL().tts_hip_timer_start()
        n_l = 12
        for _ in range(n_l):
            lib.tts_hip_llm_forward_device(d_hid.ptr, d_e.ptr, pos)
        ms = BL().tts_hip_timer_stop_ms() / n_l
        nb = step_bytes(pos)
        assert np.all(np.isfinite(d_hid.to_numpy(np.float32, S.DIM)))
        w[f"decode @{pos} cached positions"] = {
            "config": 2, "kernel": "vt_decode_step_kernel", "ms": round(ms, 4), "launches": n_l, "bytes_per_launch": int(nb),
            "achieved": round(nb / ms / 1e6, 1), "unit": "GB/s", "frac": round(nb / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    # the generation loop (voxtral_tts.c:301-321) on the device: backbone step + acoustic frame + code embedding
    table = S.bf16_normal((AUDIO_ROWS, S.DIM), 4242, 0.05)
    offs = np.zeros(S.CODES, np.int32)
    offs[1] = 8194
    for i in range(2, S.CODES):
        offs[i] = offs[i - 1] + 23
    assert lib.tts_hip_upload_audio_embeddings(table.ctypes.data, AUDIO_ROWS, offs.ctypes.data) == 0
    noise = S.f32_normal((16, S.ACOUSTIC_DIM), 4300)
    lib.tts_hip_to_device(d_e.ptr, emb_row(24).ctypes.data, S.DIM * 4)
    pos, n_f = PROMPT, 12
    for f in range(4):
        lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, noise[f].ctypes.data, pos + f)
    t0 = time.perf_counter()
    for f in range(4, 4 + n_f):
        lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, noise[f].ctypes.data, pos + f)
    ms = (time.perf_counter() - t0) * 1e3 / n_f
    fb = step_bytes(pos + 4 + (n_f - 1) / 2.0) + acoustic_frame_bytes() + S.CODES * S.DIM * 2
    w["generation loop (backbone step + acoustic frame + code embedding)"] = {
        "config": "2+4", "kernel": "vt_decode_step_kernel + vt_ac_phase_kernel launches", "ms": round(ms, 4), "launches": n_f,
        "frames_per_s": round(1000.0 / ms, 1), "realtime_factor": round(FRAME_SECONDS * 1000.0 / ms, 1),
        "bytes_per_frame": int(fb), "achieved": round(fb / ms / 1e6, 1), "unit": "GB/s",
        "frac": round(fb / ms / 1e6 / HBM_PEAK_GBPS, 4), "timed": "host clock, one synchronisation per frame"}
    for b in (d_e, d_hid):
        b.free()
    # the codec decoder on 200 frames (16 s of audio), codes and waveform resident
    cw = S.CodecWeights(5)
    cs = cw.struct()
    assert lib.tts_hip_upload_codec_weights(C.addressof(cs)) == 0, lib.tts_hip_last_error()
    d_codes = H.DevBuf.from_numpy(lib, cw.random_codes(CODEC_FRAMES, 77))
    d_wave = H.DevBuf(lib, CODEC_FRAMES * 1920 * 4)
    for _ in range(2):
        assert lib.tts_hip_codec_decode_device(d_codes.ptr, CODEC_FRAMES, d_wave.ptr) == 0
    lib.tts_hip_sync()
    BL().tts_hip_timer_start()
    for _ in range(6):
        lib.tts_hip_codec_decode_device(d_codes.ptr, CODEC_FRAMES, d_wave.ptr)
    ms = BL().tts_hip_timer_stop_ms() / 6
    assert np.all(np.isfinite(d_wave.to_numpy(np.float32, (CODEC_FRAMES * 1920,))))
    ms_l = sum(BL().tts_hip_bench_kernel(k, 12) for k in (20, 21, 22, 23))
    fl_l = 2.0 * 1600 * 1024 * (3072 + 1024 + 8192 + 4096)
    w["codec decode, 200 frames"] = {
        "config": "N4", "kernel": "vt_codec_gemm_kernel (the four products of a last-stage layer)", "ms": round(ms, 4), "launches": 6,
        "tflops_whole_decode": round(codec_flops(CODEC_FRAMES) / ms / 1e9, 1),
        "times_real_time": round(CODEC_FRAMES * FRAME_SECONDS * 1e3 / ms, 1), "us_products_per_layer": round(ms_l * 1e3, 1),
        "achieved": round(fl_l / ms_l / 1e9, 1), "unit": "TFLOP/s", "frac": round(fl_l / ms_l / 1e9 / MFMA_F32_PEAK_TFLOPS, 4)}
    for b in (d_codes, d_wave):
        b.free()
    hip.check()
    return w


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=("decode", "prefill", "acoustic", "frame", "codec", "matvec", "layer"), default="decode",
                    help="decode = the headline metric; prefill / acoustic = the other two configurations")
    ap.add_argument("--mode", type=int, default=0, choices=(0, 1), help="0 persistent kernel, 1 per-phase kernels")
    ap.add_argument("--prefill-mode", type=int, default=0, choices=(0, 1),
                    help="--workload prefill: 0 one launch per product and row pass, 1 one persistent launch per layer")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--no-workloads", action="store_true",
                    help="leave the short runs of the other configurations out of the default line")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain elementwise kernel (vt_add_kernel, a += b over 64 Mi floats: "
                         "512 MiB read, 256 MiB written) so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "can be scaled by a kernel of known traffic")
    ap.add_argument("--no-traffic", action="store_true",
                    help="do not measure the step kernel's HBM traffic with two rocprofv3 --pmc child runs "
                         "(roofline.traffic then comes from profiles/hbm_traffic.json)")
    ap.add_argument("--traffic-kib", type=float, default=None,
                    help="HBM bytes per launch measured with rocprofv3 --pmc (KiB), if known")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus above 1 is not supported "
                 "(batch-1 decode is one dependent chain of layers and is not sharded)")
    if args.workload == "prefill":
        return bench_prefill(args)
    if args.workload == "acoustic":
        return bench_acoustic(args)
    if args.workload == "codec":
        return bench_codec(args)
    if args.workload == "frame":
        return bench_frame(args)
    if args.workload == "matvec":
        return bench_matvec(args)
    if args.workload == "layer":
        return bench_layer(args)
    K, W = args.steps, args.warmup
    workers = min(16, os.cpu_count() or 8)

    # HBM traffic of the step kernel, before this process touches the GPU (not under a profiler: a run
    # that calibrates is one of the child runs itself, or somebody's own rocprofv3 command)
    live_traffic, live_source = None, None
    under_profiler = any(k.startswith("ROCP") for k in os.environ)
    if args.mode == 0 and args.traffic_kib is None and not (args.no_traffic or args.calibrate or under_profiler):
        live_traffic, live_source = live_decode_traffic()

    t0 = time.time()
    layers = make_layers(N_LAYERS, workers)
    final_norm = S.norm_weight(S.DIM, 99)
    proj = S.bf16_normal((S.DIM, S.DIM), 31337)
    ids = np.random.default_rng(7).integers(0, 131072, PROMPT)
    prompt = np.stack([emb_row(t) for t in ids]).astype(np.float32)
    t_gen = time.time() - t0

    n_cpu = 6 if args.cpu_seconds > 0 else 0
    kv_max = max(PROMPT + n_cpu + 2 * (W + K) + 8, PREFILL_LEN + 8)     # room for the 512-row workloads below
    if not args.no_workloads:
        kv_max = max(kv_max, 2008)                                      # and for the decode workload at 2000 positions
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
    BL().tts_hip_timer_start()
    run(K, True)
    ms_total = BL().tts_hip_timer_stop_ms()
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
    BL().tts_hip_timer_start()
    run(K, False)
    ms_kernel = BL().tts_hip_timer_stop_ms() / K
    lib.tts_hip_sync()
    hip.check()

    # what a grid of this shape can stream at all: the same grid, per-wave shares, loads and ring depth over the
    # same 26 layers of weights, with no arithmetic, staging or hand-overs
    nbytes_c = C.c_double(0.0)
    ms_ceiling = BL().tts_hip_bench_stream_ceiling(max(3, min(K, 20)), C.byref(nbytes_c))
    hip.check()

    # the drop-in entry point with host pointers (12 KB up, 12 KB down and one synchronisation per
    # step, as voxtral_tts_llm.c calls it): wall clock over the same positions, reported beside `value`
    pos = pos0
    e_host = d_e.to_numpy(np.float32, S.DIM)
    h_host = np.zeros(S.DIM, np.float32)
    n_host = min(K, 50)
    lib.tts_hip_llm_forward(h_host.ctypes.data, e_host.ctypes.data, pos)
    t0 = time.perf_counter()
    for i in range(n_host):
        lib.tts_hip_llm_forward(h_host.ctypes.data, e_host.ctypes.data, pos + i)
    ms_host = (time.perf_counter() - t0) * 1e3 / n_host
    hip.check()

    avg_pos = pos0 + (K - 1) / 2.0
    bytes_launch = step_bytes(avg_pos)
    achieved = bytes_launch / (ms_kernel * 1e-3) / 1e9
    traffic_source = TRAFFIC_SOURCE
    if args.traffic_kib is not None:
        traffic, traffic_source = args.traffic_kib * 1024.0, "--traffic-kib"
    elif live_traffic is not None:
        traffic, traffic_source = live_traffic, live_source
    else:
        traffic = measured_traffic("decode")
        if live_source:
            traffic_source += "; live measurement skipped: " + live_source
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
            "schedule": ("persistent whole-step kernel", "one kernel per phase")[args.mode],
        },
        "frames_per_s": round(1000.0 / ms_step, 1),
        "hbm_gbps": round((bytes_launch + 2 * S.DIM * S.DIM) / (ms_step * 1e-3) / 1e9, 1),
        "hbm_frac_of_peak": round((bytes_launch + 2 * S.DIM * S.DIM) / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "ms_per_frame_normalised_6p8GB": round(ms_kernel * 6.8e9 / bytes_launch, 4),
        "ms_per_frame_host_pointers": round(ms_host, 4),
        "roofline": {
            "kernel": ("vt_decode_step_kernel", "5 phase kernels per layer")[args.mode],
            "bound": "hbm",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "bytes_per_launch": int(bytes_launch),
            "ms_per_launch": round(ms_kernel, 4),
            "stream_ceiling_gbps": round(nbytes_c.value / ms_ceiling / 1e6, 1),
            "stream_ceiling_ms": round(ms_ceiling, 4),
            "frac_of_stream_ceiling": round(achieved / (nbytes_c.value / ms_ceiling / 1e6), 4),
            "stream_ceiling": "a plain streaming kernel with this kernel's grid, per-wave shares, 16-byte non-temporal "
                              "loads and 18 loads in flight per wave over the same 26 layers of weights",
        },
        "setup_s": {"generate": round(t_gen, 1), "upload": round(t_up, 1)},
    }
    if not args.no_workloads:
        out["workloads"] = other_workloads(hip, kv_max)
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
