"""bench.py's command line contract that needs no GPU: more than one GPU is refused with a message
(this path runs on one GPU), the workloads of BASELINE.json's configs are all selectable, and the
byte / flop accounting behind the roofline figures matches the numbers derived from the model's
shapes (voxtral_tts.h:19-44)."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""                     # no JSON line for a run that did not happen


def test_every_config_has_a_workload():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0
    for w in ("decode", "matvec", "layer", "prefill", "acoustic", "frame", "codec"):
        assert w in r.stdout, w


def test_algorithmic_bytes_and_flops():
    b = load_bench()
    dim, q, kv, ffn, layers = 3072, 4096, 1024, 9216, 26
    per_layer = 2 * (dim * (q + 2 * kv) + q * dim + 3 * ffn * dim)
    assert per_layer == 232_783_872 == b.LAYER_WEIGHT_BYTES
    pos = 100
    want = (layers * per_layer + (2 * layers + 1) * dim * 4 + layers * 2 * (pos + 1) * kv * 4
            + layers * 2 * kv * 4 + 2 * dim * 4)
    assert b.step_bytes(pos) == want
    gemm, attn = b.prefill_flops(512)
    assert gemm == 2 * 512 * (per_layer // 2) * layers
    assert attn == 4 * 128 * 32 * (512 * 513 // 2) * layers
