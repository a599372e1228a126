"""Shared helpers for the test-suite: ctypes bindings of the CPU checker
libraries (oracle/liboracle.so, oracle/_ref/libvoxtral_ref.so), synthetic
weight generation and the comparison metrics.

The oracle is test infrastructure: it is only ever loaded from here (tests),
from the smoke check and from the benchmark's cpu_baseline leg.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

DIM, HEADS, KV_HEADS, HEAD_DIM = 3072, 32, 8, 128
Q_DIM, KV_DIM, FFN = 4096, 1024, 9216
EPS, THETA = 1e-5, 1000000.0
ACOUSTIC_DIM, SEM_PADDED, CODES = 36, 8320, 37

f32p = C.POINTER(C.c_float)
u16p = C.POINTER(C.c_uint16)
i32p = C.POINTER(C.c_int)
u64p = C.POINTER(C.c_uint64)


def fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(f32p)


def up(a):
    assert a.dtype == np.uint16 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(u16p)


def ip(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(i32p)


# --------------------------------------------------------------------------
# synthetic data
# --------------------------------------------------------------------------

def f32_to_bf16_trunc(a):
    """bf16 by truncation (bits >> 16), as the reference test does
    (test_kernels.c:68-76)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    return (a.view(np.uint32) >> 16).astype(np.uint16)


def bf16_to_f32(h):
    return (h.astype(np.uint32) << 16).view(np.float32)


def bf16_normal(shape, seed, std=0.02):
    g = np.random.default_rng(seed)
    return f32_to_bf16_trunc(g.standard_normal(shape, dtype=np.float32) * np.float32(std))


def f32_normal(shape, seed, std=1.0):
    g = np.random.default_rng(seed)
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def norm_weight(n, seed):
    """Positive RMSNorm gains |N(0,1)|*0.1+0.01 in the style of the reference
    test's fill_random_positive (test_kernels.c:62-66); O(1) after scaling so
    that hidden states stay O(1) through many layers."""
    g = np.random.default_rng(seed)
    return (np.abs(g.standard_normal(n, dtype=np.float32)) * np.float32(0.5)
            + np.float32(0.75)).astype(np.float32)


class Layer:
    """One transformer layer of synthetic weights (numpy, host)."""
    FIELDS = ("wq", "wk", "wv", "wo", "w1", "w2", "w3")
    SHAPES = dict(wq=(Q_DIM, DIM), wk=(KV_DIM, DIM), wv=(KV_DIM, DIM), wo=(DIM, Q_DIM),
                  w1=(FFN, DIM), w2=(DIM, FFN), w3=(FFN, DIM))

    def __init__(self, seed, std=0.02):
        for i, f in enumerate(self.FIELDS):
            setattr(self, f, bf16_normal(self.SHAPES[f], seed * 16 + i, std))
        self.attention_norm = norm_weight(DIM, seed * 16 + 8)
        self.ffn_norm = norm_weight(DIM, seed * 16 + 9)


class Acoustic:
    """Synthetic acoustic-transformer weights (numpy, host)."""

    def __init__(self, seed, n_layers=3, bias=True, std=0.02):
        self.n_layers = n_layers
        self.layers = [Layer(seed + 1 + i, std) for i in range(n_layers)]
        self.time_inv_freq = np.zeros(DIM // 2, np.float32)
        oracle().orc_default_time_inv_freq(fp(self.time_inv_freq), DIM // 2)
        self.input_proj = bf16_normal((DIM, ACOUSTIC_DIM), seed * 16 + 1, 0.2)
        self.time_proj = bf16_normal((DIM, DIM), seed * 16 + 2, std)
        self.llm_proj = bf16_normal((DIM, DIM), seed * 16 + 3, std)
        self.semantic_out = bf16_normal((SEM_PADDED, DIM), seed * 16 + 4, std)
        self.semantic_out_bias = f32_normal(SEM_PADDED, seed * 16 + 5, 0.1) if bias else None
        self.acoustic_out = bf16_normal((ACOUSTIC_DIM, DIM), seed * 16 + 6, std)
        self.norm = norm_weight(DIM, seed * 16 + 7)


# --------------------------------------------------------------------------
# oracle (our CPU restatement)
# --------------------------------------------------------------------------

class OrcLayer(C.Structure):
    _fields_ = [("wq", u16p), ("wk", u16p), ("wv", u16p), ("wo", u16p),
                ("attention_norm", f32p),
                ("w1", u16p), ("w2", u16p), ("w3", u16p),
                ("ffn_norm", f32p)]


class OrcAcoustic(C.Structure):
    _fields_ = [("time_inv_freq", f32p), ("input_proj", u16p), ("time_proj", u16p),
                ("llm_proj", u16p), ("semantic_out", u16p), ("semantic_out_bias", f32p),
                ("acoustic_out", u16p), ("norm", f32p),
                ("layers", C.POINTER(OrcLayer)), ("n_layers", C.c_int)]


_oracle = None
_ref = None


def _build_oracle():
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR, "liboracle.so"])


def oracle():
    global _oracle
    if _oracle is None:
        path = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(path):
            _build_oracle()
        lib = C.CDLL(path)
        lib.orc_randn.restype = C.c_float
        lib.orc_randn.argtypes = [u64p]
        lib.orc_get_threads.restype = C.c_int
        lib.orc_linear_bf16.argtypes = [f32p, f32p, u16p, f32p, C.c_int, C.c_int, C.c_int]
        lib.orc_rms_norm.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_float]
        lib.orc_compute_rope_freqs.argtypes = [f32p, i32p, C.c_int, C.c_int, C.c_float]
        lib.orc_apply_rope.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_int]
        lib.orc_causal_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5 + \
            [C.c_float, C.c_int, C.c_int]
        lib.orc_bidirectional_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 4 + \
            [C.c_float]
        lib.orc_llm_forward.argtypes = [C.POINTER(OrcLayer), C.c_int, f32p, f32p, f32p,
                                        C.c_int, C.c_int, f32p, f32p]
        lib.orc_llm_prefill.argtypes = [C.POINTER(OrcLayer), C.c_int, f32p, f32p,
                                        C.c_int, C.c_int, f32p, C.c_int, f32p]
        lib.orc_time_embedding.argtypes = [f32p, C.c_float, f32p, C.c_int]
        lib.orc_default_time_inv_freq.argtypes = [f32p, C.c_int]
        lib.orc_predict_velocity.argtypes = [C.POINTER(OrcAcoustic), f32p, f32p, C.c_float, f32p]
        lib.orc_acoustic_forward.argtypes = [C.POINTER(OrcAcoustic), f32p, u64p, i32p, f32p]
        lib.orc_audio_embed_forward.argtypes = [u16p, i32p, i32p, f32p, C.c_int]
        lib.orc_embed_token_bf16.argtypes = [f32p, u16p, C.c_int, C.c_int]
        lib.orc_silu.argtypes = [f32p, C.c_int]
        lib.orc_mul_inplace.argtypes = [f32p, f32p, C.c_int]
        lib.orc_add_inplace.argtypes = [f32p, f32p, C.c_int]
        lib.orc_rng_seed.argtypes = [u64p, C.c_uint64]
        lib.orc_randn_fill.argtypes = [u64p, f32p, C.c_int]
        lib.orc_set_threads.argtypes = [C.c_int]
        _oracle = lib
    return _oracle


def orc_layers(layers):
    """ctypes array of OrcLayer for a list of Layer (keeps numpy refs alive)."""
    arr = (OrcLayer * len(layers))()
    for i, l in enumerate(layers):
        arr[i] = OrcLayer(up(l.wq), up(l.wk), up(l.wv), up(l.wo), fp(l.attention_norm),
                          up(l.w1), up(l.w2), up(l.w3), fp(l.ffn_norm))
    arr._keep = layers
    return arr


def orc_acoustic(ac):
    larr = orc_layers(ac.layers)
    bias = fp(ac.semantic_out_bias) if ac.semantic_out_bias is not None else f32p()
    s = OrcAcoustic(fp(ac.time_inv_freq), up(ac.input_proj), up(ac.time_proj),
                    up(ac.llm_proj), up(ac.semantic_out), bias, up(ac.acoustic_out),
                    fp(ac.norm), larr, ac.n_layers)
    s._keep = (ac, larr)
    return s


# --------------------------------------------------------------------------
# the compiled reference (only where oracle/_ref was built)
# --------------------------------------------------------------------------

def ref_path():
    return os.path.join(ORACLE_DIR, "_ref", "libvoxtral_ref.so")


def have_ref():
    return os.path.exists(ref_path())


def ref():
    global _ref
    if _ref is None:
        lib = C.CDLL(ref_path())
        vp = C.c_void_p
        lib.ref_ctx_new.restype = vp
        lib.ref_ctx_new.argtypes = [C.c_int]
        lib.ref_ctx_free.argtypes = [vp]
        lib.ref_set_dec_layer.argtypes = [vp, C.c_int, u16p, u16p, u16p, u16p, f32p,
                                          u16p, u16p, u16p, f32p]
        lib.ref_set_ac_layer.argtypes = lib.ref_set_dec_layer.argtypes
        lib.ref_set_dec_norm.argtypes = [vp, f32p]
        lib.ref_set_acoustic.argtypes = [vp, f32p, u16p, u16p, u16p, u16p, f32p, u16p, f32p]
        lib.ref_kv_k.restype = f32p
        lib.ref_kv_k.argtypes = [vp]
        lib.ref_kv_v.restype = f32p
        lib.ref_kv_v.argtypes = [vp]
        lib.ref_get_kv_len.argtypes = [vp]
        lib.ref_set_kv_len.argtypes = [vp, C.c_int]
        lib.ref_seed.argtypes = [vp, C.c_uint64]
        lib.ref_rng_state.restype = C.c_uint64
        lib.ref_rng_state.argtypes = [vp]
        lib.ref_llm_forward.argtypes = [vp, f32p, f32p]
        lib.ref_llm_prefill.argtypes = [vp, f32p, C.c_int]
        lib.ref_acoustic_forward.argtypes = [vp, f32p, i32p]
        lib.ref_predict_velocity.argtypes = [vp, f32p, f32p, C.c_float, f32p]
        lib.ref_time_embedding.argtypes = [vp, C.c_float, f32p]
        lib.ref_audio_embed_set.argtypes = [vp, u16p]
        lib.ref_audio_embed_forward.argtypes = [vp, i32p, f32p]
        # the reference's own kernels, same signatures as the oracle's
        lib.tts_linear_bf16.argtypes = [f32p, f32p, u16p, f32p, C.c_int, C.c_int, C.c_int]
        lib.tts_linear_nobias_bf16.argtypes = [f32p, f32p, u16p, C.c_int, C.c_int, C.c_int]
        lib.tts_rms_norm.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_float]
        lib.tts_compute_rope_freqs.argtypes = [f32p, i32p, C.c_int, C.c_int, C.c_float]
        lib.tts_apply_rope.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_int]
        lib.tts_causal_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5 + \
            [C.c_float, C.c_int, C.c_int]
        lib.tts_bidirectional_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 4 + \
            [C.c_float]
        lib.tts_silu.argtypes = [f32p, C.c_int]
        lib.tts_mul_inplace.argtypes = [f32p, f32p, C.c_int]
        lib.tts_add_inplace.argtypes = [f32p, f32p, C.c_int]
        lib.tts_rng_seed.argtypes = [u64p, C.c_uint64]
        lib.tts_randn.restype = C.c_float
        lib.tts_randn.argtypes = [u64p]
        lib.tts_randn_fill.argtypes = [u64p, f32p, C.c_int]
        lib.tts_embed_token_bf16.argtypes = [f32p, u16p, C.c_int, C.c_int]
        _ref = lib
    return _ref


def ref_bind_decoder(ctx, layers, final_norm):
    """Point the reference ctx's 26 decoder layers at `layers`, cycling when
    fewer than 26 distinct layers are given (pointers may alias)."""
    r = ref()
    n = r.ref_dec_layers()
    for i in range(n):
        l = layers[i % len(layers)]
        r.ref_set_dec_layer(ctx, i, up(l.wq), up(l.wk), up(l.wv), up(l.wo),
                            fp(l.attention_norm), up(l.w1), up(l.w2), up(l.w3), fp(l.ffn_norm))
    r.ref_set_dec_norm(ctx, fp(final_norm))
    return n


def ref_bind_acoustic(ctx, ac):
    r = ref()
    assert ac.n_layers == r.ref_ac_layers()
    for i, l in enumerate(ac.layers):
        r.ref_set_ac_layer(ctx, i, up(l.wq), up(l.wk), up(l.wv), up(l.wo),
                           fp(l.attention_norm), up(l.w1), up(l.w2), up(l.w3), fp(l.ffn_norm))
    bias = fp(ac.semantic_out_bias) if ac.semantic_out_bias is not None else f32p()
    r.ref_set_acoustic(ctx, fp(ac.time_inv_freq), up(ac.input_proj), up(ac.time_proj),
                       up(ac.llm_proj), up(ac.semantic_out), bias, up(ac.acoustic_out),
                       fp(ac.norm))


# --------------------------------------------------------------------------
# comparison metrics
# --------------------------------------------------------------------------

def rel_errors(ref_v, test_v):
    """(max|d|/rms(ref), ||d||2/||ref||2) for one hidden-state vector."""
    ref_v = np.asarray(ref_v, np.float64).ravel()
    test_v = np.asarray(test_v, np.float64).ravel()
    d = test_v - ref_v
    rms = np.sqrt(np.mean(ref_v ** 2)) + 1e-30
    return float(np.max(np.abs(d)) / rms), float(np.linalg.norm(d) / (np.linalg.norm(ref_v) + 1e-30))


def compare_tensors(ref_v, test_v, rtol, atol):
    """The reference's rtol-OR-atol rule (test_kernels.c:79-116): an element
    is bad iff rel > rtol and |d| > atol; pass iff no bad element and
    (max_rel <= rtol or max_abs <= atol)."""
    ref_v = np.asarray(ref_v, np.float32).ravel()
    test_v = np.asarray(test_v, np.float32).ravel()
    diff = np.abs(ref_v - test_v)
    denom = np.maximum(np.abs(ref_v), np.float32(1e-8))
    rel = diff / denom
    n_bad = int(np.sum((rel > rtol) & (diff > atol)))
    ok = (rel.max() <= rtol or diff.max() <= atol) and n_bad == 0
    return bool(ok), float(rel.max()), float(diff.max()), n_bad
