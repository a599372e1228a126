"""Shared helpers for the test-suite: ctypes bindings of the CPU checker
libraries (oracle/liboracle.so, oracle/_ref/libvoxtral_ref.so), synthetic
weight generation and the comparison metrics.

The oracle is test infrastructure: it is only ever loaded from here (tests),
from the smoke check and from the benchmark's cpu_baseline leg.
"""
import ctypes as C
import importlib.util
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

PKG_DIR = os.path.join(ROOT, "voxtral-tts.c_amd")


def load_package():
    """Import the package directory (its name is not a Python identifier)."""
    name = "voxtral_tts_c_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


load_package()
from voxtral_tts_c_amd import synth as _synth  # noqa: E402
from voxtral_tts_c_amd.synth import (  # noqa: E402,F401  (the seeded generators and metrics, shared with bench.py)
    DIM, HEADS, KV_HEADS, HEAD_DIM, Q_DIM, KV_DIM, FFN, EPS, THETA, ACOUSTIC_DIM, SEM_PADDED, CODES,
    f32_to_bf16_trunc, bf16_to_f32, bf16_normal, f32_normal, norm_weight, Layer, rel_errors, compare_tensors)

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


class Acoustic(_synth.Acoustic):
    """Synthetic acoustic-transformer weights whose time-embedding table is the oracle's
    (orc_default_time_inv_freq), so that oracle, compiled reference and GPU get the same one."""

    def __init__(self, seed, n_layers=3, bias=True, std=0.02):
        t = np.zeros(DIM // 2, np.float32)
        oracle().orc_default_time_inv_freq(fp(t), DIM // 2)
        super().__init__(seed, n_layers, bias, std, time_inv_freq=t)


