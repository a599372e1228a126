"""Host-side Python mirror of the C ABI in include/voxtral_tts_hip.h.

The product is the shared library csrc/libvoxtral_tts_hip.so (hand-written HIP
for gfx950 behind `extern "C"` entry points named after the reference's
`tts_cuda_*` interface).  This module only loads it with ctypes and declares
the signatures; there is no CPU fallback: a missing library raises.

The directory name is not a Python identifier; load it with
`importlib` (see `load()` in tests/hipsupport.py or __graft_entry__.py).
"""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
# VOXTRAL_TTS_HIP_LIB selects another build of the same library (e.g. an instrumented one).
LIB_PATH = os.environ.get("VOXTRAL_TTS_HIP_LIB") or os.path.join(CSRC, "libvoxtral_tts_hip.so")

DEC_LAYERS = 26
AC_LAYERS = 3

f32p = C.POINTER(C.c_float)
u16p = C.POINTER(C.c_uint16)
i32p = C.POINTER(C.c_int)
vp = C.c_void_p


class HostLayer(C.Structure):
    """tts_hip_host_layer_t == tts_dec_layer_t / tts_ac_layer_t (voxtral_tts.h:101-114)."""
    _fields_ = [("wq_bf16", vp), ("wk_bf16", vp), ("wv_bf16", vp), ("wo_bf16", vp),
                ("attention_norm", vp),
                ("w1_bf16", vp), ("w2_bf16", vp), ("w3_bf16", vp),
                ("ffn_norm", vp)]


class HostDecoder(C.Structure):
    """tts_hip_host_decoder_t == tts_decoder_t (voxtral_tts.h:116-125)."""
    _fields_ = [("tok_embeddings_bf16", vp), ("layers", HostLayer * DEC_LAYERS), ("norm", vp)]


class HostAcoustic(C.Structure):
    """tts_hip_host_acoustic_t == tts_acoustic_t (voxtral_tts.h:146-165)."""
    _fields_ = [("time_inv_freq", vp), ("input_proj_bf16", vp), ("time_proj_bf16", vp),
                ("llm_proj_bf16", vp), ("semantic_out_bf16", vp), ("semantic_out_bias", vp),
                ("acoustic_out_bf16", vp), ("norm", vp), ("layers", HostLayer * AC_LAYERS)]


class HostConv(C.Structure):
    """tts_hip_host_conv_t == tts_conv_t (voxtral_tts.h:172-180)."""
    _fields_ = [("weight", vp), ("bias", vp), ("in_ch", C.c_int), ("out_ch", C.c_int),
                ("kernel", C.c_int), ("stride", C.c_int), ("is_transpose", C.c_int)]


class HostCodecLayer(C.Structure):
    """tts_hip_host_codec_layer_t == tts_codec_layer_t (voxtral_tts.h:183-205)."""
    _fields_ = [("wq", vp), ("wk", vp), ("wv", vp), ("wo", vp), ("q_norm", vp), ("k_norm", vp),
                ("attention_norm", vp), ("w1", vp), ("w2", vp), ("w3", vp), ("ffn_norm", vp),
                ("attn_scale", vp), ("ffn_scale", vp), ("window_size", C.c_int)]


class HostCodec(C.Structure):
    """tts_hip_host_codec_t == tts_codec_t (voxtral_tts.h:207-225)."""
    _fields_ = [("semantic_embedding", vp), ("input_conv", HostConv),
                ("transformers", HostCodecLayer * 8), ("stage_convs", HostConv * 4),
                ("output_proj", HostConv), ("alibi_slopes", C.c_float * 8)]


class HipCtx(C.Structure):
    """tts_hip_ctx_t (the exported global g_hip)."""
    _fields_ = [("kv_cache_k_gpu", vp), ("kv_cache_v_gpu", vp), ("kv_cache_max", C.c_int),
                ("initialized", C.c_int), ("n_cu", C.c_int), ("dec_layers_uploaded", C.c_int),
                ("ac_layers_uploaded", C.c_int)]


# name -> (restype, argtypes); every symbol include/voxtral_tts_hip.h declares
SIGNATURES = {
    "tts_hip_init": (C.c_int, [C.c_int]),
    "tts_hip_upload_llm_weights": (C.c_int, [vp]),
    "tts_hip_upload_acoustic_weights": (C.c_int, [vp]),
    "tts_hip_free": (None, []),
    "tts_hip_available": (C.c_int, []),
    "tts_hip_linear_bf16": (None, [vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "tts_hip_rms_norm": (None, [vp, vp, vp, C.c_int, C.c_int, C.c_float]),
    "tts_hip_apply_rope": (None, [vp, vp, C.c_int, C.c_int, C.c_int]),
    "tts_hip_compute_rope_freqs": (None, [vp, C.c_int, C.c_int, C.c_int, C.c_float]),
    "tts_hip_silu_mul": (None, [vp, vp, C.c_int]),
    "tts_hip_add_inplace": (None, [vp, vp, C.c_int]),
    "tts_hip_causal_attention_decode": (None, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.c_float, C.c_int]),
    "tts_hip_causal_attention_prefill": (None, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int,
                                                C.c_int, C.c_float]),
    "tts_hip_bidirectional_attention": (None, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.c_float]),
    "tts_hip_embed_token": (None, [vp, vp, C.c_int, C.c_int]),
    "tts_hip_llm_forward": (None, [vp, vp, C.c_int]),
    "tts_hip_llm_prefill": (None, [vp, C.c_int, C.c_int]),
    "tts_hip_predict_velocity": (None, [vp, vp, vp, C.c_float]),
    "tts_hip_to_device": (None, [vp, vp, C.c_size_t]),
    "tts_hip_to_host": (None, [vp, vp, C.c_size_t]),
    "tts_hip_memset": (None, [vp, C.c_int, C.c_size_t]),
    "tts_hip_alloc": (vp, [C.c_size_t]),
    "tts_hip_free_ptr": (None, [vp]),
    "tts_hip_sync": (None, []),
    "tts_hip_upload_llm_weights_n": (C.c_int, [vp, C.c_int]),
    "tts_hip_upload_llm_layer": (C.c_int, [C.c_int, C.POINTER(HostLayer)]),
    "tts_hip_upload_llm_norm": (C.c_int, [vp]),
    "tts_hip_llm_forward_device": (None, [vp, vp, C.c_int]),
    "tts_hip_layer_decode": (None, [C.c_int, vp, C.c_int]),
    "tts_hip_llm_prefill_out": (None, [vp, C.c_int, C.c_int, vp]),
    "tts_hip_predict_velocity_cfg": (None, [vp, vp, vp, vp, C.c_float]),
    "tts_hip_acoustic_frame": (None, [vp, vp, vp, vp]),
    "tts_hip_set_decode_mode": (None, [C.c_int]),
    "tts_hip_set_prefill_mode": (None, [C.c_int]),
    "tts_hip_error_count": (C.c_int, []),
    "tts_hip_last_error": (C.c_char_p, []),
    "tts_hip_split_planes": (C.c_int, [vp, vp, vp, C.c_size_t]),
    "tts_hip_upload_audio_embeddings": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "tts_hip_audio_embed": (None, [C.c_void_p, C.c_void_p]),
    "tts_hip_generate_frame": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]),
    "tts_hip_set_barrier_timeout": (None, [C.c_ulonglong]),
    "tts_hip_set_acoustic_grid": (None, [C.c_int]),
    "tts_hip_set_decode_grid": (None, [C.c_int]),
    "tts_hip_upload_codec_weights": (C.c_int, [vp]),
    "tts_hip_codec_decode": (None, [vp, C.c_int, C.POINTER(f32p), i32p]),
    "tts_hip_codec_decode_device": (C.c_int, [vp, C.c_int, vp]),
    "tts_hip_load_safetensors": (C.c_int, [C.c_char_p]),
    "tts_hip_linear_bf16_noalloc": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "tts_hip_default_time_inv_freq": (None, [vp, C.c_int]),
    "tts_hip_safetensors_probe": (C.c_int, [C.c_char_p, C.c_char_p, C.c_char_p, C.c_void_p,
                                            C.c_void_p, C.c_void_p]),
}

# every symbol include/voxtral_tts_hip_bench.h declares (csrc/libvoxtral_tts_hip_bench.so, the benchmark
# companion: timing loops around the product's own launches; links against the library above)
BENCH_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libvoxtral_tts_hip_bench.so")
BENCH_SIGNATURES = {
    "tts_hip_timer_start": (None, []),
    "tts_hip_timer_stop_ms": (C.c_float, []),
    "tts_hip_bench_kernel": (C.c_float, [C.c_int, C.c_int]),
    "tts_hip_bench_matvec": (C.c_float, [vp, vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int]),
    "tts_hip_bench_stream_ceiling": (C.c_float, [C.c_int, C.POINTER(C.c_double)]),
    "tts_hip_bench_fill_f32": (C.c_int, [vp, C.c_size_t]),
}

_lib = None
_bench_lib = None


def build(force=False):
    """Compile the library for gfx950 with hipcc (cross-compiles without a GPU)."""
    if force:
        subprocess.check_call(["make", "-s", "-C", CSRC, "clean"])
    subprocess.check_call(["make", "-s", "-j8", "-C", CSRC])
    return LIB_PATH


def lib():
    """The loaded C-ABI library with typed entry points.  Fails loudly if it
    has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built; run `make -C {CSRC}` "
                               "(or __graft_entry__.build())")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)          # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def bench_lib():
    """The benchmark companion library (shares the product library's context)."""
    global _bench_lib
    if _bench_lib is None:
        lib()                              # the product library first: the companion links against it
        if not os.path.exists(BENCH_LIB_PATH):
            raise RuntimeError(f"{BENCH_LIB_PATH} is not built; run `make -C {CSRC}`")
        l = C.CDLL(BENCH_LIB_PATH)
        for name, (res, args) in BENCH_SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _bench_lib = l
    return _bench_lib


def ctx():
    """The exported global context g_hip."""
    return HipCtx.in_dll(lib(), "g_hip")


class HipError(RuntimeError):
    pass


def check_errors(before):
    """Raise if the library recorded a failure since `before` (compute entry
    points are `void`, like the reference's)."""
    l = lib()
    n = l.tts_hip_error_count()
    if n != before:
        raise HipError(l.tts_hip_last_error().decode())
