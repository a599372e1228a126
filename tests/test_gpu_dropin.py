"""Drop-in proof on the GPU: the reference's UNMODIFIED host files, compiled
with -DUSE_CUDA against this library through include/compat/voxtral_tts_cuda.h
(oracle/Makefile target `dropin`, built where the reference tree is mounted),
drive the gfx950 backend:

  * the reference's own kernel test harness (test_kernels.c) with its own
    tolerances;
  * voxtral_tts_llm.c: CPU prefill + KV upload through g_cuda + GPU decode;
  * voxtral_tts_acoustic.c: the frame loop on the host with predict_velocity
    dispatched to the GPU.
"""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu

REF_DIR = os.path.join(S.ORACLE_DIR, "_ref")
HARNESS = os.path.join(REF_DIR, "test_kernels_hip")
DROPIN = os.path.join(REF_DIR, "libvoxtral_dropin.so")


@pytest.mark.skipif(not os.path.exists(HARNESS), reason="drop-in harness not built")
def test_reference_kernel_harness_passes_against_this_backend():
    r = subprocess.run([HARNESS], capture_output=True, text=True, timeout=170)
    print(r.stdout[-3000:], r.stderr[-1000:])
    assert r.returncode == 0
    assert "GPU initialized successfully" in r.stdout
    assert "11/11 passed, 0 failed" in r.stdout
    assert "cpu-self" not in r.stdout          # every case compared CPU vs GPU


def _dropin():
    lib = C.CDLL(DROPIN)
    vp = C.c_void_p
    lib.ref_ctx_new.restype = vp
    lib.ref_ctx_new.argtypes = [C.c_int]
    for n in ("ref_decoder_ptr", "ref_acoustic_ptr"):
        getattr(lib, n).restype = vp
        getattr(lib, n).argtypes = [vp]
    lib.ref_set_dec_layer.argtypes = [vp, C.c_int, S.u16p, S.u16p, S.u16p, S.u16p, S.f32p,
                                      S.u16p, S.u16p, S.u16p, S.f32p]
    lib.ref_set_ac_layer.argtypes = lib.ref_set_dec_layer.argtypes
    lib.ref_set_dec_norm.argtypes = [vp, S.f32p]
    lib.ref_set_acoustic.argtypes = [vp, S.f32p, S.u16p, S.u16p, S.u16p, S.u16p, S.f32p, S.u16p, S.f32p]
    lib.ref_llm_forward.argtypes = [vp, S.f32p, S.f32p]
    lib.ref_llm_prefill.argtypes = [vp, S.f32p, C.c_int]
    lib.ref_acoustic_forward.argtypes = [vp, S.f32p, S.i32p]
    lib.ref_seed.argtypes = [vp, C.c_uint64]
    lib.ref_ctx_free.argtypes = [vp]
    lib.ref_get_kv_len.argtypes = [vp]
    return lib


@pytest.mark.skipif(not os.path.exists(DROPIN), reason="drop-in library not built")
def test_unmodified_llm_host_code_decodes_on_the_gpu():
    gold = np.load(os.path.join(S.GOLDEN_DIR, "llm.npz"))
    d = _dropin()
    layers = [S.Layer(1), S.Layer(2)]
    norm = S.norm_weight(S.DIM, 99)
    hip = H.Hip(kv_max=cases.KV_MAX)             # tts_hip_init, as voxtral_tts.c:96 does
    ctx = d.ref_ctx_new(cases.KV_MAX)
    try:
        for i in range(26):
            l = layers[i % 2]
            d.ref_set_dec_layer(ctx, i, S.up(l.wq), S.up(l.wk), S.up(l.wv), S.up(l.wo),
                                S.fp(l.attention_norm), S.up(l.w1), S.up(l.w2), S.up(l.w3),
                                S.fp(l.ffn_norm))
        d.ref_set_dec_norm(ctx, S.fp(norm))
        assert hip.lib.tts_hip_upload_llm_weights(d.ref_decoder_ptr(ctx)) == 0
        emb = S.f32_normal((3, S.DIM), 5)
        d.ref_llm_prefill(ctx, S.fp(emb), 3)      # CPU prefill, then the whole KV cache goes up
        e = S.f32_normal(S.DIM, 6)
        for step in range(2):
            h = np.zeros(S.DIM, np.float32)
            d.ref_llm_forward(ctx, S.fp(e), S.fp(h))          # -> tts_hip_llm_forward
            mx, l2 = S.rel_errors(gold["hidden"][step], h)
            assert mx < 1e-3 and l2 < 1e-3, (step, mx, l2)
            e = gold["hidden"][step].copy()
        assert d.ref_get_kv_len(ctx) == 5
        hip.check()
    finally:
        d.ref_ctx_free(ctx)
        hip.close()


@pytest.mark.skipif(not os.path.exists(DROPIN), reason="drop-in library not built")
def test_unmodified_acoustic_host_code_samples_identical_codes():
    gold = np.load(os.path.join(S.GOLDEN_DIR, "acoustic.npz"))
    d = _dropin()
    ac = S.Acoustic(50)
    hip = H.Hip(kv_max=8)
    ctx = d.ref_ctx_new(0)
    try:
        for i, l in enumerate(ac.layers):
            d.ref_set_ac_layer(ctx, i, S.up(l.wq), S.up(l.wk), S.up(l.wv), S.up(l.wo),
                               S.fp(l.attention_norm), S.up(l.w1), S.up(l.w2), S.up(l.w3),
                               S.fp(l.ffn_norm))
        d.ref_set_acoustic(ctx, S.fp(ac.time_inv_freq), S.up(ac.input_proj), S.up(ac.time_proj),
                           S.up(ac.llm_proj), S.up(ac.semantic_out), S.fp(ac.semantic_out_bias),
                           S.up(ac.acoustic_out), S.fp(ac.norm))
        assert hip.lib.tts_hip_upload_acoustic_weights(d.ref_acoustic_ptr(ctx)) == 0
        d.ref_seed(ctx, 42)
        for f in range(gold["codes"].shape[0]):
            codes = np.zeros(S.CODES, np.int32)
            d.ref_acoustic_forward(ctx, S.fp(S.f32_normal(S.DIM, 20 + f)), S.ip(codes))
            assert np.array_equal(codes, gold["codes"][f]), (f, codes, gold["codes"][f])
        hip.check()
    finally:
        d.ref_ctx_free(ctx)
        hip.close()
