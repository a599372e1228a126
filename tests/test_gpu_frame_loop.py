"""The per-frame generation loop on the device (voxtral_tts.c:301-321): backbone step ->
acoustic frame -> audio-code embedding of the 37 codes as the next backbone input, against
the oracle's chain of the same three functions.  The embedding is an ordered fp32 sum of 37
bf16 rows and must be bit-equal (tts_audio_embed_forward, voxtral_tts_voice.c:292-315)."""
import ctypes as C

import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu

AUDIO_ROWS = 8194 + 36 * 23


def offsets():
    offs = np.zeros(S.CODES, np.int32)
    offs[1] = 8194
    for i in range(2, S.CODES):
        offs[i] = offs[i - 1] + 23
    return offs


def random_codes(seed):
    r = np.random.default_rng(seed)
    c = np.zeros(S.CODES, np.int32)
    c[0] = r.integers(2, 8194)
    c[1:] = r.integers(2, 23, S.CODES - 1)
    return c


# runs before the module's session exists: the backend has one global context
def test_embed_without_table_is_an_error():
    hip = H.Hip(kv_max=8)
    try:
        n0 = hip.lib.tts_hip_error_count()
        out = np.zeros(S.DIM, np.float32)
        hip.lib.tts_hip_audio_embed(out.ctypes.data, random_codes(1).ctypes.data)
        assert hip.lib.tts_hip_error_count() == n0 + 1
    finally:
        hip.close()


@pytest.fixture(scope="module")
def session():
    table = S.bf16_normal((AUDIO_ROWS, S.DIM), 4242, 0.05)
    ac = S.Acoustic(50)
    layers = [S.Layer(1), S.Layer(2)]
    norm = S.norm_weight(S.DIM, 99)
    hip = H.Hip(kv_max=16)
    hip.upload_decoder(layers, norm, 2)
    hip.upload_acoustic(ac)
    rc = hip.lib.tts_hip_upload_audio_embeddings(table.ctypes.data, AUDIO_ROWS, offsets().ctypes.data)
    assert rc == 0, hip.lib.tts_hip_last_error()
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, 16, n_layers=2)
    orc.ac_open(ac)
    yield hip, orc, table
    hip.close()


def test_audio_embed_bit_exact(session):
    hip, orc, table = session
    for seed in (1, 2, 3):
        codes = random_codes(seed)
        got = np.zeros(S.DIM, np.float32)
        hip.lib.tts_hip_audio_embed(got.ctypes.data, codes.ctypes.data)
        hip.check()
        assert np.array_equal(got, orc.audio_embed(table, codes))
    # the extreme rows of every codebook
    lo = np.full(S.CODES, 0, np.int32)
    hi = np.full(S.CODES, 22, np.int32)
    hi[0] = 8193
    for codes in (lo, hi):
        got = np.zeros(S.DIM, np.float32)
        hip.lib.tts_hip_audio_embed(got.ctypes.data, codes.ctypes.data)
        assert np.array_equal(got, orc.audio_embed(table, codes))


# scaled units of the FSQ rounding (21 levels over [-1, 1]): 10 x the bound of 1e-4 on the latent's
# accumulated fp32 noise that tests/test_gpu_fullsize.py holds over 200 frames (measured 5.9e-5)
FSQ_NOISE = 1e-3


def fsq_margin(x):
    """Distance of the oracle's latent from the nearest FSQ rounding boundary, in the scaled
    units of `(int)((x + 1) / 2 * 20 + 0.5)` (voxtral_tts_acoustic.c:356-366), in float64."""
    scaled = (np.clip(np.float64(x), -1.0, 1.0) + 1.0) / 2.0 * 20.0 + 0.5
    return abs(scaled - round(scaled))


def test_generation_loop_matches_the_oracle_chain(session):
    """Three turns of the loop from one start embedding.  Noise comes from the host RNG
    restated by the oracle (the reference draws it on the host).  Codes must be equal frame by
    frame, and then the next embedding is bit-equal.  A differing FSQ code is accepted only where
    the oracle's latent sits within fp32 noise of a rounding boundary; the two chains then feed
    different embeddings, so the comparison ends there, with that assertion."""
    hip, orc, table = session
    st = C.c_uint64(0)
    S.oracle().orc_rng_seed(C.byref(st), 7)
    e = S.f32_normal(S.DIM, 77)
    d_e = H.DevBuf.from_numpy(hip.lib, e)
    hip.pos = 0
    orc.pos = 0
    compared = 0
    for frame in range(3):
        h = orc.llm_forward(e)
        rc, _, rx = orc.acoustic_forward(h, seed=7 if frame == 0 else None, want_x=True)
        x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
        S.oracle().orc_randn_fill(C.byref(st), S.fp(x0), S.ACOUSTIC_DIM)
        codes = np.zeros(S.CODES, np.int32)
        hip.lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, x0.ctypes.data, frame)
        hip.check()
        compared += 1
        assert codes[0] == rc[0], (frame, codes[0], rc[0])
        differing = np.nonzero(codes[1:] != rc[1:])[0]
        for i in differing:
            assert abs(int(codes[1 + i]) - int(rc[1 + i])) == 1, (frame, i, codes[1 + i], rc[1 + i])
            assert fsq_margin(rx[i]) < FSQ_NOISE, (frame, i, fsq_margin(rx[i]))
        if len(differing):
            break
        e = orc.audio_embed(table, rc)
        assert np.array_equal(d_e.to_numpy(np.float32, S.DIM), e), frame
    assert compared >= 1


def test_abandoned_backbone_step_fails_the_frame(session):
    """A barrier budget of one tick (a host-side setting; every kernel still runs to its end)
    makes the backbone step of tts_hip_generate_frame leave early: the call reports it, hands no
    codes back, and the next call with the default budget runs clean."""
    hip, orc, table = session
    lib = hip.lib
    e = S.f32_normal(S.DIM, 78)
    d_e = H.DevBuf.from_numpy(lib, e)
    x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
    codes = np.full(S.CODES, -7, np.int32)
    n0 = lib.tts_hip_error_count()
    lib.tts_hip_set_barrier_timeout(1)
    try:
        lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, x0.ctypes.data, 0)
    finally:
        lib.tts_hip_set_barrier_timeout(0)
    assert lib.tts_hip_error_count() == n0 + 1
    assert b"barrier timed out" in lib.tts_hip_last_error()
    assert np.all(codes == -7)
    hip.err0 = lib.tts_hip_error_count()
    # the same turn again, clean: the codes are those of the oracle's chain from this embedding
    lib.tts_hip_to_device(d_e.ptr, e.ctypes.data, e.nbytes)
    lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, x0.ctypes.data, 0)
    hip.check()
    orc.pos = 0
    h = orc.llm_forward(e)
    ref_codes, ref_x = hip.acoustic_frame(h, x0)      # the frame kernels on the oracle's hidden state
    assert codes[0] == ref_codes[0], (codes, ref_codes)
    # the two hidden states differ by the backbone's summation noise: a code may differ by one level, and
    # only where the latent lies on a rounding boundary (the rule of test_generation_loop above)
    for i in np.nonzero(codes[1:] != ref_codes[1:])[0]:
        assert abs(int(codes[1 + i]) - int(ref_codes[1 + i])) == 1, (i, codes[1 + i], ref_codes[1 + i])
        assert fsq_margin(ref_x[i]) < FSQ_NOISE, (i, fsq_margin(ref_x[i]))
