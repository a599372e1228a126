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


def test_generation_loop_matches_the_oracle_chain(session):
    """Three turns of the loop from one start embedding.  Noise comes from the host RNG
    restated by the oracle (the reference draws it on the host).  Codes must be equal frame by
    frame (a differing FSQ code is tolerated only where the oracle's latent sits within fp32
    noise of a rounding boundary), and then the next embedding is bit-equal."""
    hip, orc, table = session
    st = C.c_uint64(0)
    S.oracle().orc_rng_seed(C.byref(st), 7)
    e = S.f32_normal(S.DIM, 77)
    d_e = H.DevBuf.from_numpy(hip.lib, e)
    hip.pos = 0
    orc.pos = 0
    for frame in range(3):
        h = orc.llm_forward(e)
        rc, _, rx = orc.acoustic_forward(h, seed=7 if frame == 0 else None, want_x=True)
        x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
        S.oracle().orc_randn_fill(C.byref(st), S.fp(x0), S.ACOUSTIC_DIM)
        codes = np.zeros(S.CODES, np.int32)
        hip.lib.tts_hip_generate_frame(codes.ctypes.data, d_e.ptr, x0.ctypes.data, frame)
        hip.check()
        assert codes[0] == rc[0], (frame, codes[0], rc[0])
        for i in np.nonzero(codes[1:] != rc[1:])[0]:
            scaled = (np.clip(rx[i], -1, 1) + 1.0) / 2.0 * 20.0 + 0.5
            assert abs(scaled - round(scaled)) < 1e-3, (frame, i, scaled)
        if not np.array_equal(codes, rc):
            pytest.skip("a code sat on an FSQ rounding boundary; the chains diverge by design from here")
        e = orc.audio_embed(table, rc)
        assert np.array_equal(d_e.to_numpy(np.float32, S.DIM), e), frame
