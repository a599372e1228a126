"""Audio codec decoder on the device (tts_codec_decode, voxtral_tts_codec.c:389-503) against
the oracle, which is bit-equal to the compiled reference on these inputs
(tests/test_oracle_golden.py).  The device sums every dot product on the fp32 matrix cores in
another order than the CPU loop, so the bar is the floating-point one: max |d| / rms and
relative L2 of the waveform <= 1e-3."""
import ctypes as C

import numpy as np
import pytest

import codecsupport as K
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu

TOL = 1e-3


def hip_decode(hip, codes):
    codes = np.ascontiguousarray(codes, np.int32)
    out = S.f32p()
    n = C.c_int(0)
    hip.lib.tts_hip_codec_decode(codes.ctypes.data, codes.shape[0], C.byref(out), C.byref(n))
    hip.check()
    assert n.value == codes.shape[0] * K.UPSAMPLE * K.PATCH
    wave = np.ctypeslib.as_array(out, shape=(n.value,)).copy()
    C.CDLL(None).free(out)
    return wave


def check(ref, got):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    worst = float(np.abs(ref - got).max()) / rms
    l2 = float(np.linalg.norm((ref - got).astype(np.float64)) / np.linalg.norm(ref.astype(np.float64)))
    assert np.isfinite(got).all()
    assert worst <= TOL and l2 <= TOL, (worst, l2)
    return worst, l2


# runs before the module's session exists: the backend has one global context
def test_decode_without_weights_is_an_error():
    hip = H.Hip(kv_max=8)
    try:
        n0 = hip.lib.tts_hip_error_count()
        out = S.f32p()
        n = C.c_int(7)
        codes = K.random_codes(2, 1)
        hip.lib.tts_hip_codec_decode(codes.ctypes.data, 2, C.byref(out), C.byref(n))
        assert hip.lib.tts_hip_error_count() == n0 + 1
        assert not out and n.value == 0
    finally:
        hip.close()


@pytest.fixture(scope="module")
def session():
    S.oracle().orc_set_threads(16)
    hc = K.HostCodec(5)
    hip = H.Hip(kv_max=8)
    cs = hc.struct()
    rc = hip.lib.tts_hip_upload_codec_weights(C.addressof(cs))
    assert rc == 0, hip.lib.tts_hip_last_error()
    yield hip, cs
    hip.close()
    S.oracle().orc_set_threads(1)


@pytest.mark.parametrize("n_frames", [1, 2, 3, 17, 40])
def test_waveform_matches_the_oracle(session, n_frames):
    hip, cs = session
    codes = K.random_codes(n_frames, 100 + n_frames)
    ref = K.oracle_decode(cs, codes)
    got = hip_decode(hip, codes)
    worst, l2 = check(ref, got)
    print(f"n_frames {n_frames}: max|d|/rms {worst:.2e}, rel l2 {l2:.2e}")


@pytest.mark.timeout(900)
def test_waveform_of_a_200_frame_utterance_matches_the_oracle(session):
    """The size the benchmark times (16 s of audio; tts_codec_decode, voxtral_tts_codec.c:389-503): the
    200- and 400-row stages under-fill the product kernel's 128-row tiles and K is cut differently than
    at a few frames, so the whole utterance is compared, and every second of it on its own."""
    hip, cs = session
    n_frames = 200
    codes = K.random_codes(n_frames, 300)
    print("codec oracle on 200 frames ...", flush=True)
    ref = K.oracle_decode(cs, codes)
    got = hip_decode(hip, codes)
    assert got.size == n_frames * 1920
    worst, l2 = check(ref, got)
    per_s = 24000
    for i in range(0, ref.size, per_s):
        check(ref[i:i + per_s], got[i:i + per_s])
    print(f"n_frames {n_frames}: max|d|/rms {worst:.2e}, rel l2 {l2:.2e}")


def test_repeat_and_shrink_are_reproducible(session):
    hip, cs = session
    codes = K.random_codes(24, 7)
    a = hip_decode(hip, codes)
    b = hip_decode(hip, codes[:5])          # smaller call reuses the larger work buffers
    c = hip_decode(hip, codes)
    assert np.array_equal(a, c)
    check(K.oracle_decode(cs, codes[:5]), b)


def test_causality(session):
    """Frame t of the codes only moves samples from 1920 t on (every stage is causal)."""
    hip, _ = session
    codes = K.random_codes(12, 9, edge=False)
    a = hip_decode(hip, codes)
    codes2 = codes.copy()
    codes2[8:] = K.random_codes(4, 10, edge=False)
    b = hip_decode(hip, codes2)
    assert np.array_equal(a[:8 * 1920], b[:8 * 1920])
    assert not np.array_equal(a[8 * 1920:], b[8 * 1920:])


def test_device_entry_equals_host_entry(session):
    hip, _ = session
    codes = K.random_codes(9, 21)
    want = hip_decode(hip, codes)
    d_codes = H.DevBuf.from_numpy(hip.lib, codes)
    d_out = H.DevBuf(hip.lib, want.nbytes)
    assert hip.lib.tts_hip_codec_decode_device(d_codes.ptr, 9, d_out.ptr) == 0
    hip.lib.tts_hip_sync()
    assert np.array_equal(d_out.to_numpy(np.float32, want.shape), want)
    d_codes.free()
    d_out.free()


def test_optional_tensors_absent():
    """No q/k norm, no layer scale, no conv bias (the NULL branches of voxtral_tts_codec.c:
    329-333, 345-351, 366-372 and of the convolutions)."""
    S.oracle().orc_set_threads(16)
    hc = K.HostCodec(6, distinct_layers=2, qk_norm=False, layer_scale=False, bias=False)
    # without layer scale the residual stream grows; damp the output matrices instead
    for l in hc.layers[:2]:
        l.wo *= np.float32(0.3)
        l.w2 *= np.float32(0.3)
    cs = hc.struct()
    hip = H.Hip(kv_max=8)
    try:
        assert hip.lib.tts_hip_upload_codec_weights(C.addressof(cs)) == 0, hip.lib.tts_hip_last_error()
        codes = K.random_codes(6, 31)
        check(K.oracle_decode(cs, codes), hip_decode(hip, codes))
    finally:
        hip.close()
        S.oracle().orc_set_threads(1)


def test_wrong_convolution_shape_is_an_error():
    hc = K.HostCodec(7, distinct_layers=1)
    cs = hc.struct()
    cs.stage_convs[1].kernel = 3
    hip = H.Hip(kv_max=8)
    try:
        n0 = hip.lib.tts_hip_error_count()
        assert hip.lib.tts_hip_upload_codec_weights(C.addressof(cs)) == -1
        assert hip.lib.tts_hip_error_count() == n0 + 1
        assert b"convolution 1" in hip.lib.tts_hip_last_error()
    finally:
        hip.close()
