"""Prefill and acoustic-transformer parity on the GPU against the oracle and
the reference-written fixtures."""
import ctypes as C
import os

import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu
TOL = 1e-3


def assert_close(ref, got, what, tol=TOL):
    mx, l2 = S.rel_errors(ref, got)
    assert np.all(np.isfinite(got)), what
    assert mx < tol and l2 < tol, (what, mx, l2)


def test_prefill_two_chunks_then_decode():
    layers = [S.Layer(1), S.Layer(2)]
    norm = S.norm_weight(S.DIM, 99)
    n_layers, s1, s2 = 3, 24, 5
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, 40, n_layers=n_layers)
    hip = H.Hip(kv_max=40)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        e1, e2 = S.f32_normal((s1, S.DIM), 5), S.f32_normal((s2, S.DIM), 6)
        for e in (e1, e2):
            rx = orc.llm_prefill(e, want_x=True)
            gx = hip.llm_prefill(e, want_x=True)
            for r in range(e.shape[0]):
                assert_close(rx[r], gx[r], f"prefill residual row {r}")
        gk, gv = hip.kv()
        n = s1 + s2
        for l in range(n_layers):
            for r in range(n):
                assert_close(orc.kv_k[l, r], gk[l, r], f"k l{l} r{r}")
                assert_close(orc.kv_v[l, r], gv[l, r], f"v l{l} r{r}")
        x = S.f32_normal(S.DIM, 7)
        assert_close(orc.llm_forward(x), hip.llm_forward(x), "decode after prefill")
    finally:
        hip.close()


def test_prefill_outside_cache_is_an_error():
    hip = H.Hip(kv_max=8)
    try:
        hip.upload_decoder([S.Layer(1)], np.ones(S.DIM, np.float32), 1)
        e = S.f32_normal((6, S.DIM), 5)
        n0 = hip.lib.tts_hip_error_count()
        hip.lib.tts_hip_llm_prefill(e.ctypes.data, 6, 4)
        assert hip.lib.tts_hip_error_count() == n0 + 1
    finally:
        hip.close()


@pytest.fixture(scope="module")
def ac_session():
    ac = S.Acoustic(50)
    hip = H.Hip(kv_max=8)
    hip.upload_acoustic(ac)
    orc = cases.OracleBackend(threads=16)
    orc.ac_open(ac)
    yield hip, orc, ac
    hip.close()


def test_predict_velocity_against_reference_fixture(ac_session):
    hip, orc, ac = ac_session
    gold = np.load(os.path.join(S.GOLDEN_DIR, "acoustic.npz"))
    x = S.f32_normal(S.ACOUSTIC_DIM, 11)
    h = S.f32_normal(S.DIM, 12)
    t = np.float32(3) / np.float32(7)
    assert_close(gold["vel_cond"], hip.predict_velocity(x, h, t), "cond")
    assert_close(gold["vel_uncond"], hip.predict_velocity(x, np.zeros(S.DIM, np.float32), t), "uncond")
    vc, vu = hip.predict_velocity_cfg(x, h, t)
    assert_close(gold["vel_cond"], vc, "cfg cond")
    assert_close(gold["vel_uncond"], vu, "cfg uncond")


def test_velocity_memo_follows_the_reference_call_pattern(ac_session):
    """The host file asks for cond then uncond (zero hidden) velocity per Euler step
    (voxtral_tts_acoustic.c:345-348).  The second call is answered from the batch of the
    first; it must equal what a fresh pass gives, also for off-grid times, and a changed
    latent or time must not be served from the memo."""
    hip, orc, ac = ac_session
    zeros = np.zeros(S.DIM, np.float32)
    for t in (np.float32(2) / np.float32(7), np.float32(0.3)):
        x = S.f32_normal(S.ACOUSTIC_DIM, 61)
        h = S.f32_normal(S.DIM, 62)
        vc = hip.predict_velocity(x, h, t)
        vu = hip.predict_velocity(x, zeros, t)             # memo
        fc, fu = hip.predict_velocity_cfg(x, h, t)         # fresh pass, both branches
        assert np.array_equal(vc, fc) and np.array_equal(vu, fu)
        assert_close(orc.predict_velocity(x, h, t), vc, "cond vs oracle")
        assert_close(orc.predict_velocity(x, zeros, t), vu, "uncond vs oracle")
        x2 = S.f32_normal(S.ACOUSTIC_DIM, 63)
        vu2 = hip.predict_velocity(x2, zeros, t)           # other latent: computed, not remembered
        assert_close(orc.predict_velocity(x2, zeros, t), vu2, "uncond, new latent")
        assert not np.array_equal(vu2, vu)


def test_acoustic_frames_codes_bit_exact(ac_session):
    """Sampled codes at a fixed seed: noise comes from the host RNG restated by
    the oracle (the reference draws it on the host too), the frame runs on the
    GPU; all 37 codes of every frame must equal the reference fixture's."""
    hip, orc, ac = ac_session
    gold = np.load(os.path.join(S.GOLDEN_DIR, "acoustic.npz"))
    st = C.c_uint64(0)
    S.oracle().orc_rng_seed(C.byref(st), 42)
    for f in range(gold["codes"].shape[0]):
        h = S.f32_normal(S.DIM, 20 + f)
        x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
        S.oracle().orc_randn_fill(C.byref(st), S.fp(x0), S.ACOUSTIC_DIM)
        codes, x = hip.acoustic_frame(h, x0)
        assert np.array_equal(codes, gold["codes"][f]), (f, codes, gold["codes"][f])
        assert int(st.value) == int(gold["rng_states"][f])


def test_more_frames_against_oracle_with_margins(ac_session):
    """Extra frames against the oracle; a code may only differ where the
    oracle's latent sits within fp32 noise of an FSQ decision boundary."""
    hip, orc, ac = ac_session
    mism = 0
    for f in range(3):
        h = S.f32_normal(S.DIM, 120 + f)
        rc, rst, rx = orc.acoustic_forward(h, seed=1000 + f, want_x=True)
        st = C.c_uint64(0)
        S.oracle().orc_rng_seed(C.byref(st), 1000 + f)
        x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
        S.oracle().orc_randn_fill(C.byref(st), S.fp(x0), S.ACOUSTIC_DIM)
        codes, x = hip.acoustic_frame(h, x0)
        assert codes[0] == rc[0]
        assert np.max(np.abs(x - rx)) < 1e-4, np.max(np.abs(x - rx))
        for i in np.nonzero(codes[1:] != rc[1:])[0]:
            # one level apart, and only where the oracle's latent is within the latent's noise bound
            # (1e-4, above; x 10 in the scaled units of the rounding) of a boundary
            scaled = (np.clip(np.float64(rx[i]), -1, 1) + 1.0) / 2.0 * 20.0 + 0.5
            assert abs(int(codes[1 + i]) - int(rc[1 + i])) == 1, (f, i, codes[1 + i], rc[1 + i])
            assert abs(scaled - round(scaled)) < 1e-3, (f, i, scaled)
            mism += 1
    assert mism <= 1


def test_frame_does_not_depend_on_the_acoustic_grid(ac_session):
    """On a smaller grid a workgroup of the product kernels walks more units: other loop tails (one,
    two or three units left), parked partial sums flushed in between.  A unit is summed the same way
    whichever workgroup takes it, so latent and codes are the same bit for bit."""
    hip, orc, ac = ac_session
    h, x0 = S.f32_normal(S.DIM, 77), S.f32_normal(S.ACOUSTIC_DIM, 78)
    ref_codes, ref_x = hip.acoustic_frame(h, x0)
    try:
        for grid in (100, 37, 7):
            hip.lib.tts_hip_set_acoustic_grid(grid)
            codes, x = hip.acoustic_frame(h, x0)
            hip.check()
            assert np.array_equal(codes, ref_codes), grid
            assert np.array_equal(x.view(np.uint32), ref_x.view(np.uint32)), grid
        hip.lib.tts_hip_set_acoustic_grid(100000)
        assert "tts_hip_set_acoustic_grid" in hip.lib.tts_hip_last_error().decode()
        hip.err0 = hip.lib.tts_hip_error_count()          # that failure was asked for
    finally:
        hip.lib.tts_hip_set_acoustic_grid(0)


def test_end_audio_frame(ac_session):
    hip, orc, ac = ac_session
    ac2 = S.Acoustic(50)
    ac2.semantic_out_bias = ac2.semantic_out_bias.copy()
    ac2.semantic_out_bias[1] = 1e9
    hip.upload_acoustic(ac2)
    codes, x = hip.acoustic_frame(S.f32_normal(S.DIM, 30), np.zeros(S.ACOUSTIC_DIM, np.float32))
    assert codes[0] == 1 and np.all(codes[1:] == 2)
    hip.upload_acoustic(ac)


def test_single_kernel_timing_modes(ac_session):
    """The event-timed launches bench.py prices its roofline on: each acoustic phase
    alone (10..13) and the four of a layer in order (14) return a positive time, the
    in-order figure lies between the largest phase and a generous multiple of their
    sum, and an unknown selector is an error, not a launch."""
    hip, orc, ac = ac_session
    alone = [hip.pkg.bench_lib().tts_hip_bench_kernel(w, 5) for w in (10, 11, 12, 13)]
    layer = hip.pkg.bench_lib().tts_hip_bench_kernel(14, 5)
    hip.check()
    assert all(0.0 < a < 1.0 for a in alone), alone
    assert max(alone) < layer < 3.0 * sum(alone), (alone, layer)
    n0 = hip.lib.tts_hip_error_count()
    assert hip.pkg.bench_lib().tts_hip_bench_kernel(15, 5) < 0
    assert hip.pkg.bench_lib().tts_hip_bench_kernel(14, 0) < 0
    assert hip.lib.tts_hip_error_count() == n0 + 2
    hip.err0 = n0 + 2                                      # the two errors above were asked for
    # the frame still runs after the timing loops used the same work buffers
    gold = np.load(os.path.join(S.GOLDEN_DIR, "acoustic.npz"))
    st = C.c_uint64(0)
    S.oracle().orc_rng_seed(C.byref(st), 42)
    x0 = np.zeros(S.ACOUSTIC_DIM, np.float32)
    S.oracle().orc_randn_fill(C.byref(st), S.fp(x0), S.ACOUSTIC_DIM)
    codes, _ = hip.acoustic_frame(S.f32_normal(S.DIM, 20), x0)
    assert np.array_equal(codes, gold["codes"][0])
