"""Backbone decode parity on the GPU against the oracle (and, through the
committed fixtures, against the compiled reference): one layer with a 512-row
cache (config 2), several layers, the 26-layer step, both launch schedules."""
import os

import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu
TOL = 1e-3          # max |d| / rms(ref) and ||d||/||ref|| per hidden state (north-star bound)


def assert_close(ref, got, what, tol=TOL):
    mx, l2 = S.rel_errors(ref, got)
    assert np.all(np.isfinite(got)), what
    assert mx < tol and l2 < tol, (what, mx, l2)
    return mx, l2


@pytest.mark.parametrize("pos", [4100, 1800, 1100, 1024, 768, 576, 575, 512, 384, 383, 300, 129, 128, 33, 1])
def test_one_layer_decode_with_cached_positions(pos):
    """Config 2: one layer, batch 1, KV cache of 512 positions ~N(0,1), hidden ~N(0,1), pos = 512.
    Caches of up to 383 positions take the attention schedule with one workgroup per query head
    (in batches of 128); from 384 / 576 positions on a head's positions are dealt to 2 / 8
    workgroups whose partials the output projection combines (1024 and 1100: one and two batches
    of requests per workgroup); from 4096 on the chunked schedule
    with its last-arriver merge runs (4100: the chunk count is at its cap of three quarters of the
    grid)."""
    kv_max = pos + 8
    layer = S.Layer(3)
    ones = np.ones(S.DIM, np.float32)
    k = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    v = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    k[0, :pos] = S.f32_normal((pos, S.KV_DIM), 200)
    v[0, :pos] = S.f32_normal((pos, S.KV_DIM), 300)
    x = S.f32_normal(S.DIM, 42)

    # oracle: one layer + final norm with unit gains == rmsnorm(x_out) ; compare the residual itself
    orc = cases.OracleBackend(threads=16)
    orc.llm_open([layer], ones, kv_max, n_layers=1)
    orc.kv_k[0], orc.kv_v[0] = k[0], v[0]
    orc.pos = pos
    ref_h = orc.llm_forward(x)

    hip = H.Hip(kv_max=kv_max)
    try:
        hip.upload_decoder([layer], ones, 1)
        hip.set_kv(k, v)
        for mode in (0, 1):
            hip.lib.tts_hip_set_decode_mode(mode)
            hip.pos = pos
            got_h = hip.llm_forward(x)
            assert_close(ref_h, got_h, f"hidden mode {mode}")
            gk, gv = hip.kv()
            assert_close(orc.kv_k[0, pos], gk[0, pos], "k row")
            assert_close(orc.kv_v[0, pos], gv[0, pos], "v row")
            assert np.array_equal(gk[0, :pos], k[0, :pos])
        # per-layer entry point on a device-resident hidden state: the raw residual stream
        dx = H.DevBuf.from_numpy(hip.lib, x)
        hip.lib.tts_hip_set_decode_mode(0)
        hip.lib.tts_hip_layer_decode(0, dx.ptr, pos)
        hip.lib.tts_hip_sync()
        hip.check()
        res = dx.to_numpy(np.float32, S.DIM)
        renorm = cases.OracleBackend(threads=1).rms_norm(res.reshape(1, -1), ones, 1)[0]
        assert_close(ref_h, renorm, "layer_decode residual")
    finally:
        hip.close()


@pytest.mark.parametrize("pos", [300, 575, 1100, 4100])
def test_one_layer_decode_on_smaller_grids(pos):
    """The whole-step kernel deals rows, attention heads and key chunks by its grid size: the same
    layer on 72, 128 and 200 workgroups (a device with fewer CUs), both schedules, at a position of
    every attention schedule."""
    kv_max = pos + 8
    layer = S.Layer(3)
    ones = np.ones(S.DIM, np.float32)
    k = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    v = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    k[0, :pos] = S.f32_normal((pos, S.KV_DIM), 200)
    v[0, :pos] = S.f32_normal((pos, S.KV_DIM), 300)
    x = S.f32_normal(S.DIM, 42)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open([layer], ones, kv_max, n_layers=1)
    orc.kv_k[0], orc.kv_v[0] = k[0], v[0]
    orc.pos = pos
    ref_h = orc.llm_forward(x)
    hip = H.Hip(kv_max=kv_max)
    try:
        hip.upload_decoder([layer], ones, 1)
        hip.set_kv(k, v)
        for grid in (72, 128, 200, 0):
            hip.lib.tts_hip_set_decode_grid(grid)
            hip.check()
            for mode in (0, 1):
                hip.lib.tts_hip_set_decode_mode(mode)
                hip.pos = pos
                got_h = hip.llm_forward(x)
                assert_close(ref_h, got_h, f"hidden grid {grid} mode {mode}")
                gk, gv = hip.kv()
                assert_close(orc.kv_k[0, pos], gk[0, pos], "k row")
                assert_close(orc.kv_v[0, pos], gv[0, pos], "v row")
        for bad in (64, 100, 4096):
            hip.lib.tts_hip_set_decode_grid(bad)
            assert "tts_hip_set_decode_grid" in hip.lib.tts_hip_last_error().decode()
        hip.err0 = hip.lib.tts_hip_error_count()          # those failures were asked for
        hip.lib.tts_hip_set_decode_mode(0)
        hip.pos = pos
        assert_close(ref_h, hip.llm_forward(x), "after the refused grids")
    finally:
        hip.close()


def test_schedules_agree_and_match_oracle_over_steps():
    """Mode 0 = persistent whole-step kernel, mode 1 = one kernel per phase.  Both run the same
    phase code and must agree bit for bit, run after run."""
    layers = [S.Layer(1), S.Layer(2), S.Layer(4)]
    norm = S.norm_weight(S.DIM, 99)
    n_layers, steps = 5, 6
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, 32, n_layers=n_layers)
    hip = H.Hip(kv_max=32)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        outs = {}
        for run, mode in enumerate((0, 1, 0)):
            hip.lib.tts_hip_set_decode_mode(mode)
            hip.pos = 0
            e = S.f32_normal(S.DIM, 6)
            hs = []
            for _ in range(steps):
                h = hip.llm_forward(e)
                hs.append(h)
                e = h.copy()
            outs[run] = np.stack(hs)
        assert np.array_equal(outs[0], outs[1]), "persistent and per-phase schedules differ"
        assert np.array_equal(outs[0], outs[2]), "the persistent schedule is not reproducible"
        n0 = hip.lib.tts_hip_error_count()
        hip.lib.tts_hip_set_decode_mode(2)              # no such schedule: refused, the mode stays
        assert hip.lib.tts_hip_error_count() == n0 + 1
        hip.err0 = n0 + 1
        # teacher-forced comparison with the oracle: feed the ORACLE's hidden to both
        hip.lib.tts_hip_set_decode_mode(0)
        hip.pos = 0
        e = S.f32_normal(S.DIM, 6)
        for s in range(steps):
            ref_h = orc.llm_forward(e)
            got_h = hip.llm_forward(e)
            assert_close(ref_h, got_h, f"step {s}")
            e = ref_h.copy()
        gk, gv = hip.kv()
        for l in range(n_layers):
            assert_close(orc.kv_k[l, :steps], gk[l, :steps], f"k cache layer {l}")
            assert_close(orc.kv_v[l, :steps], gv[l, :steps], f"v cache layer {l}")
    finally:
        hip.close()


def test_five_layers_on_136_workgroups():
    """Layer-to-layer hand-overs on a grid that is no power of two: teacher-forced steps against the
    oracle, and the two schedules bit for bit."""
    layers = [S.Layer(1), S.Layer(2), S.Layer(4)]
    norm = S.norm_weight(S.DIM, 99)
    n_layers, steps = 5, 4
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, 32, n_layers=n_layers)
    hip = H.Hip(kv_max=32)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        hip.lib.tts_hip_set_decode_grid(136)
        hip.check()
        refs, e = [], S.f32_normal(S.DIM, 6)
        for s in range(steps):
            refs.append(orc.llm_forward(e))
            e = refs[-1].copy()
        outs = {}
        for mode in (0, 1):
            hip.lib.tts_hip_set_decode_mode(mode)
            hip.pos = 0
            e, hs = S.f32_normal(S.DIM, 6), []
            for s in range(steps):
                hs.append(hip.llm_forward(e))
                assert_close(refs[s], hs[-1], f"mode {mode} step {s}")
                e = refs[s].copy()
            outs[mode] = np.stack(hs)
        assert np.array_equal(outs[0], outs[1])
    finally:
        hip.close()


@pytest.mark.parametrize("start", [381, 573])
def test_steps_across_a_change_of_attention_schedule(start):
    """Six teacher-forced steps over two layers that start three positions below a threshold of
    the attention schedule (384: a head's positions go to 2 workgroups, 576: to 8): the rows
    the kernel appended in the earlier steps are read by the later ones under the other
    schedule, and by the workgroups that prefetch the next layer's rows into L2."""
    steps, n_layers = 6, 2
    layers = [S.Layer(5), S.Layer(6)]
    norm = S.norm_weight(S.DIM, 98)
    kv_max = start + steps + 2
    k = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    v = np.zeros((26, kv_max, S.KV_DIM), np.float32)
    for l in range(n_layers):
        k[l, :start] = S.f32_normal((start, S.KV_DIM), 400 + l)
        v[l, :start] = S.f32_normal((start, S.KV_DIM), 500 + l)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, kv_max, n_layers=n_layers)
    for l in range(n_layers):
        orc.kv_k[l], orc.kv_v[l] = k[l], v[l]
    orc.pos = start
    hip = H.Hip(kv_max=kv_max)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        hip.set_kv(k, v)
        hip.lib.tts_hip_set_decode_mode(0)
        hip.pos = start
        e = S.f32_normal(S.DIM, 7)
        for s_ in range(steps):
            ref_h = orc.llm_forward(e)
            got_h = hip.llm_forward(e)
            assert_close(ref_h, got_h, f"step {s_} at position {start + s_}")
            e = ref_h.copy()
        gk, gv = hip.kv()
        for l in range(n_layers):
            assert_close(orc.kv_k[l, start:start + steps], gk[l, start:start + steps], f"k rows layer {l}")
            assert_close(orc.kv_v[l, start:start + steps], gv[l, start:start + steps], f"v rows layer {l}")
    finally:
        hip.close()


def test_26_layers_against_reference_fixture():
    """The committed fixture was written by the compiled reference: 26 layers
    cycling over two synthetic layers, 3 prefill rows then 2 decode steps
    (tests/golden/cases.py).  Prefill runs on the GPU too."""
    gold = np.load(os.path.join(S.GOLDEN_DIR, "llm.npz"))
    layers = [S.Layer(1), S.Layer(2)]
    norm = S.norm_weight(S.DIM, 99)
    hip = H.Hip(kv_max=cases.KV_MAX)
    try:
        hip.upload_decoder(layers, norm, 26)
        hip.llm_prefill(S.f32_normal((3, S.DIM), 5))
        e = S.f32_normal(S.DIM, 6)
        h0 = hip.llm_forward(e)
        assert_close(gold["hidden"][0], h0, "step 0")
        # teacher forcing for the second step: feed the reference's own hidden
        h1 = hip.llm_forward(gold["hidden"][0].copy())
        assert_close(gold["hidden"][1], h1, "step 1")
        gk, gv = hip.kv()
        for l in (0, 1, 12, 25):
            for r in range(4):          # rows 0..2 from the GPU prefill, row 3 appended by the first decode step
                assert_close(gold[f"kv_k_l{l}"][r], gk[l, r], f"k layer {l} row {r}")
                assert_close(gold[f"kv_v_l{l}"][r], gv[l, r], f"v layer {l} row {r}")
    finally:
        hip.close()


def test_position_outside_cache_is_an_error_not_a_fault():
    hip = H.Hip(kv_max=8)
    try:
        hip.upload_decoder([S.Layer(1)], np.ones(S.DIM, np.float32), 1)
        out = np.zeros(S.DIM, np.float32)
        n0 = hip.lib.tts_hip_error_count()
        hip.lib.tts_hip_llm_forward(out.ctypes.data, out.ctypes.data, 8)
        assert hip.lib.tts_hip_error_count() == n0 + 1
        assert b"outside the KV cache" in hip.lib.tts_hip_last_error()
    finally:
        hip.close()


def test_barrier_budget_exhausted_is_reported_and_recoverable():
    """The grid barrier spins against a wall-clock budget.  With a budget of one tick the
    first unfinished poll gives up: every workgroup leaves the kernel, the call is counted as
    failed, and with the default budget back the same step runs and matches the oracle."""
    layers = [S.Layer(1)]
    ones = np.ones(S.DIM, np.float32)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, ones, 16, n_layers=4)
    e = S.f32_normal(S.DIM, 6)
    ref = orc.llm_forward(e)
    hip = H.Hip(kv_max=16)
    try:
        hip.upload_decoder(layers, ones, 4)
        lib = hip.lib
        n0 = lib.tts_hip_error_count()
        lib.tts_hip_set_barrier_timeout(1)
        out = np.zeros(S.DIM, np.float32)
        lib.tts_hip_llm_forward(out.ctypes.data, e.ctypes.data, 0)
        assert lib.tts_hip_error_count() == n0 + 1
        assert b"barrier timed out" in lib.tts_hip_last_error()
        lib.tts_hip_set_barrier_timeout(0)
        hip.err0 = lib.tts_hip_error_count()
        hip.pos = 0
        got = hip.llm_forward(e)
        assert_close(ref, got, "after the timed-out step")
    finally:
        hip.lib.tts_hip_set_barrier_timeout(0)
        hip.close()


def test_abandoned_step_of_an_asynchronous_entry_is_reported_at_the_next_synchronisation():
    """tts_hip_llm_forward_device and tts_hip_layer_decode only queue the whole-step kernel.  A
    barrier that ran out of budget is reported by the call that next waits for the stream
    (tts_hip_sync, tts_hip_to_host, the event timer): one error per abandoned region, flag and
    epochs reset, and the same step then runs clean.  The budget of one tick is a host-side
    setting; every kernel still runs to its end."""
    layers = [S.Layer(1)]
    ones = np.ones(S.DIM, np.float32)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, ones, 16, n_layers=4)
    e = S.f32_normal(S.DIM, 6)
    ref = orc.llm_forward(e)
    hip = H.Hip(kv_max=16)
    try:
        hip.upload_decoder(layers, ones, 4)
        lib = hip.lib
        d_e = H.DevBuf.from_numpy(lib, e)
        d_h = H.DevBuf(lib, S.DIM * 4)

        def clean_step(what):
            lib.tts_hip_set_barrier_timeout(0)
            n = lib.tts_hip_error_count()
            lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, 0)
            lib.tts_hip_sync()
            assert lib.tts_hip_error_count() == n, (what, lib.tts_hip_last_error())
            assert_close(ref, d_h.to_numpy(np.float32, S.DIM), what)

        clean_step("before")
        # (1) forward_device, noticed by tts_hip_sync; two abandoned launches are one report
        n0 = lib.tts_hip_error_count()
        lib.tts_hip_set_barrier_timeout(1)
        lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, 0)
        lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, 1)
        assert lib.tts_hip_error_count() == n0          # nothing has waited for the stream yet
        lib.tts_hip_sync()
        assert lib.tts_hip_error_count() == n0 + 1
        assert b"barrier timed out" in lib.tts_hip_last_error()
        clean_step("after forward_device")
        # (2) layer_decode, noticed by the copy that fetches the result
        n0 = lib.tts_hip_error_count()
        lib.tts_hip_set_barrier_timeout(1)
        d_x = H.DevBuf.from_numpy(lib, e)
        lib.tts_hip_layer_decode(0, d_x.ptr, 0)
        d_x.to_numpy(np.float32, S.DIM)
        assert lib.tts_hip_error_count() == n0 + 1
        clean_step("after layer_decode")
        # (3) a timed region: the timer gives no figure for a region with an abandoned step
        n0 = lib.tts_hip_error_count()
        lib.tts_hip_set_barrier_timeout(1)
        bl = hip.pkg.bench_lib()
        bl.tts_hip_timer_start()
        lib.tts_hip_llm_forward_device(d_h.ptr, d_e.ptr, 0)
        assert bl.tts_hip_timer_stop_ms() < 0
        assert lib.tts_hip_error_count() == n0 + 1
        clean_step("after the timed region")
    finally:
        hip.lib.tts_hip_set_barrier_timeout(0)
        hip.close()


def test_second_utterance_overwrites_the_cache_rows_of_the_first():
    """The cache rows of an utterance are read with ordinary (cached) loads, and a second utterance
    in the same session rewrites rows 0.. with other values: what the attention then reads must be
    the new rows, also where an L2 still holds the old ones.  Modes 0 and 1, positions that take the
    per-head attention path."""
    n_layers, steps = 3, 40
    layers = [S.Layer(1), S.Layer(2), S.Layer(3)]
    ones = np.ones(S.DIM, np.float32)
    hip = H.Hip(kv_max=64)
    try:
        hip.upload_decoder(layers, ones, n_layers)
        for mode in (0, 1):
            hip.lib.tts_hip_set_decode_mode(mode)
            for utt, seed in enumerate((100, 200, 300)):
                orc = cases.OracleBackend(threads=16)
                orc.llm_open(layers, ones, 64, n_layers=n_layers)
                hip.pos = 0
                e = S.f32_normal(S.DIM, seed + mode)
                for s in range(steps):
                    ref_h = orc.llm_forward(e)
                    got_h = hip.llm_forward(e)
                    assert_close(ref_h, got_h, f"mode {mode} utterance {utt} step {s}")
                    e = ref_h.copy()
    finally:
        hip.lib.tts_hip_set_decode_mode(0)
        hip.close()


def test_backbone_is_the_leading_run_of_complete_layers():
    """Layers may be uploaded one at a time and in any order; the step runs over the leading
    layers that are complete, an upload that fails takes its layer out again, and a step without
    a first layer is an error instead of a launch on missing weights."""
    import ctypes as C
    layers = [S.Layer(1), S.Layer(2)]
    ones = np.ones(S.DIM, np.float32)
    e = S.f32_normal(S.DIM, 5)
    hip = H.Hip(kv_max=16)
    try:
        lib, pkg = hip.lib, hip.pkg
        assert lib.tts_hip_upload_llm_norm(ones.ctypes.data) == 0
        h1 = H.host_layer(pkg, layers[1])
        assert lib.tts_hip_upload_llm_layer(1, C.byref(h1)) == 0
        assert pkg.ctx().dec_layers_uploaded == 0              # layer 0 is still missing
        n0 = lib.tts_hip_error_count()
        out = np.zeros(S.DIM, np.float32)
        lib.tts_hip_llm_forward(out.ctypes.data, e.ctypes.data, 0)
        assert lib.tts_hip_error_count() == n0 + 1 and b"no weights" in lib.tts_hip_last_error()
        h0 = H.host_layer(pkg, layers[0])
        assert lib.tts_hip_upload_llm_layer(0, C.byref(h0)) == 0
        assert pkg.ctx().dec_layers_uploaded == 2

        orc = cases.OracleBackend(threads=8)
        orc.llm_open(layers, ones, 16, n_layers=2)
        hip.err0 = lib.tts_hip_error_count()
        assert_close(orc.llm_forward(e), hip.llm_forward(e), "two layers uploaded one by one")

        # a layer with a missing tensor is refused and the backbone ends in front of it
        broken = H.host_layer(pkg, layers[1])
        broken.w2_bf16 = None
        assert lib.tts_hip_upload_llm_layer(1, C.byref(broken)) == -1
        assert pkg.ctx().dec_layers_uploaded == 1
        orc1 = cases.OracleBackend(threads=8)
        orc1.llm_open(layers[:1], ones, 16, n_layers=1)
        hip.err0 = lib.tts_hip_error_count()
        hip.pos = 0
        assert_close(orc1.llm_forward(e), hip.llm_forward(e), "one layer left")
    finally:
        hip.close()
