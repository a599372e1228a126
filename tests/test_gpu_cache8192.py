"""The reference's own cache size: tts_load allocates kv_cache_max = 8192 rows and hands that to the
backend's init (voxtral_tts.c:64, :96).  One context of that size, against the oracle:

* one decoder layer at positions 6000 and 8191 (the last row of the cache and of the RoPE table),
  both launch schedules, on the default grid and on 72 and 200 workgroups: from 4096 positions on
  the chunked attention schedule with its last-arriver merge runs, at its cap of chunks;
* the causal attention entry point over rows that end at 8192 (256 key tiles per kv head);
* a two-layer prefill whose rows end at 8192 on a cache that is already 8128 rows long.
"""
import ctypes as C

import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]
TOL = 1e-3
KV_MAX = 8192
ROW_BYTES = S.KV_DIM * 4


def assert_close(ref, got, what, tol=TOL):
    mx, l2 = S.rel_errors(ref, got)
    assert np.all(np.isfinite(got)), what
    assert mx < tol and l2 < tol, (what, mx, l2)


class Cache:
    """Rows of the device cache of one layer, without moving the 1.7 GB of all 26."""

    def __init__(self, hip):
        self.hip = hip
        ctx = hip.pkg.ctx()
        assert ctx.kv_cache_max == KV_MAX
        self.k, self.v = ctx.kv_cache_k_gpu, ctx.kv_cache_v_gpu

    def put(self, layer, k_rows, v_rows, row0=0):
        off = (layer * KV_MAX + row0) * ROW_BYTES
        self.hip.lib.tts_hip_to_device(self.k + off, k_rows.ctypes.data, k_rows.nbytes)
        self.hip.lib.tts_hip_to_device(self.v + off, v_rows.ctypes.data, v_rows.nbytes)

    def rows(self, layer, row0, n):
        k = np.empty((n, S.KV_DIM), np.float32)
        v = np.empty((n, S.KV_DIM), np.float32)
        off = (layer * KV_MAX + row0) * ROW_BYTES
        self.hip.lib.tts_hip_to_host(k.ctypes.data, self.k + off, k.nbytes)
        self.hip.lib.tts_hip_to_host(v.ctypes.data, self.v + off, v.nbytes)
        return k, v


@pytest.fixture(scope="module")
def session():
    hip = H.Hip(kv_max=KV_MAX)
    layers = [S.Layer(3), S.Layer(5)]
    ones = np.ones(S.DIM, np.float32)
    hip.upload_decoder(layers, ones, 2)
    k = S.f32_normal((KV_MAX, S.KV_DIM), 200)
    v = S.f32_normal((KV_MAX, S.KV_DIM), 300)
    yield hip, layers, ones, k, v
    hip.close()


@pytest.mark.parametrize("pos", [6000, 8191])
def test_one_layer_decode_deep_in_an_8192_row_cache(session, pos):
    hip, layers, ones, k, v = session
    cache = Cache(hip)
    x = S.f32_normal(S.DIM, 42)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open([layers[0]], ones, KV_MAX, n_layers=1)
    orc.kv_k[0], orc.kv_v[0] = k, v
    orc.pos = pos
    ref_h = orc.llm_forward(x)
    renorm = cases.OracleBackend(threads=1)
    dx = H.DevBuf(hip.lib, S.DIM * 4)
    try:
        for grid in (0, 72, 200):
            hip.lib.tts_hip_set_decode_grid(grid)
            hip.check()
            for mode in (0, 1):
                hip.lib.tts_hip_set_decode_mode(mode)
                print(f"decode pos {pos} grid {grid} mode {mode}", flush=True)
                cache.put(0, k, v)                              # row `pos` is overwritten by every step
                hip.lib.tts_hip_to_device(dx.ptr, x.ctypes.data, x.nbytes)
                hip.lib.tts_hip_layer_decode(0, dx.ptr, pos)
                hip.lib.tts_hip_sync()
                hip.check()
                res = dx.to_numpy(np.float32, S.DIM)
                got_h = renorm.rms_norm(res.reshape(1, -1), ones, 1)[0]   # the oracle's hidden is normalised (unit gains)
                assert_close(ref_h, got_h, f"hidden pos {pos} grid {grid} mode {mode}")
                gk, gv = cache.rows(0, pos, 1)
                assert_close(orc.kv_k[0, pos], gk[0], "appended k row")
                assert_close(orc.kv_v[0, pos], gv[0], "appended v row")
                if pos > 0:
                    pk, pv = cache.rows(0, pos - 1, 1)
                    assert np.array_equal(pk[0], k[pos - 1]) and np.array_equal(pv[0], v[pos - 1])
    finally:
        hip.lib.tts_hip_set_decode_grid(0)
        hip.lib.tts_hip_set_decode_mode(0)
        dx.free()


def test_causal_attention_over_rows_that_end_at_8192(session):
    hip, layers, ones, k, v = session
    seq, start = 48, KV_MAX - 48
    Q = S.f32_normal((seq, S.Q_DIM), 400)
    dQ, dK, dV = (H.DevBuf.from_numpy(hip.lib, a) for a in (Q, k, v))
    dO = H.DevBuf(hip.lib, Q.nbytes)
    scale = float(1.0 / np.sqrt(np.float32(S.HEAD_DIM)))
    try:
        print("attention 48 queries over 8192 rows", flush=True)
        hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, start, S.HEADS,
                                                 S.KV_HEADS, S.HEAD_DIM, scale)
        hip.lib.tts_hip_sync()
        hip.check()
        got = dO.to_numpy(np.float32, Q.shape)
        ref = cases.OracleBackend(threads=16).causal_attention(Q, k, v, seq, KV_MAX, start)
        # matrix-core path: (hi, lo) bf16 operands, floor scaled to the output (as tests/test_gpu_kernels.py)
        ok, mr, ma, bad = S.compare_tensors(ref, got, 1e-3, 1e-3 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2))))
        assert ok, (mr, ma, bad)
        for r in range(seq):
            assert_close(ref[r], got[r], f"attention row {r}")
    finally:
        for b in (dQ, dK, dV, dO):
            b.free()


def test_two_layer_prefill_that_ends_at_row_8192(session):
    hip, layers, ones, k, v = session
    cache = Cache(hip)
    seq, start = 64, KV_MAX - 64
    embeds = S.f32_normal((seq, S.DIM), 77)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, ones, KV_MAX, n_layers=2)
    for l in range(2):
        orc.kv_k[l, :start], orc.kv_v[l, :start] = k[:start], v[:start]
        cache.put(l, k[:start], v[:start])
    orc.pos = start
    ref_x = orc.llm_prefill(embeds, want_x=True)
    print("prefill of rows 8128..8191, 2 layers", flush=True)
    hip.pos = start
    got_x = hip.llm_prefill(embeds, want_x=True)
    for l in range(2):
        gk, gv = cache.rows(l, start, seq)
        for r in (0, 1, 31, 32, 62, 63):
            assert_close(orc.kv_k[l, start + r], gk[r], f"k layer {l} row {start + r}")
            assert_close(orc.kv_v[l, start + r], gv[r], f"v layer {l} row {start + r}")
        pk, pv = cache.rows(l, start - 1, 1)
        assert np.array_equal(pk[0], k[start - 1]) and np.array_equal(pv[0], v[start - 1])
    for r in range(seq):
        assert_close(ref_x[r], got_x[r], f"residual row {start + r}")
    # and the step behind it would be out of the cache: refused, nothing launched
    n0 = hip.lib.tts_hip_error_count()
    out = np.zeros(S.DIM, np.float32)
    hip.lib.tts_hip_llm_forward(out.ctypes.data, embeds[0].ctypes.data, KV_MAX)
    assert hip.lib.tts_hip_error_count() == n0 + 1
    assert b"outside the KV cache" in hip.lib.tts_hip_last_error()
    hip.err0 = hip.lib.tts_hip_error_count()
