"""Sequence-level (prefill) kernels on the matrix cores against the oracle:
the bf16 product on (hi, lo) activation planes, the causal attention (both of its
products on the same planes) and the whole prefill at sequence length 512, through the C ABI.
The oracle's seq_len > 1 linear is the reference's triple loop
(voxtral_tts_kernels.c:127-138); the bound is the path's 1e-3 per output
vector, and a much tighter one (5e-5 of the row's rms: the sequential fp32 sum of
the CPU path itself carries about 2e-5 at K = 9216) that a missing `lo` plane
(about 2e-3) or a misplaced tile cannot meet."""
import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu

SCALE = float(1.0 / np.sqrt(np.float32(128)))


@pytest.fixture(scope="module")
def hip():
    h = H.Hip(kv_max=64)
    yield h
    h.close()


@pytest.fixture(scope="module")
def orc():
    return cases.OracleBackend(threads=16)


def rows_close(ref, got, what, tight=5e-5):
    assert np.all(np.isfinite(got)), what
    for r in range(ref.shape[0]):
        mx, l2 = S.rel_errors(ref[r], got[r])
        assert mx < tight and l2 < tight, (what, r, mx, l2)


@pytest.mark.parametrize("m,n,k", [(512, 1024, 3072), (512, 3072, 9216), (512, 4096, 3072),
                                   (130, 256, 4096), (8, 128, 64), (77, 384, 192)])
def test_linear_rows_on_matrix_cores(hip, orc, m, n, k):
    W = S.bf16_normal((n, k), 3000 + m + n)
    x = S.f32_normal((m, k), 3100 + k)
    ref = orc.linear(x, W, None, m)
    dx, dW, dy = H.DevBuf.from_numpy(hip.lib, x), H.DevBuf.from_numpy(hip.lib, W), H.DevBuf(hip.lib, ref.nbytes)
    hip.lib.tts_hip_linear_bf16(dy.ptr, dx.ptr, None, m, k, n, dW.ptr)
    hip.lib.tts_hip_sync()
    hip.check()
    rows_close(ref, dy.to_numpy(np.float32, ref.shape), f"linear {m}x{n}x{k}")
    # host pointers take the same path
    y = np.zeros_like(ref)
    hip.lib.tts_hip_linear_bf16(y.ctypes.data, x.ctypes.data, W.ctypes.data, m, k, n, None)
    hip.check()
    rows_close(ref, y, f"linear host {m}x{n}x{k}")
    for b in (dx, dW, dy):
        b.free()


def test_linear_closed_forms(hip):
    """One-hot and constant weights: the product must pick / sum activations exactly
    up to the (hi, lo) representation (2^-17 relative per element)."""
    m, n, k = 40, 128, 256
    x = S.f32_normal((m, k), 9)
    W = np.zeros((n, k), np.float32)
    for j in range(n):
        W[j, (7 * j) % k] = 1.0
    Wb = S.f32_to_bf16_trunc(W)
    y = np.zeros((m, n), np.float32)
    hip.lib.tts_hip_linear_bf16(y.ctypes.data, x.ctypes.data, Wb.ctypes.data, m, k, n, None)
    hip.check()
    want = x[:, [(7 * j) % k for j in range(n)]]
    assert np.max(np.abs(y - want) / np.maximum(np.abs(want), 1e-30)) < 2.0 ** -16
    Wb = S.f32_to_bf16_trunc(np.ones((n, k), np.float32))
    hip.lib.tts_hip_linear_bf16(y.ctypes.data, x.ctypes.data, Wb.ctypes.data, m, k, n, None)
    hip.check()
    want = x.astype(np.float64).sum(axis=1, keepdims=True).repeat(n, axis=1)
    assert np.max(np.abs(y - want)) < 1e-4 * np.sqrt(k)


@pytest.mark.parametrize("seq,start", [(8, 0), (77, 19), (512, 0), (32, 0), (33, 31)])
def test_causal_attention_tiles(hip, orc, seq, start):
    """(In this order the library's buffer of K/V tile images grows twice after it has been used.)"""
    Q = S.f32_normal((seq, S.Q_DIM), 700 + seq)
    K = S.f32_normal((start + seq, S.KV_DIM), 701 + seq)
    V = S.f32_normal((start + seq, S.KV_DIM), 702 + seq)
    dQ, dK, dV = (H.DevBuf.from_numpy(hip.lib, a) for a in (Q, K, V))
    dO = H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, start, S.HEADS,
                                             S.KV_HEADS, S.HEAD_DIM, SCALE)
    hip.lib.tts_hip_sync()
    hip.check()
    ref = orc.causal_attention(Q, K, V, seq, start + seq, start)
    got = dO.to_numpy(np.float32, Q.shape)
    # Q, K, V and the probabilities enter the matrix cores as (hi, lo) bf16 pairs: 16 mantissa bits, an
    # error of up to 2^-17 of each operand, i.e. absolute errors of a few 1e-5 on sums of O(1) terms that
    # may cancel.  The reference's rule with its attention rtol (test_kernels.c:79-116, :463-468) and the
    # absolute floor scaled to the output (1e-3 of its rms), then every row against its own rms.
    ok, mr, ma, bad = S.compare_tensors(ref, got, 1e-3, 1e-3 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2))))
    assert ok, (mr, ma, bad)
    # per row: the l2 error stays near 2^-17; the largest element error is 2^-16 of the largest term p v of
    # its sum, which in a row of many keys is several times the row's rms (measured worst: 1.3e-4)
    rows_close(ref, got, f"attention {seq}+{start}", tight=3e-4)
    for b in (dQ, dK, dV, dO):
        b.free()


def test_causal_attention_honours_the_callers_scale(hip):
    """The reference's entry takes the softmax scale as an argument (voxtral_tts_cuda.h:142-146);
    the matrix-core path (8 or more queries, aligned pointers) must use it like the generic path,
    not the model's 1/sqrt(128)."""
    seq, scale = 40, 0.03
    Q = S.f32_normal((seq, S.Q_DIM), 811)
    K = S.f32_normal((seq, S.KV_DIM), 812)
    V = S.f32_normal((seq, S.KV_DIM), 813)
    ref = np.zeros_like(Q)
    S.oracle().orc_causal_attention(S.fp(ref), S.fp(Q), S.fp(K), S.fp(V), seq, seq, S.HEADS, S.KV_HEADS,
                                    S.HEAD_DIM, scale, 0, 0)
    dQ, dK, dV = (H.DevBuf.from_numpy(hip.lib, a) for a in (Q, K, V))
    dO = H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, 0, S.HEADS,
                                             S.KV_HEADS, S.HEAD_DIM, scale)
    hip.lib.tts_hip_sync()
    hip.check()
    got = dO.to_numpy(np.float32, Q.shape)
    rows_close(ref, got, "attention with scale 0.03", tight=1e-4)
    # and the two scales really give different answers on this input
    ref_default = cases.OracleBackend(threads=16).causal_attention(Q, K, V, seq, seq, 0)
    assert np.max(np.abs(ref_default - ref)) > 1e-2
    for b in (dQ, dK, dV, dO):
        b.free()


def test_attention_first_key_only_and_equal_keys(hip):
    """Closed forms: query 0 sees one key, so its output is V row 0 of its KV head;
    with all keys equal every query returns the mean of the visible V rows."""
    seq = 40
    Q = S.f32_normal((seq, S.Q_DIM), 1)
    K = np.tile(S.f32_normal((1, S.KV_DIM), 2), (seq, 1))
    V = S.f32_normal((seq, S.KV_DIM), 3)
    dQ, dK, dV = (H.DevBuf.from_numpy(hip.lib, a) for a in (Q, K, V))
    dO = H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, 0, S.HEADS,
                                             S.KV_HEADS, S.HEAD_DIM, SCALE)
    hip.lib.tts_hip_sync()
    got = dO.to_numpy(np.float32, Q.shape).reshape(seq, S.HEADS, S.HEAD_DIM)
    Vh = V.reshape(seq, S.KV_HEADS, S.HEAD_DIM).astype(np.float64)
    # V passes through the (hi, lo) split: 16 mantissa bits, at most 2^-17 of |v| off per row
    atol = 2.0 ** -16 * float(np.abs(V).max())
    for h in (0, 5, 31):
        assert np.allclose(got[0, h], Vh[0, h // 4], rtol=0, atol=atol)
        for i in (1, 31, 32, 39):
            assert np.allclose(got[i, h], Vh[: i + 1, h // 4].mean(axis=0), rtol=0, atol=atol)


def _prefill_case(n_layers, chunks, kv_max, check_rows):
    layers = [S.Layer(11), S.Layer(12)]
    norm = S.norm_weight(S.DIM, 98)
    orc = cases.OracleBackend(threads=16)
    orc.llm_open(layers, norm, kv_max, n_layers=n_layers)
    hip = H.Hip(kv_max=kv_max)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        n = 0
        for ci, s in enumerate(chunks):
            e = S.f32_normal((s, S.DIM), 50 + ci)
            rx = orc.llm_prefill(e, want_x=True)
            gx = hip.llm_prefill(e, want_x=True)
            hip.check()
            for r in range(s):
                mx, l2 = S.rel_errors(rx[r], gx[r])
                assert mx < 1e-3 and l2 < 1e-3, ("residual", ci, r, mx, l2)
            n += s
        gk, gv = hip.kv()
        for l in range(n_layers):
            for r in check_rows(n):
                for name, a, b in (("k", orc.kv_k, gk), ("v", orc.kv_v, gv)):
                    mx, l2 = S.rel_errors(a[l, r], b[l, r])
                    assert mx < 1e-3 and l2 < 1e-3, (name, l, r, mx, l2)
        x = S.f32_normal(S.DIM, 7)
        mx, l2 = S.rel_errors(orc.llm_forward(x), hip.llm_forward(x))
        assert mx < 1e-3 and l2 < 1e-3, ("decode after prefill", mx, l2)
    finally:
        hip.close()


def test_prefill_512_one_layer():
    _prefill_case(1, [512], 516, lambda n: range(n))


def test_prefill_chunks_three_layers():
    _prefill_case(3, [150, 45, 1], 200, lambda n: range(0, n, 3))


def test_prefill_row_counts_with_uneven_k_cuts():
    """300 rows are 3 row tiles: the output and down products then run in 7 K cuts of 5 or 4 (11 or 10)
    pairs of steps and q|k|v in 3; 650 rows (6 tiles) take 3 cuts and none."""
    _prefill_case(1, [300, 650], 960, lambda n: range(0, n, 7))


@pytest.mark.parametrize("chunks", [[512], [64], [130, 7], [300], [1, 650]])
def test_prefill_schedules_agree_bit_for_bit(chunks):
    """Schedule 1 runs everything behind a layer's attention as one persistent launch whose work items
    wait for each other per block of 128 rows; schedule 0 is one launch per product and row pass.  Same K
    cuts, same tile walk, same sums in the same order: cache rows and residual stream must be equal bit
    for bit, run after run (3 layers, so that the q|k|v product of the next layer inside the persistent
    launch and the last layer without one are both walked)."""
    layers = [S.Layer(11), S.Layer(12)]
    norm = S.norm_weight(S.DIM, 98)
    n_layers, kv_max = 3, sum(chunks) + 8
    hip = H.Hip(kv_max=kv_max)
    try:
        hip.upload_decoder(layers, norm, n_layers)
        outs = {}
        for run, mode in enumerate((1, 0, 1)):
            hip.lib.tts_hip_set_prefill_mode(mode)
            hip.check()
            hip.lib.tts_hip_memset(hip.pkg.ctx().kv_cache_k_gpu, 0, 26 * kv_max * S.KV_DIM * 4)
            hip.lib.tts_hip_memset(hip.pkg.ctx().kv_cache_v_gpu, 0, 26 * kv_max * S.KV_DIM * 4)
            hip.pos = 0
            xs = []
            for ci, s in enumerate(chunks):
                print(f"prefill schedule {mode}, chunk of {s} rows at {hip.pos}", flush=True)
                xs.append(hip.llm_prefill(S.f32_normal((s, S.DIM), 60 + ci), want_x=True))
            gk, gv = hip.kv()
            outs[run] = (np.concatenate(xs), gk[:n_layers].copy(), gv[:n_layers].copy())
        for run in (1, 2):
            for a, b, what in zip(outs[0], outs[run], ("residual stream", "k rows", "v rows")):
                assert np.all(np.isfinite(a)), what
                assert np.array_equal(a, b), (what, run, float(np.abs(a - b).max()))
        hip.lib.tts_hip_set_prefill_mode(7)
        assert b"tts_hip_set_prefill_mode" in hip.lib.tts_hip_last_error()
        hip.err0 = hip.lib.tts_hip_error_count()
    finally:
        hip.lib.tts_hip_set_prefill_mode(0)
        hip.close()
