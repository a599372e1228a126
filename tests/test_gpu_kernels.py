"""Kernel-level parity on the GPU, through the C ABI, against the oracle.
Cases, seeds' style and tolerances follow the reference's test_kernels.c
(:122-430): add 0/0, silu_mul 1e-5/1e-7, rms_norm 1e-4/1e-6,
gemm_bf16 1e-3/1e-4, attention 1e-3/1e-5; plus the config-1 matvec shapes with
the norm-relative bound 1e-3 per output vector."""
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


def dev(hip, a):
    return H.DevBuf.from_numpy(hip.lib, a)


def test_add_inplace_exact(hip, orc):
    a, b = S.f32_normal(S.DIM, 1000, 0.1), S.f32_normal(S.DIM, 1001, 0.1)
    da, db = dev(hip, a), dev(hip, b)
    hip.lib.tts_hip_add_inplace(da.ptr, db.ptr, S.DIM)
    hip.lib.tts_hip_sync()
    got = da.to_numpy(np.float32, S.DIM)
    assert np.array_equal(got, orc.add(a, b))


def test_silu_mul(hip, orc):
    g, u = S.f32_normal(S.FFN, 800, 0.1), S.f32_normal(S.FFN, 900, 0.1)
    dg, du = dev(hip, g), dev(hip, u)
    hip.lib.tts_hip_silu_mul(dg.ptr, du.ptr, S.FFN)
    hip.lib.tts_hip_sync()
    ok, mr, ma, bad = S.compare_tensors(orc.silu_mul(g, u), dg.to_numpy(np.float32, S.FFN), 1e-5, 1e-7)
    assert ok, (mr, ma, bad)


@pytest.mark.parametrize("seq", [1, 3, 17])
def test_rms_norm(hip, orc, seq):
    x = S.f32_normal((seq, S.DIM), 42, 0.1)
    w = S.norm_weight(S.DIM, 123)
    dx, dw, do = dev(hip, x), dev(hip, w), H.DevBuf(hip.lib, x.nbytes)
    hip.lib.tts_hip_rms_norm(do.ptr, dx.ptr, dw.ptr, seq, S.DIM, S.EPS)
    hip.lib.tts_hip_sync()
    ok, mr, ma, bad = S.compare_tensors(orc.rms_norm(x, w, seq), do.to_numpy(np.float32, x.shape), 1e-4, 1e-6)
    assert ok, (mr, ma, bad)


def test_rope_table_is_bit_equal_and_rotation_matches(hip, orc):
    pos0, seq = 5, 9
    fr = orc.rope_freqs(list(range(pos0, pos0 + seq)))
    dfr = H.DevBuf(hip.lib, fr.nbytes)
    hip.lib.tts_hip_compute_rope_freqs(dfr.ptr, pos0, seq, S.HEAD_DIM, S.THETA)
    assert np.array_equal(dfr.to_numpy(np.float32, fr.shape), fr)
    for heads, dim in ((S.HEADS, S.Q_DIM), (S.KV_HEADS, S.KV_DIM)):
        x = S.f32_normal((seq, dim), 9 + heads)
        dx = dev(hip, x)
        hip.lib.tts_hip_apply_rope(dx.ptr, dfr.ptr, seq, heads, S.HEAD_DIM)
        hip.lib.tts_hip_sync()
        assert np.array_equal(dx.to_numpy(np.float32, x.shape), orc.apply_rope(x, fr, seq, heads))


def _linear(hip, x, W, seq, device_io):
    out_dim, in_dim = W.shape
    y = np.zeros((seq, out_dim), np.float32)
    dW = dev(hip, W)
    if device_io:
        dx, dy = dev(hip, x), H.DevBuf(hip.lib, y.nbytes)
        hip.lib.tts_hip_linear_bf16(dy.ptr, dx.ptr, None, seq, in_dim, out_dim, dW.ptr)
        hip.lib.tts_hip_sync()
        y = dy.to_numpy(np.float32, y.shape)
        dx.free(); dy.free()
    else:
        hip.lib.tts_hip_linear_bf16(y.ctypes.data, x.ctypes.data, None, seq, in_dim, out_dim, dW.ptr)
    dW.free()
    hip.check()
    return y


def test_gemm_bf16_reference_case(hip, orc):
    """test_kernels.c:388-430: M=1, K=3072, N=4096, x ~ 0.1 N(0,1), rtol 1e-3 / atol 1e-4."""
    W = S.bf16_normal((4096, 3072), 1200)
    x = S.f32_normal((1, 3072), 1100, 0.1)
    ref = orc.linear(x, W, None, 1)
    for device_io in (True, False):
        ok, mr, ma, bad = S.compare_tensors(ref, _linear(hip, x, W, 1, device_io), 1e-3, 1e-4)
        assert ok, (device_io, mr, ma, bad)


@pytest.mark.parametrize("n,k", [(9216, 3072), (3072, 9216), (131072, 3072), (3072, 36), (36, 3072)])
def test_config1_matvec_shapes(hip, orc, n, k):
    W = S.bf16_normal((n, k), 1000 + n % 97 + k)
    x = S.f32_normal((1, k), 42)
    ref = orc.linear(x, W, None, 1)
    got = _linear(hip, x, W, 1, True)
    mx, l2 = S.rel_errors(ref, got)
    assert mx < 1e-3 and l2 < 1e-3, (mx, l2)
    ok, mr, ma, bad = S.compare_tensors(ref, got, 1e-3, 1e-3 * float(np.sqrt(np.mean(ref ** 2))))
    assert ok, (mr, ma, bad)


@pytest.mark.parametrize("n,k", [(1000, 512), (5, 1024), (777, 2560), (257, 9216), (300, 16384), (64, 520)])
def test_matvec_ragged_shapes(hip, orc, n, k):
    """Single-row products whose rows do not divide over the workgroups, with one or many 512-wide
    chunks per row; 16384 columns do not fit the stream kernel's LDS and 520 are not whole chunks:
    those two take the wave-per-row kernel."""
    W = S.bf16_normal((n, k), 31 * n + k)
    x = S.f32_normal((1, k), 17)
    ref = orc.linear(x, W, None, 1)
    got = _linear(hip, x, W, 1, True)
    mx, l2 = S.rel_errors(ref, got)
    assert mx < 1e-3 and l2 < 1e-3, (n, k, mx, l2)
    again = _linear(hip, x, W, 1, True)
    assert np.array_equal(got, again)              # fixed summation order: reproducible


@pytest.mark.parametrize("seq", [3, 6, 19])
def test_linear_several_rows_and_host_weights(hip, orc, seq):
    W = S.bf16_normal((200, 3072), 77)
    x = S.f32_normal((seq, 3072), 78)
    ref = orc.linear(x, W, None, seq)
    y = np.zeros_like(ref)
    hip.lib.tts_hip_linear_bf16(y.ctypes.data, x.ctypes.data, W.ctypes.data, seq, 3072, 200, None)
    hip.check()
    mx, l2 = S.rel_errors(ref, y)
    assert mx < 1e-3 and l2 < 1e-3, (mx, l2)


@pytest.mark.parametrize("seq_k", [1, 3, 10, 50, 100, 225, 513])
def test_causal_attention_decode(hip, orc, seq_k):
    """test_kernels.c:168-232 (seq_k 1..225, data 0.1 N(0,1)), plus 513 and unit-scale data."""
    for std in (0.1, 1.0):
        Q = S.f32_normal((1, S.Q_DIM), 100 + seq_k, std)
        K = S.f32_normal((seq_k, S.KV_DIM), 200 + seq_k, std)
        V = S.f32_normal((seq_k, S.KV_DIM), 300 + seq_k, std)
        ref = orc.causal_attention(Q, K, V, 1, seq_k, seq_k - 1)
        dQ, dK, dV, dO = dev(hip, Q), dev(hip, K), dev(hip, V), H.DevBuf(hip.lib, Q.nbytes)
        hip.lib.tts_hip_causal_attention_decode(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq_k, S.HEADS,
                                                S.KV_HEADS, S.HEAD_DIM, SCALE, S.KV_DIM)
        hip.lib.tts_hip_sync()
        got = dO.to_numpy(np.float32, Q.shape)
        ok, mr, ma, bad = S.compare_tensors(ref, got, 1e-3, 1e-5)
        assert ok, (seq_k, std, mr, ma, bad)
        for b in (dQ, dK, dV, dO):
            b.free()


def test_bidirectional_attention(hip, orc):
    Q = S.f32_normal((3, S.Q_DIM), 500, 0.1)
    K = S.f32_normal((3, S.KV_DIM), 600, 0.1)
    V = S.f32_normal((3, S.KV_DIM), 700, 0.1)
    dQ, dK, dV, dO = dev(hip, Q), dev(hip, K), dev(hip, V), H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_bidirectional_attention(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, 3, S.HEADS, S.KV_HEADS,
                                            S.HEAD_DIM, SCALE)
    hip.lib.tts_hip_sync()
    ok, mr, ma, bad = S.compare_tensors(orc.bidir_attention(Q, K, V, 3), dO.to_numpy(np.float32, Q.shape),
                                        1e-3, 1e-5)
    assert ok, (mr, ma, bad)


def test_causal_attention_prefill_with_offset(hip, orc):
    seq, start = 12, 5
    Q = S.f32_normal((seq, S.Q_DIM), 400)
    K = S.f32_normal((start + seq, S.KV_DIM), 401)
    V = S.f32_normal((start + seq, S.KV_DIM), 402)
    dQ, dK, dV, dO = dev(hip, Q), dev(hip, K), dev(hip, V), H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, start, S.HEADS,
                                             S.KV_HEADS, S.HEAD_DIM, SCALE)
    hip.lib.tts_hip_sync()
    ref = orc.causal_attention(Q, K, V, seq, start + seq, start)
    # 8 or more queries with the model's head counts run on the matrix cores, which are fed (hi, lo) bf16
    # pairs (16 mantissa bits per operand): the reference's rule with the absolute floor scaled to the
    # output, as for the seq > 1 linear
    ok, mr, ma, bad = S.compare_tensors(ref, dO.to_numpy(np.float32, Q.shape), 1e-3,
                                        1e-3 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2))))
    assert ok, (mr, ma, bad)


@pytest.mark.parametrize("seq,start,heads,kv_heads", [(5, 3, S.HEADS, S.KV_HEADS), (12, 5, 8, 2), (7, 0, 4, 4)])
def test_causal_attention_prefill_fp32_path(hip, orc, seq, start, heads, kv_heads):
    """Fewer than 8 queries, or head counts other than the model's, take the fp32 row kernel: the
    reference's own tolerances for its decode attention apply unchanged (test_kernels.c:168-232,
    rtol 1e-3 / atol 1e-5)."""
    Q = S.f32_normal((seq, heads * S.HEAD_DIM), 410 + seq)
    K = S.f32_normal((start + seq, kv_heads * S.HEAD_DIM), 411 + seq)
    V = S.f32_normal((start + seq, kv_heads * S.HEAD_DIM), 412 + seq)
    dQ, dK, dV, dO = dev(hip, Q), dev(hip, K), dev(hip, V), H.DevBuf(hip.lib, Q.nbytes)
    hip.lib.tts_hip_causal_attention_prefill(dO.ptr, dQ.ptr, dK.ptr, dV.ptr, seq, start, heads,
                                             kv_heads, S.HEAD_DIM, SCALE)
    hip.lib.tts_hip_sync()
    hip.check()
    ref = orc.causal_attention(Q, K, V, seq, start + seq, start, heads=heads, kv_heads=kv_heads)
    ok, mr, ma, bad = S.compare_tensors(ref, dO.to_numpy(np.float32, Q.shape), 1e-3, 1e-5)
    assert ok, (mr, ma, bad)


def test_embed_token_exact(hip, orc):
    emb = S.bf16_normal((50, S.DIM), 77, 1.0)
    de, do = dev(hip, emb), H.DevBuf(hip.lib, S.DIM * 4)
    hip.lib.tts_hip_embed_token(do.ptr, de.ptr, 33, S.DIM)
    hip.lib.tts_hip_sync()
    assert np.array_equal(do.to_numpy(np.float32, S.DIM), orc.embed_token(emb, 33))


def _bf16_rne(x):
    """bf16 bits of fp32 values, round to nearest even, in integer arithmetic (finite inputs)."""
    u = x.view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def test_split_planes_bit_exact(hip):
    """hi = bf16(x), lo = bf16(x - hi) with round to nearest even: the device uses the
    packed hardware conversion, the model here is integer arithmetic.  Random values over
    many magnitudes, exact ties in both directions, values that round up into the next
    binade, zeros of both signs, the largest finite value bf16 does not round to
    infinity, and residuals that fall into the fp32 denormal range."""
    rng = np.random.default_rng(5)
    parts = [
        (rng.standard_normal(1 << 16) * np.exp(rng.uniform(-20, 20, 1 << 16))).astype(np.float32),
        # ties: low half exactly 0x8000 with even and odd bf16 mantissas, and just around them
        np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0xBF808000, 0xBF818000,
                  0x3FFF8000, 0x3FFFFFFF, 0x7F7F7FFF, 0x00000000, 0x80000000,
                  0x00810000, 0x00808000, 0x00FF8000, 0x01000001, 0x0C000001], np.uint32).view(np.float32),
        np.float32(1.0) + np.arange(1 << 12, dtype=np.float32) * np.float32(2.0 ** -20),
    ]
    x = np.concatenate(parts)
    if x.size & 1:
        x = x[:-1]
    d_x = dev(hip, x)
    d_hi = H.DevBuf(hip.lib, 2 * x.size)
    d_lo = H.DevBuf(hip.lib, 2 * x.size)
    assert hip.lib.tts_hip_split_planes(d_hi.ptr, d_lo.ptr, d_x.ptr, x.size) == 0
    hip.lib.tts_hip_sync()
    hip.check()
    hi = d_hi.to_numpy(np.uint16, x.shape)
    lo = d_lo.to_numpy(np.uint16, x.shape)
    want_hi = _bf16_rne(x)
    hi_f = (want_hi.astype(np.uint32) << 16).view(np.float32)
    resid = x - hi_f                                          # exact in fp32
    want_lo = _bf16_rne(resid)
    assert np.array_equal(hi, want_hi), np.flatnonzero(hi != want_hi)[:8]
    bad = np.flatnonzero(lo != want_lo)
    assert bad.size == 0, (bad[:8], x[bad[:8]].view(np.uint32), lo[bad[:8]], want_lo[bad[:8]])
    # hi + lo carries x to 2^-16 of its magnitude or better
    back = hi_f.astype(np.float64) + (lo.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    big = np.abs(x) > 1e-30
    assert np.max(np.abs(back[big] - x[big]) / np.abs(x[big])) < 2.0 ** -16
    # an odd count and a misaligned pointer are refused
    n0 = hip.lib.tts_hip_error_count()
    assert hip.lib.tts_hip_split_planes(d_hi.ptr, d_lo.ptr, d_x.ptr, 3) == -1
    assert hip.lib.tts_hip_split_planes(d_hi.ptr, d_lo.ptr, d_x.ptr + 4, 2) == -1
    assert hip.lib.tts_hip_error_count() == n0 + 2
    hip.err0 = n0 + 2
    for b in (d_x, d_hi, d_lo):
        b.free()


def test_bad_arguments_are_reported_not_executed(hip):
    n0 = hip.lib.tts_hip_error_count()
    hip.lib.tts_hip_rms_norm(None, None, None, 0, S.DIM, S.EPS)
    hip.lib.tts_hip_causal_attention_decode(None, None, None, None, 4, 32, 5, 128, SCALE, 0)
    assert hip.lib.tts_hip_error_count() == n0 + 2
    hip.err0 = hip.lib.tts_hip_error_count()
