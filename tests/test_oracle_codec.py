"""The oracle's codec decoder: against the committed fixture written by the compiled reference
(bit for bit), against the compiled reference directly where it is built, and against what the
mathematics fixes (delta kernels, windows of one, closed-form ALiBi weights, a float64 numpy
model of the whole decoder written from the textbook formulas)."""
import os

import numpy as np
import pytest

import codecsupport as K
import vtsupport as S

import sys
sys.path.insert(0, S.GOLDEN_DIR)
import codec_cases as CC  # noqa: E402


def test_codec_matches_reference_fixture():
    gold = np.load(os.path.join(S.GOLDEN_DIR, "codec.npz"))
    got = CC.codec_cases(CC.OracleCodecBackend(threads=8))
    assert set(got.keys()) == set(gold.files)
    for k in gold.files:
        a, b = np.ascontiguousarray(got[k]), gold[k]
        assert a.shape == b.shape and a.dtype == b.dtype, k
        assert a.tobytes() == b.tobytes(), f"{k}: max|d|={np.max(np.abs(a.astype(np.float64) - b))}"


def test_threads_do_not_change_bits():
    b1, b8 = CC.OracleCodecBackend(threads=1), CC.OracleCodecBackend(threads=5)
    x, w = S.f32_normal((3, 9), 1, 1.0), S.f32_normal((3, 2, 4), 2, 1.0)
    assert b1.conv_transpose(x, w, None, 2, 4, 2).tobytes() == b8.conv_transpose(x, w, None, 2, 4, 2).tobytes()
    q = S.f32_normal((9, 1024), 3, 1.0)
    sl = np.full(8, 0.25, np.float32)
    assert b1.alibi_attention(q, q, q, 9, 8, 8, 4, sl).tobytes() == b8.alibi_attention(q, q, q, 9, 8, 8, 4, sl).tobytes()


@pytest.mark.skipif(not S.have_ref(), reason="oracle/_ref not built (reference tree absent)")
def test_oracle_equals_compiled_reference_directly():
    a = CC.codec_cases(CC.RefCodecBackend())
    b = CC.codec_cases(CC.OracleCodecBackend(threads=8))
    for k in a:
        assert a[k].tobytes() == b[k].tobytes(), k


# ---- closed forms ---------------------------------------------------------------------------

def test_weight_norm_rows_have_length_g_and_direction_v():
    b = CC.OracleCodecBackend()
    v, g = S.f32_normal((6, 40), 5, 1.0), S.f32_normal(6, 6, 1.0)
    w = b.weight_norm(v, g).astype(np.float64)
    assert np.allclose(np.linalg.norm(w, axis=1), np.abs(g), rtol=1e-6)
    unit = v / np.linalg.norm(v.astype(np.float64), axis=1, keepdims=True)
    assert np.allclose(w, unit * g[:, None].astype(np.float64), rtol=1e-5, atol=1e-7)


def test_semantic_embedding_floor_and_alibi_slopes():
    o = K.bind_oracle()
    es = S.f32_normal((K.SEM_SIZE, K.SEM_DIM), 7, 1.0)
    usage = np.full(K.SEM_SIZE, 2.0, np.float32)
    usage[3] = 0.0
    usage[4] = 1e-7
    emb = np.zeros_like(es)
    o.orc_codec_semantic_embedding(S.fp(emb), S.fp(es), S.fp(usage))
    assert np.array_equal(emb[0], es[0] / np.float32(2.0))
    assert np.array_equal(emb[3], es[3] / np.float32(1e-5)) and np.array_equal(emb[4], es[4] / np.float32(1e-5))
    sl = np.zeros(8, np.float32)
    o.orc_codec_alibi_slopes(S.fp(sl))
    assert np.array_equal(sl, np.float32(2.0) ** -np.arange(1, 9, dtype=np.float32))


def test_conv1d_delta_taps_are_identity_and_reflected_shift():
    b = CC.OracleCodecBackend()
    n, k = 9, 5
    x = S.f32_normal((2, n), 8, 1.0)
    for tap in range(k):
        w = np.zeros((2, 2, k), np.float32)
        w[0, 1, tap] = 1.0                  # out channel 0 reads in channel 1
        w[1, 0, tap] = 1.0
        y = b.conv1d(x, w, None, 2, k, 1, n)
        src = np.abs(np.arange(n) + tap - (k - 1))   # causal: the last tap is "now"; before the start: mirrored
        assert np.array_equal(y[0], x[1][src]) and np.array_equal(y[1], x[0][src]), tap
    bias = np.array([0.5, -2.0], np.float32)
    y = b.conv1d(x, np.zeros((2, 2, k), np.float32), bias, 2, k, 1, n)
    assert np.array_equal(y, np.repeat(bias[:, None], n, 1))


def test_conv1d_stride2_against_float64():
    b = CC.OracleCodecBackend()
    ci, co, n, k, s = 3, 4, 10, 4, 2
    x, w = S.f32_normal((ci, n), 9, 1.0), S.f32_normal((co, ci, k), 10, 0.5)
    out_len = CC.conv1d_out_len(n, k, s)
    assert out_len == n // s
    y = b.conv1d(x, w, None, co, k, s, out_len)
    xp = np.pad(x.astype(np.float64), ((0, 0), (k - s, 0)), mode="reflect")
    ref = np.zeros((co, out_len))
    for ol in range(out_len):
        ref[:, ol] = np.einsum("oik,ik->o", w.astype(np.float64), xp[:, ol * s:ol * s + k])
    assert np.allclose(y, ref, rtol=1e-5, atol=1e-6)


def test_conv_transpose_delta_taps_place_samples():
    b = CC.OracleCodecBackend()
    n = 6
    x = S.f32_normal((2, n), 11, 1.0)
    for tap in range(4):
        w = np.zeros((2, 2, 4), np.float32)   # [in, out, tap]
        w[0, 1, tap] = 1.0
        w[1, 0, tap] = 1.0
        y = b.conv_transpose(x, w, None, 2, 4, 2)
        assert y.shape == (2, 2 * n)          # the two trailing raw samples are trimmed
        want = np.zeros((2, 2 * n + 2), np.float32)
        want[1, tap:tap + 2 * n:2] = x[0]
        want[0, tap:tap + 2 * n:2] = x[1]
        assert np.array_equal(y, want[:, :2 * n]), tap


def test_conv_transpose_against_float64_scatter():
    b = CC.OracleCodecBackend()
    ci, co, n = 5, 3, 7
    x, w = S.f32_normal((ci, n), 12, 1.0), S.f32_normal((ci, co, 4), 13, 0.5)
    bias = S.f32_normal(co, 14, 0.5)
    y = b.conv_transpose(x, w, bias, co, 4, 2)
    raw = np.zeros((co, 2 * n + 2))
    for il in range(n):
        raw[:, 2 * il:2 * il + 4] += np.einsum("i,iok->ok", x[:, il].astype(np.float64), w.astype(np.float64))
    assert np.allclose(y, raw[:, :2 * n] + bias[:, None], rtol=1e-5, atol=1e-6)


def alibi64(Q, Kk, V, window, slopes, heads=8, kv_heads=8):
    seq = Q.shape[0]
    out = np.zeros((seq, heads * 128))
    for h in range(heads):
        kv = h // (heads // kv_heads)
        q, k, v = (a.astype(np.float64)[:, i * 128:(i + 1) * 128] for a, i in ((Q, h), (Kk, kv), (V, kv)))
        for i in range(seq):
            j0 = max(0, i - window + 1) if window > 0 else 0
            j = np.arange(j0, i + 1)
            s = k[j] @ q[i] / np.sqrt(128.0) + float(slopes[h]) * (j - i)
            p = np.exp(s - s.max())
            out[i, h * 128:(h + 1) * 128] = (p / p.sum()) @ v[j]
    return out


def test_alibi_window_one_returns_the_value_row_and_zero_query_gives_geometric_weights():
    b = CC.OracleCodecBackend()
    seq = 7
    sl = np.float32(2.0) ** -np.arange(1, 9, dtype=np.float32)
    Q, Kk, V = (S.f32_normal((seq, 1024), 20 + i, 1.0) for i in range(3))
    assert np.array_equal(b.alibi_attention(Q, Kk, V, seq, 8, 8, 1, sl), V)
    # q = 0: the weight of key j is exp(slope (j - i)), a geometric sequence over the window
    out = b.alibi_attention(np.zeros_like(Q), Kk, V, seq, 8, 8, 3, sl)
    for h in (0, 7):
        r = np.exp(-float(sl[h]))
        w = np.array([r * r, r, 1.0])
        want = (w / w.sum()) @ V[4:7, h * 128:(h + 1) * 128].astype(np.float64)
        assert np.allclose(out[6, h * 128:(h + 1) * 128], want, rtol=1e-5, atol=1e-6)


def test_alibi_against_two_pass_softmax_in_float64():
    b = CC.OracleCodecBackend()
    seq = 13
    sl = np.float32(2.0) ** -np.arange(1, 9, dtype=np.float32)
    Q = S.f32_normal((seq, 1024), 30, 1.0)
    for kvh, window in ((8, 4), (8, 0), (2, 16)):
        Kk, V = S.f32_normal((seq, kvh * 128), 31, 1.0), S.f32_normal((seq, kvh * 128), 32, 1.0)
        got = b.alibi_attention(Q, Kk, V, seq, 8, kvh, window, sl)
        assert np.allclose(got, alibi64(Q, Kk, V, window, sl, 8, kvh), rtol=1e-4, atol=1e-5)


# ---- a float64 model of the whole decoder ------------------------------------------------------

def rms64(x, w, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def layer64(l, slopes, x):
    f = lambda a: a.astype(np.float64)
    xn = rms64(x, f(l.attention_norm), 1e-2)
    q, k, v = xn @ f(l.wq).T, xn @ f(l.wk).T, xn @ f(l.wv).T
    if l.q_norm is not None:
        q, k = rms64(q, f(l.q_norm), 1e-6), rms64(k, f(l.k_norm), 1e-6)
    att = alibi64(q, k, v, l.window, slopes)
    p = att @ f(l.wo).T
    x = x + (p * f(l.attn_scale) if l.attn_scale is not None else p)
    xn = rms64(x, f(l.ffn_norm), 1e-2)
    g, u = xn @ f(l.w1).T, xn @ f(l.w3).T
    p = (g / (1 + np.exp(-g)) * u) @ f(l.w2).T
    return x + (p * f(l.ffn_scale) if l.ffn_scale is not None else p)


def decode64(hc, codes):
    f = lambda a: a.astype(np.float64)
    n = codes.shape[0]
    sem = np.clip(codes[:, 0] - 2, 0, K.SEM_SIZE - 1)
    fsq = np.clip(codes[:, 1:] - 2, 0, K.LEVELS - 1) * 2.0 / (K.LEVELS - 1) - 1.0
    e = np.concatenate([f(hc.semantic_embedding)[sem], fsq], 1)          # [T, 292]

    def conv(x, cv):                                                         # token-major, stride 1
        k = cv.kernel
        w = f(cv.weight).reshape(cv.out_ch, cv.in_ch, k)
        idx = np.abs(np.arange(x.shape[0])[:, None] + np.arange(k)[None, :] - (k - 1))
        taps = np.where((idx < x.shape[0])[:, :, None], x[np.minimum(idx, x.shape[0] - 1)], 0.0)   # [T, k, C]
        y = np.einsum("tkc,ock->to", taps, w)
        return y + (f(cv.bias) if cv.bias is not None else 0.0)

    x = conv(e, hc.input_conv)
    for st in range(4):
        for l in hc.layers[2 * st:2 * st + 2]:
            x = layer64(l, hc.slopes, x)
        if st < 3:
            cv = hc.stage_convs[st]
            w = f(cv.weight).reshape(K.CDIM, K.CDIM, 4)                      # [in, out, tap]
            raw = np.zeros((2 * x.shape[0] + 2, K.CDIM))
            for tap in range(4):
                raw[tap:tap + 2 * x.shape[0]:2] += x @ w[:, :, tap]
            x = raw[:2 * x.shape[0]] + (f(cv.bias) if cv.bias is not None else 0.0)
    return conv(x, hc.output_proj).reshape(-1)


def test_decoder_against_float64_model():
    hc = K.HostCodec(9, distinct_layers=2)
    codes = K.random_codes(3, 90)
    b = CC.OracleCodecBackend(threads=8)
    b.open(hc)
    got = b.decode(codes)
    b.close()
    want = decode64(hc, codes)
    assert got.shape == want.shape == (3 * 8 * 240,)
    rms = np.sqrt(np.mean(want ** 2))
    assert np.abs(got - want).max() / rms < 2e-4
