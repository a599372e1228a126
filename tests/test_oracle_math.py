"""Pins of the oracle that do not depend on the reference at all: closed forms,
invariants and brute force in float64, each chosen so that a plausible mistake
(dropped term, wrong sign or index, transposed operand, wrong head mapping)
fails."""
import ctypes as C

import numpy as np

import cases
import vtsupport as S

B = cases.OracleBackend(threads=1)


def test_linear_one_hot_rows_pick_x_and_bias_is_added():
    W = np.zeros((5, 36), np.float32)
    for r in range(5):
        W[r, 7 * r] = 1.0
    x = S.f32_normal((1, 36), 1)
    bias = S.f32_normal(5, 2)
    y = B.linear(x, S.f32_to_bf16_trunc(W), bias, 1)[0]
    assert np.array_equal(y, x[0, ::7][:5] + bias)


def test_linear_against_float64_and_not_transposed():
    W = S.bf16_normal((17, 100), 3, 1.0)
    x = S.f32_normal((3, 100), 4)
    y = B.linear(x, W, None, 3)
    ref = x.astype(np.float64) @ S.bf16_to_f32(W).astype(np.float64).T
    assert y.shape == (3, 17)
    assert np.max(np.abs(y - ref)) < 1e-4


def test_rms_norm_constant_vector_closed_form():
    c = np.float32(3.0)
    x = np.full((1, S.DIM), c, np.float32)
    w = S.norm_weight(S.DIM, 5)
    out = B.rms_norm(x, w, 1)[0]
    expect = c / np.sqrt(np.float64(c) ** 2 + 1e-5) * w.astype(np.float64)
    assert np.max(np.abs(out - expect)) < 1e-5
    assert not np.any(B.rms_norm(np.zeros((1, S.DIM), np.float32), w, 1))


def test_rope_identity_at_pos0_norm_preserving_and_angle():
    fr = B.rope_freqs([0, 5])
    assert np.array_equal(fr[0, 0::2], np.ones(64, np.float32))
    assert np.array_equal(fr[0, 1::2], np.zeros(64, np.float32))
    # pair d=0 has frequency 1: angle == pos
    assert abs(fr[1, 0] - np.cos(5.0)) < 1e-6 and abs(fr[1, 1] - np.sin(5.0)) < 1e-6
    # last pair: theta^(-126/128)
    ang = 5.0 * 1e6 ** (-126.0 / 128.0)
    assert abs(fr[1, 126] - np.cos(ang)) < 1e-6 and abs(fr[1, 127] - np.sin(ang)) < 1e-6
    x = S.f32_normal((2, S.KV_DIM), 6)
    y = B.apply_rope(x, fr, 2, S.KV_HEADS)
    assert np.array_equal(y[0], x[0])
    n0 = x[1].reshape(-1, 2).astype(np.float64)
    n1 = y[1].reshape(-1, 2).astype(np.float64)
    assert np.allclose((n0 ** 2).sum(1), (n1 ** 2).sum(1), rtol=1e-5)
    # rotation direction: (1,0) at angle a -> (cos a, sin a), adjacent pairs
    e = np.zeros((2, S.KV_DIM), np.float32)
    e[1, 0] = 1.0
    r = B.apply_rope(e, fr, 2, S.KV_HEADS)
    assert abs(r[1, 0] - np.cos(5.0)) < 1e-6 and abs(r[1, 1] - np.sin(5.0)) < 1e-6


def _softmax_attention64(Q, K, V, causal_offset=None):
    seq_q = Q.shape[0]
    out = np.zeros((seq_q, S.Q_DIM))
    for h in range(S.HEADS):
        kh = h // 4
        q = Q[:, h * 128:(h + 1) * 128].astype(np.float64)
        k = K[:, kh * 128:(kh + 1) * 128].astype(np.float64)
        v = V[:, kh * 128:(kh + 1) * 128].astype(np.float64)
        s = q @ k.T / np.sqrt(128.0)
        if causal_offset is not None:
            for i in range(seq_q):
                s[i, causal_offset + i + 1:] = -np.inf
        p = np.exp(s - s.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        out[:, h * 128:(h + 1) * 128] = p @ v
    return out


def test_attention_single_key_returns_value_row_with_gqa_mapping():
    Q = S.f32_normal((1, S.Q_DIM), 7)
    K = S.f32_normal((1, S.KV_DIM), 8)
    V = S.f32_normal((1, S.KV_DIM), 9)
    out = B.causal_attention(Q, K, V, 1, 1, 0)[0]
    for h in range(S.HEADS):
        assert np.array_equal(out[h * 128:(h + 1) * 128], V[0, (h // 4) * 128:(h // 4 + 1) * 128])


def test_attention_equal_keys_give_mean_of_values():
    Q = S.f32_normal((1, S.Q_DIM), 10)
    K = np.tile(S.f32_normal((1, S.KV_DIM), 11), (6, 1))
    V = S.f32_normal((6, S.KV_DIM), 12)
    out = B.causal_attention(Q, K, V, 1, 6, 5)[0].reshape(S.HEADS, 128)
    mean = V.astype(np.float64).mean(0).reshape(S.KV_HEADS, 128)
    for h in range(S.HEADS):
        assert np.max(np.abs(out[h] - mean[h // 4])) < 1e-5


def test_attention_matches_two_pass_softmax_in_float64():
    Q = S.f32_normal((4, S.Q_DIM), 13)
    K = S.f32_normal((7, S.KV_DIM), 14)
    V = S.f32_normal((7, S.KV_DIM), 15)
    got = B.causal_attention(Q, K, V, 4, 7, 3)
    assert np.max(np.abs(got - _softmax_attention64(Q, K, V, 3))) < 1e-4
    Q3, K3, V3 = Q[:3].copy(), K[:3].copy(), V[:3].copy()
    got = B.bidir_attention(Q3, K3, V3, 3)
    assert np.max(np.abs(got - _softmax_attention64(Q3, K3, V3))) < 1e-4


def test_silu_limits():
    g = np.array([0.0, 50.0, -50.0, 1.0], np.float32)
    u = np.array([3.0, 2.0, 2.0, 1.0], np.float32)
    out = B.silu_mul(g, u)
    assert out[0] == 0.0 and out[1] == 100.0 and abs(out[2]) < 1e-18
    assert abs(out[3] - 1.0 / (1.0 + np.exp(-1.0))) < 1e-7


def test_rng_integer_state_is_xorshift_13_7_17():
    m = (1 << 64) - 1
    s = 0x12345678ABCDEF01         # seed 0 maps to this constant
    draws = 0
    vals, st = B.rng(0, 5)
    # replay: each normal consumes two uniforms (rejections are astronomically rare)
    for _ in range(10):
        s ^= (s << 13) & m
        s ^= s >> 7
        s ^= (s << 17) & m
        draws += 1
    assert int(st) == s
    big, _ = B.rng(123, 20000)
    assert abs(float(big.mean())) < 0.03 and abs(float(big.std()) - 1.0) < 0.03


def test_fsq_and_argmax_rules():
    """Semantic argmax keeps the FIRST maximum; masked slots can never win;
    END (code 1) yields 36 codes of value 2 and draws no noise."""
    ac = S.Acoustic(51, n_layers=0, bias=True)
    ac.semantic_out = np.zeros_like(ac.semantic_out)        # logits == bias
    ac.semantic_out_bias = np.zeros(S.SEM_PADDED, np.float32)
    ac.semantic_out_bias[[0, 5, 9, 8200]] = [9.0, 4.0, 4.0, 8.0]   # 0 and 8200 are masked
    B.ac_open(ac)
    h = S.f32_normal(S.DIM, 16)
    codes, st, x = B.acoustic_forward(h, seed=3, want_x=True)
    assert codes[0] == 5
    expect = np.clip(x, -1, 1)
    expect = ((expect + np.float32(1)) / np.float32(2) * np.float32(20) + np.float32(0.5)).astype(np.int32) + 2
    assert np.array_equal(codes[1:], expect)
    assert codes[1:].min() >= 2 and codes[1:].max() <= 22
    ac.semantic_out_bias[1] = 10.0
    B.ac_open(ac)
    st0 = C.c_uint64(0)
    S.oracle().orc_rng_seed(C.byref(st0), 3)
    codes, st = B.acoustic_forward(h, seed=3)
    assert codes[0] == 1 and np.all(codes[1:] == 2) and int(st) == st0.value


def test_audio_embed_sum_uses_cumulative_offsets():
    emb = np.zeros((8194 + 36 * 23, S.DIM), np.float32)
    codes = np.arange(2, 2 + S.CODES, dtype=np.int32) % 20 + 2
    rows = [codes[0]] + [8194 + 23 * (cb - 1) + codes[cb] for cb in range(1, S.CODES)]
    for i, r in enumerate(rows):
        emb[r, i] = 1.0
    out = B.audio_embed(S.f32_to_bf16_trunc(emb), codes)
    assert np.array_equal(out[:S.CODES], np.ones(S.CODES, np.float32))
    assert not np.any(out[S.CODES:])


def _check_time_inv_freq(f):
    """What the mathematics fixes for f[i] = exp(-log(10000) i / 1536) evaluated in fp32
    (voxtral_tts_acoustic.c:48-60): f[0] is exactly 1; the fp32 argument (-logf(1e4) * i) / 1536
    carries at most three roundings (logf, product, quotient: 3 * 2^-24 relative, |argument| <= 9.21,
    so 1.65e-6 absolute), expf adds an ulp: every entry lies within 2e-6 relative of the float64
    value.  An index off by one is 6e-3 away, a dropped sign or a wrong base much more."""
    half = S.DIM // 2
    assert f.shape == (half,) and f.dtype == np.float32
    assert f[0] == np.float32(1.0)
    ref = np.exp(-np.log(10000.0) * np.arange(half, dtype=np.float64) / half)
    assert np.max(np.abs(f.astype(np.float64) / ref - 1.0)) < 2e-6
    assert np.all(np.diff(f) < 0)
    assert abs(float(f[half - 1]) - 1.0060e-4) < 1e-8
    assert abs(float(f[half // 2]) - 1e-2) < 1e-7          # the middle entry is 10000^-0.5


def test_default_time_inv_freq_closed_form():
    f = np.zeros(S.DIM // 2, np.float32)
    S.oracle().orc_default_time_inv_freq(S.fp(f), S.DIM // 2)
    _check_time_inv_freq(f)


def test_time_embedding_is_cos_then_sin_of_t_times_freq():
    """out[i] = cos(t f_i), out[1536 + i] = sin(t f_i) (voxtral_tts_acoustic.c:166-176), against
    float64 on a table pinned above; t = 0 gives (1, 0)."""
    f = np.zeros(S.DIM // 2, np.float32)
    S.oracle().orc_default_time_inv_freq(S.fp(f), S.DIM // 2)
    out = np.zeros(S.DIM, np.float32)
    S.oracle().orc_time_embedding(S.fp(f), np.float32(0.0), S.fp(out), S.DIM)
    assert np.array_equal(out[:S.DIM // 2], np.ones(S.DIM // 2, np.float32)) and not np.any(out[S.DIM // 2:])
    t = np.float32(3) / np.float32(7)
    S.oracle().orc_time_embedding(S.fp(f), t, S.fp(out), S.DIM)
    ang = (t * f).astype(np.float64)
    assert np.max(np.abs(out[:S.DIM // 2] - np.cos(ang))) < 1e-6
    assert np.max(np.abs(out[S.DIM // 2:] - np.sin(ang))) < 1e-6
