"""Seeded cases shared by the fixture generator (make_golden.py, which runs
them on the COMPILED REFERENCE) and by the tests (which run them on the oracle
and compare bit-for-bit with the committed fixtures).

Inputs are regenerated from seeds; only outputs live in the fixtures.
"""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import vtsupport as S  # noqa: E402

N_DEC_LAYERS = 26      # the reference's layer count is a compile-time constant
KV_MAX = 16


class RefBackend:
    """Runs on oracle/_ref/libvoxtral_ref.so (the reference's own code)."""
    name = "reference"

    def __init__(self):
        self.lib = S.ref()

    def linear(self, x, W, bias, seq):
        out_dim, in_dim = W.shape
        y = np.zeros((seq, out_dim), np.float32)
        self.lib.tts_linear_bf16(S.fp(y), S.fp(x), S.up(W),
                                 S.fp(bias) if bias is not None else S.f32p(),
                                 seq, in_dim, out_dim)
        return y

    def rms_norm(self, x, w, seq):
        out = np.zeros_like(x)
        self.lib.tts_rms_norm(S.fp(out), S.fp(x), S.fp(w), seq, x.size // seq, S.EPS)
        return out

    def rope_freqs(self, pos):
        pos = np.asarray(pos, np.int32)
        f = np.zeros((len(pos), S.HEAD_DIM), np.float32)
        self.lib.tts_compute_rope_freqs(S.fp(f), S.ip(pos), len(pos), S.HEAD_DIM, S.THETA)
        return f

    def apply_rope(self, x, freqs, seq, heads):
        x = x.copy()
        self.lib.tts_apply_rope(S.fp(x), S.fp(freqs), seq, heads, S.HEAD_DIM)
        return x

    def causal_attention(self, Q, K, V, seq_q, seq_k, q_offset, heads=S.HEADS, kv_heads=S.KV_HEADS):
        out = np.zeros_like(Q)
        self.lib.tts_causal_attention(S.fp(out), S.fp(Q), S.fp(K), S.fp(V), seq_q, seq_k,
                                      heads, kv_heads, S.HEAD_DIM,
                                      1.0 / np.sqrt(np.float32(S.HEAD_DIM)), 0, q_offset)
        return out

    def bidir_attention(self, Q, K, V, seq):
        out = np.zeros_like(Q)
        self.lib.tts_bidirectional_attention(S.fp(out), S.fp(Q), S.fp(K), S.fp(V), seq,
                                             S.HEADS, S.KV_HEADS, S.HEAD_DIM,
                                             1.0 / np.sqrt(np.float32(S.HEAD_DIM)))
        return out

    def silu_mul(self, g, u):
        g = g.copy()
        self.lib.tts_silu(S.fp(g), g.size)
        self.lib.tts_mul_inplace(S.fp(g), S.fp(u), g.size)
        return g

    def add(self, a, b):
        a = a.copy()
        self.lib.tts_add_inplace(S.fp(a), S.fp(b), a.size)
        return a

    def rng(self, seed, n):
        st = C.c_uint64(0)
        self.lib.tts_rng_seed(C.byref(st), seed)
        buf = np.zeros(n, np.float32)
        self.lib.tts_randn_fill(C.byref(st), S.fp(buf), n)
        return buf, np.uint64(st.value)

    def embed_token(self, emb, tok):
        out = np.zeros(emb.shape[1], np.float32)
        self.lib.tts_embed_token_bf16(S.fp(out), S.up(emb), tok, emb.shape[1])
        return out

    # -- backbone session ---------------------------------------------------
    def llm_open(self, layers, final_norm, kv_max):
        self.ctx = self.lib.ref_ctx_new(kv_max)
        self.kv_max = kv_max
        self._keep = (layers, final_norm)
        n = S.ref_bind_decoder(self.ctx, layers, final_norm)
        assert n == N_DEC_LAYERS

    def llm_prefill(self, embeds):
        self.lib.ref_llm_prefill(self.ctx, S.fp(embeds), embeds.shape[0])

    def llm_forward(self, embed):
        out = np.zeros(S.DIM, np.float32)
        self.lib.ref_llm_forward(self.ctx, S.fp(embed), S.fp(out))
        return out

    def llm_kv(self):
        n = N_DEC_LAYERS * self.kv_max * S.KV_DIM
        k = np.ctypeslib.as_array(self.lib.ref_kv_k(self.ctx), (n,)).copy()
        v = np.ctypeslib.as_array(self.lib.ref_kv_v(self.ctx), (n,)).copy()
        shp = (N_DEC_LAYERS, self.kv_max, S.KV_DIM)
        return k.reshape(shp), v.reshape(shp)

    def llm_close(self):
        self.lib.ref_ctx_free(self.ctx)
        self.ctx = None

    # -- acoustic -------------------------------------------------------------
    def ac_open(self, ac):
        self.actx = self.lib.ref_ctx_new(0)
        self._keep_ac = ac
        S.ref_bind_acoustic(self.actx, ac)

    def predict_velocity(self, x_t, h, t):
        v = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.ref_predict_velocity(self.actx, S.fp(x_t), S.fp(h), t, S.fp(v))
        return v

    def time_embedding(self, t):
        out = np.zeros(S.DIM, np.float32)
        self.lib.ref_time_embedding(self.actx, t, S.fp(out))
        return out

    def acoustic_forward(self, h, seed=None):
        if seed is not None:
            self.lib.ref_seed(self.actx, seed)
        codes = np.zeros(S.CODES, np.int32)
        self.lib.ref_acoustic_forward(self.actx, S.fp(h), S.ip(codes))
        return codes, np.uint64(self.lib.ref_rng_state(self.actx))

    def audio_embed(self, emb, codes):
        self.lib.ref_audio_embed_set(self.actx, S.up(emb))
        out = np.zeros(S.DIM, np.float32)
        self.lib.ref_audio_embed_forward(self.actx, S.ip(codes), S.fp(out))
        return out

    def ac_close(self):
        self.lib.ref_ctx_free(self.actx)
        self.actx = None


class OracleBackend:
    """Runs on oracle/liboracle.so (our CPU restatement)."""
    name = "oracle"

    def __init__(self, threads=8):
        self.lib = S.oracle()
        self.lib.orc_set_threads(threads)

    def linear(self, x, W, bias, seq):
        out_dim, in_dim = W.shape
        y = np.zeros((seq, out_dim), np.float32)
        self.lib.orc_linear_bf16(S.fp(y), S.fp(x), S.up(W),
                                 S.fp(bias) if bias is not None else S.f32p(),
                                 seq, in_dim, out_dim)
        return y

    def rms_norm(self, x, w, seq):
        out = np.zeros_like(x)
        self.lib.orc_rms_norm(S.fp(out), S.fp(x), S.fp(w), seq, x.size // seq, S.EPS)
        return out

    def rope_freqs(self, pos):
        pos = np.asarray(pos, np.int32)
        f = np.zeros((len(pos), S.HEAD_DIM), np.float32)
        self.lib.orc_compute_rope_freqs(S.fp(f), S.ip(pos), len(pos), S.HEAD_DIM, S.THETA)
        return f

    def apply_rope(self, x, freqs, seq, heads):
        x = x.copy()
        self.lib.orc_apply_rope(S.fp(x), S.fp(freqs), seq, heads, S.HEAD_DIM)
        return x

    def causal_attention(self, Q, K, V, seq_q, seq_k, q_offset, heads=S.HEADS, kv_heads=S.KV_HEADS):
        out = np.zeros_like(Q)
        self.lib.orc_causal_attention(S.fp(out), S.fp(Q), S.fp(K), S.fp(V), seq_q, seq_k,
                                      heads, kv_heads, S.HEAD_DIM,
                                      1.0 / np.sqrt(np.float32(S.HEAD_DIM)), 0, q_offset)
        return out

    def bidir_attention(self, Q, K, V, seq):
        out = np.zeros_like(Q)
        self.lib.orc_bidirectional_attention(S.fp(out), S.fp(Q), S.fp(K), S.fp(V), seq,
                                             S.HEADS, S.KV_HEADS, S.HEAD_DIM,
                                             1.0 / np.sqrt(np.float32(S.HEAD_DIM)))
        return out

    def silu_mul(self, g, u):
        g = g.copy()
        self.lib.orc_silu(S.fp(g), g.size)
        self.lib.orc_mul_inplace(S.fp(g), S.fp(u), g.size)
        return g

    def add(self, a, b):
        a = a.copy()
        self.lib.orc_add_inplace(S.fp(a), S.fp(b), a.size)
        return a

    def rng(self, seed, n):
        st = C.c_uint64(0)
        self.lib.orc_rng_seed(C.byref(st), seed)
        buf = np.zeros(n, np.float32)
        self.lib.orc_randn_fill(C.byref(st), S.fp(buf), n)
        return buf, np.uint64(st.value)

    def embed_token(self, emb, tok):
        out = np.zeros(emb.shape[1], np.float32)
        self.lib.orc_embed_token_bf16(S.fp(out), S.up(emb), tok, emb.shape[1])
        return out

    def llm_open(self, layers, final_norm, kv_max, n_layers=N_DEC_LAYERS):
        self.n_layers = n_layers
        self.larr = S.orc_layers([layers[i % len(layers)] for i in range(n_layers)])
        self.final_norm = final_norm
        self.kv_max = kv_max
        self.kv_k = np.zeros((n_layers, kv_max, S.KV_DIM), np.float32)
        self.kv_v = np.zeros((n_layers, kv_max, S.KV_DIM), np.float32)
        self.pos = 0

    def llm_prefill(self, embeds, want_x=False):
        seq = embeds.shape[0]
        out_x = np.zeros((seq, S.DIM), np.float32) if want_x else None
        self.lib.orc_llm_prefill(self.larr, self.n_layers, S.fp(self.kv_k), S.fp(self.kv_v),
                                 self.kv_max, self.pos, S.fp(embeds), seq,
                                 S.fp(out_x) if want_x else S.f32p())
        self.pos += seq
        return out_x

    def llm_forward(self, embed):
        out = np.zeros(S.DIM, np.float32)
        self.lib.orc_llm_forward(self.larr, self.n_layers, S.fp(self.final_norm),
                                 S.fp(self.kv_k), S.fp(self.kv_v), self.kv_max, self.pos,
                                 S.fp(embed), S.fp(out))
        self.pos += 1
        return out

    def llm_kv(self):
        return self.kv_k.copy(), self.kv_v.copy()

    def llm_close(self):
        pass

    def ac_open(self, ac):
        self.ac = S.orc_acoustic(ac)
        self.rng_state = C.c_uint64(0)
        self.lib.orc_rng_seed(C.byref(self.rng_state), 0)

    def predict_velocity(self, x_t, h, t):
        v = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.orc_predict_velocity(C.byref(self.ac), S.fp(x_t), S.fp(h), t, S.fp(v))
        return v

    def time_embedding(self, t):
        out = np.zeros(S.DIM, np.float32)
        self.lib.orc_time_embedding(self.ac.time_inv_freq, t, S.fp(out), S.DIM)
        return out

    def acoustic_forward(self, h, seed=None, want_x=False):
        if seed is not None:
            self.lib.orc_rng_seed(C.byref(self.rng_state), seed)
        codes = np.zeros(S.CODES, np.int32)
        x = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.orc_acoustic_forward(C.byref(self.ac), S.fp(h), C.byref(self.rng_state),
                                      S.ip(codes), S.fp(x))
        if want_x:
            return codes, np.uint64(self.rng_state.value), x
        return codes, np.uint64(self.rng_state.value)

    def audio_embed(self, emb, codes):
        offs = np.zeros(S.CODES + 1, np.int32)
        offs[1] = 8194
        for i in range(2, S.CODES + 1):
            offs[i] = offs[i - 1] + 23
        out = np.zeros(S.DIM, np.float32)
        self.lib.orc_audio_embed_forward(S.up(emb), S.ip(offs), S.ip(codes), S.fp(out), S.DIM)
        return out

    def ac_close(self):
        pass


# --------------------------------------------------------------------------
# cases
# --------------------------------------------------------------------------

def kernel_cases(b):
    """Kernel-level known answers (small, fast)."""
    out = {}
    # matvec / linear: a 64-row slice of each config-1 shape, plus seq=3 with bias
    for name, (n, k) in dict(qkv=(64, 3072), down=(48, 9216), wo=(40, 4096), inp=(32, 36)).items():
        W = S.bf16_normal((n, k), 1000 + k + n)
        x = S.f32_normal((1, k), 42 + k)
        out[f"linear1_{name}"] = b.linear(x, W, None, 1)
    W = S.bf16_normal((56, 3072), 1200)
    x3 = S.f32_normal((3, 3072), 1100)
    bias = S.f32_normal(56, 1300, 0.1)
    out["linear3_bias"] = b.linear(x3, W, bias, 3)
    out["linear1_bias"] = b.linear(x3[:1].copy(), W, bias, 1)
    # row counts that are no multiple of anything: 13 and 57 output rows, 5 / 19 / 40 rows of x
    # (the oracle advances 8 output rows, or 8 / 32 rows of x, side by side)
    W = S.bf16_normal((13, 200), 1400)
    out["linear1_13rows"] = b.linear(S.f32_normal((1, 200), 1401), W, S.f32_normal(13, 1402, 0.1), 1)
    W = S.bf16_normal((57, 328), 1410)
    bias = S.f32_normal(57, 1411, 0.1)
    for seq in (5, 19, 40):
        out[f"linear{seq}_57rows"] = b.linear(S.f32_normal((seq, 328), 1420 + seq), W, bias if seq != 19 else None, seq)
    # rms norm
    x = S.f32_normal((3, S.DIM), 7)
    w = S.norm_weight(S.DIM, 8)
    out["rms_norm3"] = b.rms_norm(x, w, 3)
    out["rms_norm_zero"] = b.rms_norm(np.zeros((1, S.DIM), np.float32), w, 1)
    # rope
    pos = [0, 1, 7, 63, 513, 8191]
    fr = b.rope_freqs(pos)
    out["rope_freqs"] = fr
    q = S.f32_normal((len(pos), S.Q_DIM), 9)
    out["rope_q"] = b.apply_rope(q, fr, len(pos), S.HEADS)
    kk = S.f32_normal((len(pos), S.KV_DIM), 10)
    out["rope_k"] = b.apply_rope(kk, fr, len(pos), S.KV_HEADS)
    # attention (the reference test's seq_k values, test_kernels.c:463-468, data scale 0.1 and 1)
    for seq_k in (1, 3, 10, 50, 225):
        for std in (0.1, 1.0):
            Q = S.f32_normal((1, S.Q_DIM), 100 + seq_k, std)
            K = S.f32_normal((seq_k, S.KV_DIM), 200 + seq_k, std)
            V = S.f32_normal((seq_k, S.KV_DIM), 300 + seq_k, std)
            out[f"causal_{seq_k}_{std}"] = b.causal_attention(Q, K, V, 1, seq_k, seq_k - 1)
    Q = S.f32_normal((6, S.Q_DIM), 400)
    K = S.f32_normal((9, S.KV_DIM), 401)
    V = S.f32_normal((9, S.KV_DIM), 402)
    out["causal_prefill_6_off3"] = b.causal_attention(Q, K, V, 6, 9, 3)
    Q = S.f32_normal((3, S.Q_DIM), 500)
    K = S.f32_normal((3, S.KV_DIM), 600)
    V = S.f32_normal((3, S.KV_DIM), 700)
    out["bidir_3"] = b.bidir_attention(Q, K, V, 3)
    # swiglu, residual
    g = S.f32_normal(S.FFN, 800, 2.0)
    u = S.f32_normal(S.FFN, 900)
    out["silu_mul"] = b.silu_mul(g, u)
    out["add"] = b.add(g, u)
    # rng: floats and the integer state after n draws
    for seed in (0, 1, 42, 0xDEADBEEF):
        vals, st = b.rng(seed, 72)
        out[f"rng_{seed}"] = vals
        out[f"rng_state_{seed}"] = np.array([st], np.uint64)
    emb = S.bf16_normal((50, S.DIM), 77, 1.0)
    out["embed_tok"] = b.embed_token(emb, 33)
    return out


def llm_cases(b, n_prefill=3, n_steps=2):
    """26-layer backbone cycling over 2 distinct synthetic layers:
    prefill n_prefill rows, then n_steps decode steps."""
    layers = [S.Layer(1), S.Layer(2)]
    final_norm = S.norm_weight(S.DIM, 99)
    b.llm_open(layers, final_norm, KV_MAX)
    out = {}
    if n_prefill:
        emb = S.f32_normal((n_prefill, S.DIM), 5)
        b.llm_prefill(emb)
    hs = []
    e = S.f32_normal(S.DIM, 6)
    for _ in range(n_steps):
        h = b.llm_forward(e)
        hs.append(h)
        e = h.copy()            # feed the hidden straight back
    out["hidden"] = np.stack(hs)
    k, v = b.llm_kv()
    n = n_prefill + n_steps
    for l in (0, 1, 12, 25):
        out[f"kv_k_l{l}"] = k[l, :n].copy()
        out[f"kv_v_l{l}"] = v[l, :n].copy()
    b.llm_close()
    return out


def acoustic_cases(b, n_frames=2):
    ac = S.Acoustic(50)
    b.ac_open(ac)
    out = {}
    out["time_emb"] = np.stack([b.time_embedding(np.float32(i) / np.float32(7)) for i in (0, 3, 6)])
    x = S.f32_normal(S.ACOUSTIC_DIM, 11)
    h = S.f32_normal(S.DIM, 12)
    out["vel_cond"] = b.predict_velocity(x, h, np.float32(3) / np.float32(7))
    out["vel_uncond"] = b.predict_velocity(x, np.zeros(S.DIM, np.float32), np.float32(3) / np.float32(7))
    codes, states = [], []
    for f in range(n_frames):
        hf = S.f32_normal(S.DIM, 20 + f)
        c, st = b.acoustic_forward(hf, seed=42 if f == 0 else None)
        codes.append(c)
        states.append(st)
    out["codes"] = np.stack(codes)
    out["rng_states"] = np.array(states, np.uint64)
    # END_AUDIO path: a huge bias on index 1 forces code 1 and draws no noise
    emb = S.bf16_normal((8194 + 36 * 23, S.DIM), 60, 1.0)
    out["audio_embed"] = b.audio_embed(emb, codes[0])
    b.ac_close()
    ac.semantic_out_bias = ac.semantic_out_bias.copy()
    ac.semantic_out_bias[1] = 1e9
    b.ac_open(ac)
    c, st = b.acoustic_forward(S.f32_normal(S.DIM, 30), seed=7)
    out["codes_end"] = c
    out["rng_state_end"] = np.array([st], np.uint64)
    b.ac_close()
    return out
