"""Seeded cases of the audio codec decoder, shared by the fixture generator (which runs them
on the COMPILED REFERENCE) and by the tests (which run them on the oracle and compare bit for
bit with the committed fixture codec.npz).  Inputs are regenerated from seeds."""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import codecsupport as K  # noqa: E402
import vtsupport as S  # noqa: E402


def _opt(a):
    return S.fp(a) if a is not None else S.f32p()


class RefCodecBackend:
    """The reference's own functions (oracle/_ref/libvoxtral_ref.so)."""

    def __init__(self):
        self.lib = K.bind_ref()
        self.ctx = None

    def weight_norm(self, v, g):
        w = np.zeros_like(v)
        self.lib.ref_weight_norm(S.fp(w), S.fp(v), S.fp(g), v.shape[0], v.shape[1])
        return w

    def conv1d(self, x, w, bias, ch_out, kernel, stride, out_len):
        ch_in, length = x.shape
        out = np.zeros((ch_out, out_len), np.float32)
        self.lib.tts_causal_conv1d(S.fp(out), S.fp(x), S.fp(w), _opt(bias), ch_in, ch_out, length, kernel, stride)
        return out

    def conv_transpose(self, x, w, bias, ch_out, kernel, stride):
        ch_in, length = x.shape
        out = np.zeros((ch_out, length * stride + kernel + 8), np.float32)
        n = C.c_int(0)
        self.lib.tts_causal_conv_transpose_1d(S.fp(out), S.fp(x), S.fp(w), _opt(bias), ch_in, ch_out, length,
                                              kernel, stride, C.byref(n))
        return np.ascontiguousarray(out.reshape(-1)[:ch_out * n.value].reshape(ch_out, n.value))

    def alibi_attention(self, Q, K_, V, seq, heads, kv_heads, window, slopes):
        out = np.zeros_like(Q)
        self.lib.tts_alibi_attention(S.fp(out), S.fp(Q), S.fp(K_), S.fp(V), seq, heads, kv_heads, 128,
                                     1.0 / np.sqrt(np.float32(128)), window, S.fp(slopes))
        return out

    def linear(self, x, W):
        y = np.zeros((x.shape[0], W.shape[0]), np.float32)
        self.lib.tts_linear_nobias(S.fp(y), S.fp(x), S.fp(W), x.shape[0], x.shape[1], W.shape[0])
        return y

    def open(self, hc):
        self.ctx = S.ref().ref_ctx_new(0)
        K.ref_bind_codec(self.ctx, hc)
        self._keep = hc

    def embed(self, codes):
        n = codes.shape[0]
        out = np.zeros((K.EMBED, n), np.float32)
        self.lib.ref_codec_embed_codes(self.ctx, S.ip(codes.reshape(-1).copy()), n, S.fp(out))
        return out

    def layer(self, i, x):
        x = x.copy()
        self.lib.ref_codec_layer(self.ctx, i, S.fp(x), x.shape[0])
        return x

    def decode(self, codes):
        n = codes.shape[0]
        out = np.zeros(n * K.UPSAMPLE * K.PATCH, np.float32)
        got = self.lib.ref_codec_decode(self.ctx, S.ip(codes.reshape(-1).copy()), n, S.fp(out))
        return out[:got].copy()

    def close(self):
        S.ref().ref_ctx_free(self.ctx)
        self.ctx = None


class OracleCodecBackend:
    """Our restatement (oracle/vt_oracle_codec.c)."""

    def __init__(self, threads=8):
        self.lib = K.bind_oracle()
        self.threads = threads
        self.cs = None

    def _t(self):
        self.lib.orc_set_threads(self.threads)

    def weight_norm(self, v, g):
        w = np.zeros_like(v)
        self.lib.orc_weight_norm(S.fp(w), S.fp(v), S.fp(g), v.shape[0], v.shape[1])
        return w

    def conv1d(self, x, w, bias, ch_out, kernel, stride, out_len):
        self._t()
        ch_in, length = x.shape
        out = np.zeros((ch_out, out_len), np.float32)
        n = self.lib.orc_causal_conv1d(S.fp(out), S.fp(x), S.fp(w), _opt(bias), ch_in, ch_out, length, kernel, stride)
        assert n == out_len
        return out

    def conv_transpose(self, x, w, bias, ch_out, kernel, stride):
        self._t()
        ch_in, length = x.shape
        out = np.zeros((ch_out, length * stride + kernel + 8), np.float32)
        n = self.lib.orc_causal_conv_transpose_1d(S.fp(out), S.fp(x), S.fp(w), _opt(bias), ch_in, ch_out, length,
                                                  kernel, stride)
        return np.ascontiguousarray(out.reshape(-1)[:ch_out * n].reshape(ch_out, n))

    def alibi_attention(self, Q, K_, V, seq, heads, kv_heads, window, slopes):
        self._t()
        out = np.zeros_like(Q)
        self.lib.orc_alibi_attention(S.fp(out), S.fp(Q), S.fp(K_), S.fp(V), seq, heads, kv_heads, 128,
                                     1.0 / np.sqrt(np.float32(128)), window, S.fp(slopes))
        return out

    def linear(self, x, W):
        self._t()
        y = np.zeros((x.shape[0], W.shape[0]), np.float32)
        self.lib.orc_linear_f32(S.fp(y), S.fp(x), S.fp(W), x.shape[0], x.shape[1], W.shape[0])
        return y

    def open(self, hc):
        self.cs = hc.struct()

    def embed(self, codes):
        n = codes.shape[0]
        out = np.zeros((K.EMBED, n), np.float32)
        self.lib.orc_codec_embed_codes(self.cs.semantic_embedding, S.ip(codes.reshape(-1).copy()), n, S.fp(out))
        return out

    def layer(self, i, x):
        self._t()
        x = x.copy()
        self.lib.orc_codec_layer(C.byref(self.cs.layers[i]), self.cs.alibi_slopes, S.fp(x), x.shape[0])
        return x

    def decode(self, codes):
        self._t()
        return K.oracle_decode(self.cs, codes)

    def close(self):
        self.cs = None
        self.lib.orc_set_threads(1)


def conv1d_out_len(length, kernel, stride):
    """Output length of the causal convolution (voxtral_tts_kernels.c:231-234)."""
    pad = kernel - stride
    return int(np.ceil(np.float32(length - kernel + pad) / np.float32(stride) + np.float32(1.0)))


def codec_cases(b):
    out = {}
    v, g = S.f32_normal((5, 12), 1, 1.0), S.f32_normal(5, 2, 1.0)
    out["weight_norm"] = b.weight_norm(v, g)
    # convolutions: stride 1 and 2, reflection on both sides, inputs shorter than the kernel
    for name, (ci, co, n, k, s, bias) in {"conv_k3s1": (3, 4, 7, 3, 1, True), "conv_k4s2": (3, 2, 9, 4, 2, True),
                                          "conv_k7s1_short": (2, 3, 2, 7, 1, False),
                                          "conv_k3s1_len1": (2, 2, 1, 3, 1, True)}.items():
        x = S.f32_normal((ci, n), 10 + k, 1.0)
        w = S.f32_normal((co, ci, k), 20 + k, 0.5)
        bv = S.f32_normal(co, 30 + k, 0.5) if bias else None
        out[name] = b.conv1d(x, w, bv, co, k, s, conv1d_out_len(n, k, s))
    for name, (ci, co, n, k, s, bias) in {"convt_k4s2": (3, 2, 5, 4, 2, True), "convt_k3s1": (2, 3, 4, 3, 1, False),
                                          "convt_k4s2_len1": (2, 2, 1, 4, 2, True)}.items():
        x = S.f32_normal((ci, n), 40 + k, 1.0)
        w = S.f32_normal((ci, co, k), 50 + k, 0.5)
        bv = S.f32_normal(co, 60 + k, 0.5) if bias else None
        out[name] = b.conv_transpose(x, w, bv, co, k, s)
    slopes = np.zeros(8, np.float32)
    K.bind_oracle().orc_codec_alibi_slopes(S.fp(slopes))
    seq = 11
    Q = S.f32_normal((seq, 8 * 128), 70, 1.0)
    for name, (kvh, window) in {"alibi_w4": (8, 4), "alibi_w1": (8, 1), "alibi_full": (8, 0),
                                "alibi_gqa_w16": (2, 16)}.items():
        Kk, V = S.f32_normal((seq, kvh * 128), 71, 1.0), S.f32_normal((seq, kvh * 128), 72, 1.0)
        out[name] = b.alibi_attention(Q, Kk, V, seq, 8, kvh, window, slopes)
    out["linear_f32"] = b.linear(S.f32_normal((3, 96), 80, 1.0), S.f32_normal((5, 96), 81, 0.1))
    # the model: one layer of each window, then codes -> waveform
    hc = K.HostCodec(9, distinct_layers=2)
    b.open(hc)
    codes = K.random_codes(4, 90)
    out["embed"] = b.embed(codes)
    x = S.f32_normal((6, K.CDIM), 91, 1.0)
    out["layer0_w2"] = b.layer(0, x)
    out["layer7_w16"] = b.layer(7, S.f32_normal((19, K.CDIM), 92, 1.0))
    out["wave_3"] = b.decode(codes[:3])
    out["wave_1"] = b.decode(codes[3:4])
    b.close()
    hc2 = K.HostCodec(10, distinct_layers=1, qk_norm=False, layer_scale=False, bias=False)
    hc2.layers[0].wo *= np.float32(0.3)
    hc2.layers[0].w2 *= np.float32(0.3)
    b.open(hc2)
    out["wave_plain_2"] = b.decode(K.random_codes(2, 93))
    b.close()
    return out
