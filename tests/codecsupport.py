"""Synthetic weights and checker bindings for the audio codec decoder (codes -> waveform).
The ctypes structs below have the layout of the reference's tts_conv_t / tts_codec_layer_t /
tts_codec_t (voxtral_tts.h:172-225), which the oracle's and the HIP library's structs share."""
import ctypes as C

import numpy as np

import vtsupport as S

f32p, i32p = S.f32p, S.i32p
CDIM, CHID, CHEADS, CHEAD_DIM = 1024, 4096, 8, 128
EMBED, SEM_DIM, SEM_SIZE, PATCH, LEVELS = 292, 256, 8192, 240, 21
WINDOWS = (2, 4, 8, 16)
UPSAMPLE = 8


class Conv(C.Structure):
    _fields_ = [("weight", f32p), ("bias", f32p), ("in_ch", C.c_int), ("out_ch", C.c_int),
                ("kernel", C.c_int), ("stride", C.c_int), ("is_transpose", C.c_int)]


class CodecLayer(C.Structure):
    _fields_ = [("wq", f32p), ("wk", f32p), ("wv", f32p), ("wo", f32p), ("q_norm", f32p),
                ("k_norm", f32p), ("attention_norm", f32p), ("w1", f32p), ("w2", f32p), ("w3", f32p),
                ("ffn_norm", f32p), ("attn_scale", f32p), ("ffn_scale", f32p), ("window_size", C.c_int)]


class Codec(C.Structure):
    _fields_ = [("semantic_embedding", f32p), ("input_conv", Conv), ("layers", CodecLayer * 8),
                ("stage_convs", Conv * 4), ("output_proj", Conv), ("alibi_slopes", C.c_float * 8)]


def _opt(a):
    return S.fp(a) if a is not None else f32p()


class HostConv:
    """Weight-normed convolution: v, g random; the effective weight comes from the oracle's
    restatement of the reference's reconstruction."""

    def __init__(self, seed, in_ch, out_ch, kernel, stride, transpose, bias=True, gain=1.0):
        rows, fan_in = (in_ch, out_ch * kernel) if transpose else (out_ch, in_ch * kernel)
        self.v = S.f32_normal((rows, fan_in), seed, 1.0)
        self.g = (np.abs(S.f32_normal(rows, seed + 1, 0.25)) + np.float32(0.75)) * np.float32(gain)
        self.g = self.g.astype(np.float32)
        self.weight = np.zeros((rows, fan_in), np.float32)
        S.oracle().orc_weight_norm(S.fp(self.weight), S.fp(self.v), S.fp(self.g), rows, fan_in)
        self.bias = S.f32_normal(out_ch, seed + 2, 0.1) if bias else None
        self.in_ch, self.out_ch, self.kernel, self.stride, self.transpose = in_ch, out_ch, kernel, stride, transpose

    def struct(self):
        return Conv(S.fp(self.weight), _opt(self.bias), self.in_ch, self.out_ch, self.kernel, self.stride,
                    int(self.transpose))


class HostCodecLayer:
    def __init__(self, seed, window, qk_norm=True, layer_scale=True):
        n = lambda shape, i, std: S.f32_normal(shape, seed * 32 + i, std)
        self.wq, self.wk = n((CDIM, CDIM), 0, 0.03), n((CDIM, CDIM), 1, 0.03)
        self.wv, self.wo = n((CDIM, CDIM), 2, 0.03), n((CDIM, CDIM), 3, 0.03)
        self.w1, self.w3 = n((CHID, CDIM), 4, 0.03), n((CHID, CDIM), 5, 0.03)
        self.w2 = n((CDIM, CHID), 6, 0.02)
        self.attention_norm = S.norm_weight(CDIM, seed * 32 + 7)
        self.ffn_norm = S.norm_weight(CDIM, seed * 32 + 8)
        self.q_norm = S.norm_weight(CDIM, seed * 32 + 9) if qk_norm else None
        self.k_norm = S.norm_weight(CDIM, seed * 32 + 10) if qk_norm else None
        self.attn_scale = (S.norm_weight(CDIM, seed * 32 + 11) * np.float32(0.5)) if layer_scale else None
        self.ffn_scale = (S.norm_weight(CDIM, seed * 32 + 12) * np.float32(0.5)) if layer_scale else None
        self.window = window

    def struct(self):
        return CodecLayer(S.fp(self.wq), S.fp(self.wk), S.fp(self.wv), S.fp(self.wo), _opt(self.q_norm),
                          _opt(self.k_norm), S.fp(self.attention_norm), S.fp(self.w1), S.fp(self.w2),
                          S.fp(self.w3), S.fp(self.ffn_norm), _opt(self.attn_scale), _opt(self.ffn_scale),
                          self.window)


class HostCodec:
    """All weights of the codec decoder.  `distinct_layers` < 8 cycles layer weights (pointers
    alias) to keep generation short; windows always follow the stage."""

    def __init__(self, seed, distinct_layers=8, qk_norm=True, layer_scale=True, bias=True):
        o = S.oracle()
        self.emb_sum = S.f32_normal((SEM_SIZE, SEM_DIM), seed * 64 + 1, 1.0)
        usage = np.abs(S.f32_normal(SEM_SIZE, seed * 64 + 2, 1.0)).astype(np.float32)
        usage[::97] = 0.0                       # unused clusters hit the 1e-5 floor
        self.cluster_usage = usage
        self.semantic_embedding = np.zeros((SEM_SIZE, SEM_DIM), np.float32)
        o.orc_codec_semantic_embedding(S.fp(self.semantic_embedding), S.fp(self.emb_sum), S.fp(usage))
        # keep the table O(1): entries of unused clusters are huge otherwise
        np.clip(self.semantic_embedding, -4.0, 4.0, out=self.semantic_embedding)
        self.slopes = np.zeros(CHEADS, np.float32)
        o.orc_codec_alibi_slopes(S.fp(self.slopes))
        self.input_conv = HostConv(seed * 64 + 3, EMBED, CDIM, 3, 1, False, bias, 0.05)
        base = [HostCodecLayer(seed * 64 + 8 + i, 0, qk_norm, layer_scale) for i in range(distinct_layers)]
        self.layers = []
        for i in range(8):
            l = HostCodecLayer.__new__(HostCodecLayer)
            l.__dict__.update(base[i % distinct_layers].__dict__)
            l.window = WINDOWS[i // 2]
            self.layers.append(l)
        self.stage_convs = [HostConv(seed * 64 + 20 + 3 * i, CDIM, CDIM, 4, 2, True, bias, 1.0) for i in range(3)]
        self.output_proj = HostConv(seed * 64 + 40, CDIM, PATCH, 7, 1, False, bias, 0.05)

    def struct(self):
        c = Codec()
        c.semantic_embedding = S.fp(self.semantic_embedding)
        c.input_conv = self.input_conv.struct()
        for i, l in enumerate(self.layers):
            c.layers[i] = l.struct()
        for i, cv in enumerate(self.stage_convs):
            c.stage_convs[i] = cv.struct()
        c.output_proj = self.output_proj.struct()
        for h in range(CHEADS):
            c.alibi_slopes[h] = self.slopes[h]
        c._keep = self
        return c


def random_codes(n_frames, seed, edge=True):
    r = np.random.default_rng(seed)
    codes = np.zeros((n_frames, S.CODES), np.int32)
    codes[:, 0] = r.integers(2, 2 + SEM_SIZE, n_frames)
    codes[:, 1:] = r.integers(2, 2 + LEVELS, (n_frames, S.CODES - 1))
    if edge and n_frames >= 3:
        codes[1, 0] = 0               # special ids clamp to code 0
        codes[1, 5] = 1
        codes[2, 0] = 2 + SEM_SIZE    # beyond the table: clamps to the last code
        codes[2, 7] = 40
    return codes


def bind_oracle():
    o = S.oracle()
    o.orc_weight_norm.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int]
    o.orc_codec_semantic_embedding.argtypes = [f32p, f32p, f32p]
    o.orc_codec_alibi_slopes.argtypes = [f32p]
    o.orc_linear_f32.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    o.orc_causal_conv1d.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5
    o.orc_causal_conv1d.restype = C.c_int
    o.orc_causal_conv_transpose_1d.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5
    o.orc_causal_conv_transpose_1d.restype = C.c_int
    o.orc_alibi_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 4 + [C.c_float, C.c_int, f32p]
    o.orc_codec_embed_codes.argtypes = [f32p, i32p, C.c_int, f32p]
    o.orc_codec_layer.argtypes = [C.POINTER(CodecLayer), f32p, f32p, C.c_int]
    o.orc_codec_decode.argtypes = [C.POINTER(Codec), i32p, C.c_int, f32p]
    o.orc_codec_decode.restype = C.c_int
    return o


def oracle_decode(codec_struct, codes):
    o = bind_oracle()
    n = codes.shape[0]
    out = np.zeros(n * UPSAMPLE * PATCH, np.float32)
    got = o.orc_codec_decode(C.byref(codec_struct), S.ip(np.ascontiguousarray(codes)), n, S.fp(out))
    return out[:got]


def bind_ref():
    r = S.ref()
    vp = C.c_void_p
    r.ref_codec_set_conv.argtypes = [vp, C.c_int, f32p, f32p] + [C.c_int] * 5
    r.ref_codec_set_layer.argtypes = [vp, C.c_int] + [f32p] * 13 + [C.c_int]
    r.ref_codec_set_tables.argtypes = [vp, f32p, f32p]
    r.ref_codec_decode.argtypes = [vp, i32p, C.c_int, f32p]
    r.ref_codec_decode.restype = C.c_int
    r.ref_codec_layer.argtypes = [vp, C.c_int, f32p, C.c_int]
    r.ref_codec_embed_codes.argtypes = [vp, i32p, C.c_int, f32p]
    r.ref_weight_norm.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int]
    r.tts_causal_conv1d.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5
    r.tts_causal_conv_transpose_1d.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 5 + [i32p]
    r.tts_alibi_attention.argtypes = [f32p, f32p, f32p, f32p] + [C.c_int] * 4 + [C.c_float, C.c_int, f32p]
    r.tts_linear_nobias.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    return r


def ref_bind_codec(ctx, hc):
    r = bind_ref()
    convs = [hc.input_conv] + hc.stage_convs + [hc.output_proj]
    for which, cv in zip((0, 1, 2, 3, 4), convs):
        r.ref_codec_set_conv(ctx, which, S.fp(cv.weight), _opt(cv.bias), cv.in_ch, cv.out_ch, cv.kernel,
                             cv.stride, int(cv.transpose))
    for i, l in enumerate(hc.layers):
        r.ref_codec_set_layer(ctx, i, S.fp(l.wq), S.fp(l.wk), S.fp(l.wv), S.fp(l.wo), _opt(l.q_norm),
                              _opt(l.k_norm), S.fp(l.attention_norm), S.fp(l.w1), S.fp(l.w2), S.fp(l.w3),
                              S.fp(l.ffn_norm), _opt(l.attn_scale), _opt(l.ffn_scale), l.window)
    r.ref_codec_set_tables(ctx, S.fp(hc.semantic_embedding), S.fp(hc.slopes))
    return r
