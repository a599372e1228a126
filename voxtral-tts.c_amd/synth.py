"""Seeded synthetic weights and inputs of the shapes the backend consumes, and the comparison metrics
of its parity statements.  Used by the benchmark and, through tests/vtsupport.py, by the tests, so
that both sides of every comparison are fed identical bytes.  Pure numpy; no GPU, no checker library.
"""
import ctypes as C

import numpy as np

DIM, HEADS, KV_HEADS, HEAD_DIM = 3072, 32, 8, 128
Q_DIM, KV_DIM, FFN = 4096, 1024, 9216
EPS, THETA = 1e-5, 1000000.0
ACOUSTIC_DIM, SEM_PADDED, CODES = 36, 8320, 37


# --------------------------------------------------------------------------
# synthetic data
# --------------------------------------------------------------------------

def f32_to_bf16_trunc(a):
    """bf16 by truncation (bits >> 16), as the reference test does
    (test_kernels.c:68-76)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    return (a.view(np.uint32) >> 16).astype(np.uint16)


def bf16_to_f32(h):
    return (h.astype(np.uint32) << 16).view(np.float32)


def bf16_normal(shape, seed, std=0.02):
    g = np.random.default_rng(seed)
    return f32_to_bf16_trunc(g.standard_normal(shape, dtype=np.float32) * np.float32(std))


def f32_normal(shape, seed, std=1.0):
    g = np.random.default_rng(seed)
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def norm_weight(n, seed):
    """Positive RMSNorm gains |N(0,1)|*0.1+0.01 in the style of the reference
    test's fill_random_positive (test_kernels.c:62-66); O(1) after scaling so
    that hidden states stay O(1) through many layers."""
    g = np.random.default_rng(seed)
    return (np.abs(g.standard_normal(n, dtype=np.float32)) * np.float32(0.5)
            + np.float32(0.75)).astype(np.float32)


class Layer:
    """One transformer layer of synthetic weights (numpy, host)."""
    FIELDS = ("wq", "wk", "wv", "wo", "w1", "w2", "w3")
    SHAPES = dict(wq=(Q_DIM, DIM), wk=(KV_DIM, DIM), wv=(KV_DIM, DIM), wo=(DIM, Q_DIM),
                  w1=(FFN, DIM), w2=(DIM, FFN), w3=(FFN, DIM))

    def __init__(self, seed, std=0.02):
        for i, f in enumerate(self.FIELDS):
            setattr(self, f, bf16_normal(self.SHAPES[f], seed * 16 + i, std))
        self.attention_norm = norm_weight(DIM, seed * 16 + 8)
        self.ffn_norm = norm_weight(DIM, seed * 16 + 9)


class Acoustic:
    """Synthetic acoustic-transformer weights (numpy, host)."""

    def __init__(self, seed, n_layers=3, bias=True, std=0.02, time_inv_freq=None):
        self.n_layers = n_layers
        self.layers = [Layer(seed + 1 + i, std) for i in range(n_layers)]
        if time_inv_freq is None:
            # the table a checkpoint without `time_embedding.inv_freq` gets (voxtral_tts_acoustic.c:48-60),
            # from the library's own host routine
            from . import lib
            time_inv_freq = np.zeros(DIM // 2, np.float32)
            lib().tts_hip_default_time_inv_freq(time_inv_freq.ctypes.data, DIM // 2)
        self.time_inv_freq = np.ascontiguousarray(time_inv_freq, np.float32)
        self.input_proj = bf16_normal((DIM, ACOUSTIC_DIM), seed * 16 + 1, 0.2)
        self.time_proj = bf16_normal((DIM, DIM), seed * 16 + 2, std)
        self.llm_proj = bf16_normal((DIM, DIM), seed * 16 + 3, std)
        self.semantic_out = bf16_normal((SEM_PADDED, DIM), seed * 16 + 4, std)
        self.semantic_out_bias = f32_normal(SEM_PADDED, seed * 16 + 5, 0.1) if bias else None
        self.acoustic_out = bf16_normal((ACOUSTIC_DIM, DIM), seed * 16 + 6, std)
        self.norm = norm_weight(DIM, seed * 16 + 7)


class CodecWeights:
    """Synthetic effective weights of the audio codec decoder (weight norm already folded, as the upload
    entry point takes them; voxtral_tts.h:172-225): convolution rows of norm about `gain`, transformer
    matrices ~N(0, 0.03), positive norm gains and layer scales.  struct() is a HostCodec for
    tts_hip_upload_codec_weights.  `distinct_layers` < 8 cycles the layer weights (pointers alias)."""
    DIM, HID, HEADS = 1024, 4096, 8
    EMBED, SEM_DIM, SEM_SIZE, PATCH, LEVELS = 292, 256, 8192, 240, 21
    WINDOWS = (2, 4, 8, 16)

    def __init__(self, seed, distinct_layers=2):
        D, Hd = self.DIM, self.HID

        def conv(sd, in_ch, out_ch, kernel, stride, transpose, gain):
            rows, fan_in = (in_ch, out_ch * kernel) if transpose else (out_ch, in_ch * kernel)
            w = f32_normal((rows, fan_in), sd, gain * 0.9 / np.sqrt(fan_in))
            return dict(weight=w, bias=f32_normal(out_ch, sd + 2, 0.1), in_ch=in_ch, out_ch=out_ch,
                        kernel=kernel, stride=stride, transpose=int(transpose))

        self.semantic_embedding = np.clip(f32_normal((self.SEM_SIZE, self.SEM_DIM), seed * 64 + 1, 1.0), -4.0, 4.0).astype(np.float32)
        self.input_conv = conv(seed * 64 + 3, self.EMBED, D, 3, 1, False, 0.05)
        self.stage_convs = [conv(seed * 64 + 20 + 3 * i, D, D, 4, 2, True, 1.0) for i in range(3)]
        self.output_proj = conv(seed * 64 + 40, D, self.PATCH, 7, 1, False, 0.05)
        self.layers = []
        for i in range(distinct_layers):
            sd = (seed * 64 + 8 + i) * 32
            n = lambda shape, k, std: f32_normal(shape, sd + k, std)
            self.layers.append(dict(
                wq=n((D, D), 0, 0.03), wk=n((D, D), 1, 0.03), wv=n((D, D), 2, 0.03), wo=n((D, D), 3, 0.03),
                w1=n((Hd, D), 4, 0.03), w3=n((Hd, D), 5, 0.03), w2=n((D, Hd), 6, 0.02),
                attention_norm=norm_weight(D, sd + 7), ffn_norm=norm_weight(D, sd + 8),
                q_norm=norm_weight(D, sd + 9), k_norm=norm_weight(D, sd + 10),
                attn_scale=(norm_weight(D, sd + 11) * np.float32(0.5)).astype(np.float32),
                ffn_scale=(norm_weight(D, sd + 12) * np.float32(0.5)).astype(np.float32)))
        self.slopes = np.array([2.0 ** -(h + 1) for h in range(self.HEADS)], np.float32)

    def struct(self):
        from . import HostCodec, HostCodecLayer, HostConv
        p = lambda a: a.ctypes.data
        c = HostCodec()
        c.semantic_embedding = p(self.semantic_embedding)

        def cv(d):
            return HostConv(p(d["weight"]), p(d["bias"]), d["in_ch"], d["out_ch"], d["kernel"], d["stride"], d["transpose"])

        c.input_conv = cv(self.input_conv)
        for i, d in enumerate(self.stage_convs):
            c.stage_convs[i] = cv(d)
        c.output_proj = cv(self.output_proj)
        for i in range(8):
            l = self.layers[i % len(self.layers)]
            c.transformers[i] = HostCodecLayer(p(l["wq"]), p(l["wk"]), p(l["wv"]), p(l["wo"]), p(l["q_norm"]), p(l["k_norm"]),
                                               p(l["attention_norm"]), p(l["w1"]), p(l["w2"]), p(l["w3"]), p(l["ffn_norm"]),
                                               p(l["attn_scale"]), p(l["ffn_scale"]), self.WINDOWS[i // 2])
        for h in range(self.HEADS):
            c.alibi_slopes[h] = float(self.slopes[h])
        c._keep = self
        return c

    def random_codes(self, n_frames, seed):
        r = np.random.default_rng(seed)
        codes = np.zeros((n_frames, CODES), np.int32)
        codes[:, 0] = r.integers(2, 2 + self.SEM_SIZE, n_frames)
        codes[:, 1:] = r.integers(2, 2 + self.LEVELS, (n_frames, CODES - 1))
        return codes


# --------------------------------------------------------------------------
# comparison metrics
# --------------------------------------------------------------------------

def rel_errors(ref_v, test_v):
    """(max|d|/rms(ref), ||d||2/||ref||2) for one hidden-state vector."""
    ref_v = np.asarray(ref_v, np.float64).ravel()
    test_v = np.asarray(test_v, np.float64).ravel()
    d = test_v - ref_v
    rms = np.sqrt(np.mean(ref_v ** 2)) + 1e-30
    return float(np.max(np.abs(d)) / rms), float(np.linalg.norm(d) / (np.linalg.norm(ref_v) + 1e-30))


def compare_tensors(ref_v, test_v, rtol, atol):
    """The reference's rtol-OR-atol rule (test_kernels.c:79-116): an element
    is bad iff rel > rtol and |d| > atol; pass iff no bad element and
    (max_rel <= rtol or max_abs <= atol)."""
    ref_v = np.asarray(ref_v, np.float32).ravel()
    test_v = np.asarray(test_v, np.float32).ravel()
    diff = np.abs(ref_v - test_v)
    denom = np.maximum(np.abs(ref_v), np.float32(1e-8))
    rel = diff / denom
    n_bad = int(np.sum((rel > rtol) & (diff > atol)))
    ok = (rel.max() <= rtol or diff.max() <= atol) and n_bad == 0
    return bool(ok), float(rel.max()), float(diff.max()), n_bad
