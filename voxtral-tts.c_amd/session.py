"""A session over the library's global context for Python callers (benchmark, tests): device
buffers from tts_hip_alloc and the upload / step / frame calls with numpy arrays on the host side.
Everything here goes through the `extern "C"` entry points only."""
import ctypes as C

import numpy as np

from . import HostAcoustic, HostDecoder, HostLayer, check_errors, ctx, lib
from . import synth as S


class DevBuf:
    """A device allocation obtained from tts_hip_alloc."""

    def __init__(self, lib, nbytes):
        self.lib = lib
        self.nbytes = int(nbytes)
        self.ptr = lib.tts_hip_alloc(self.nbytes)
        assert self.ptr, "tts_hip_alloc failed"

    @classmethod
    def from_numpy(cls, lib, a):
        a = np.ascontiguousarray(a)
        b = cls(lib, a.nbytes)
        lib.tts_hip_to_device(b.ptr, a.ctypes.data, a.nbytes)
        return b

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        self.lib.tts_hip_to_host(out.ctypes.data, self.ptr, out.nbytes)
        return out

    def at(self, byte_offset):
        return self.ptr + int(byte_offset)

    def free(self):
        if self.ptr:
            self.lib.tts_hip_free_ptr(self.ptr)
            self.ptr = None


def host_layer(*args):
    """HostLayer struct over the numpy weights of a synth.Layer (the last argument)."""
    l = args[-1]
    return HostLayer(l.wq.ctypes.data, l.wk.ctypes.data, l.wv.ctypes.data, l.wo.ctypes.data,
                         l.attention_norm.ctypes.data, l.w1.ctypes.data, l.w2.ctypes.data,
                         l.w3.ctypes.data, l.ffn_norm.ctypes.data)


class Hip:
    """Session over the global backend context."""

    def __init__(self, kv_max=64):
        import sys
        self.pkg = sys.modules[__package__]
        self.lib = lib()
        self.lib.tts_hip_free()
        rc = self.lib.tts_hip_init(kv_max)
        assert rc == 0, self.lib.tts_hip_last_error()
        self.kv_max = kv_max
        self.err0 = self.lib.tts_hip_error_count()
        self.pos = 0

    def check(self):
        check_errors(self.err0)

    def close(self):
        self.lib.tts_hip_free()

    # -- backbone ------------------------------------------------------------
    def upload_decoder(self, layers, final_norm, n_layers):
        """n_layers device layers cycling over the given distinct host layers."""
        dec = HostDecoder()
        dec.tok_embeddings_bf16 = None
        for i in range(n_layers):
            dec.layers[i] = host_layer(layers[i % len(layers)])
        dec.norm = final_norm.ctypes.data
        self._keep = (layers, final_norm)
        rc = self.lib.tts_hip_upload_llm_weights_n(C.addressof(dec), n_layers)
        assert rc == 0, self.lib.tts_hip_last_error()
        self.n_layers = n_layers
        self.pos = 0

    def llm_forward(self, embed):
        out = np.zeros(S.DIM, np.float32)
        embed = np.ascontiguousarray(embed, np.float32)
        self.lib.tts_hip_llm_forward(out.ctypes.data, embed.ctypes.data, self.pos)
        self.check()
        self.pos += 1
        return out

    def llm_prefill(self, embeds, want_x=False):
        embeds = np.ascontiguousarray(embeds, np.float32)
        seq = embeds.shape[0]
        out_x = np.zeros((seq, S.DIM), np.float32) if want_x else None
        self.lib.tts_hip_llm_prefill_out(embeds.ctypes.data, seq, self.pos,
                                         out_x.ctypes.data if want_x else None)
        self.check()
        self.pos += seq
        return out_x

    def kv(self, n_layers=None):
        """Device KV caches as numpy [26, kv_max, 1024] (only uploaded layers are meaningful)."""
        g = ctx()
        shp = (26, self.kv_max, S.KV_DIM)
        k = np.empty(shp, np.float32)
        v = np.empty(shp, np.float32)
        self.lib.tts_hip_to_host(k.ctypes.data, g.kv_cache_k_gpu, k.nbytes)
        self.lib.tts_hip_to_host(v.ctypes.data, g.kv_cache_v_gpu, v.nbytes)
        return k, v

    def set_kv(self, k, v):
        g = ctx()
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        assert k.shape == (26, self.kv_max, S.KV_DIM)
        self.lib.tts_hip_to_device(g.kv_cache_k_gpu, k.ctypes.data, k.nbytes)
        self.lib.tts_hip_to_device(g.kv_cache_v_gpu, v.ctypes.data, v.nbytes)

    # -- acoustic --------------------------------------------------------------
    def upload_acoustic(self, ac):
        h = HostAcoustic()
        h.time_inv_freq = ac.time_inv_freq.ctypes.data
        h.input_proj_bf16 = ac.input_proj.ctypes.data
        h.time_proj_bf16 = ac.time_proj.ctypes.data
        h.llm_proj_bf16 = ac.llm_proj.ctypes.data
        h.semantic_out_bf16 = ac.semantic_out.ctypes.data
        h.semantic_out_bias = ac.semantic_out_bias.ctypes.data if ac.semantic_out_bias is not None else None
        h.acoustic_out_bf16 = ac.acoustic_out.ctypes.data
        h.norm = ac.norm.ctypes.data
        for i, l in enumerate(ac.layers):
            h.layers[i] = host_layer(l)
        self._keep_ac = ac
        rc = self.lib.tts_hip_upload_acoustic_weights(C.addressof(h))
        assert rc == 0, self.lib.tts_hip_last_error()

    def predict_velocity(self, x_t, h, t):
        v = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.tts_hip_predict_velocity(v.ctypes.data, x_t.ctypes.data, h.ctypes.data, float(t))
        self.check()
        return v

    def predict_velocity_cfg(self, x_t, h, t):
        vc = np.zeros(S.ACOUSTIC_DIM, np.float32)
        vu = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.tts_hip_predict_velocity_cfg(vc.ctypes.data, vu.ctypes.data, x_t.ctypes.data,
                                              h.ctypes.data, float(t))
        self.check()
        return vc, vu

    def acoustic_frame(self, h, x0):
        codes = np.zeros(S.CODES, np.int32)
        x = np.zeros(S.ACOUSTIC_DIM, np.float32)
        self.lib.tts_hip_acoustic_frame(codes.ctypes.data, h.ctypes.data, x0.ctypes.data, x.ctypes.data)
        self.check()
        return codes, x
