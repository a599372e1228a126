"""Checkpoint file -> device: a .safetensors file written by the `safetensors` package under
the reference's tensor names (voxtral_tts_llm.c:45-100, voxtral_tts_acoustic.c:40-130,
voxtral_tts_voice.c:251-290) must give the same device state as the struct upload of the
same arrays: every output below is compared bit for bit between the two sessions."""
import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu

AUDIO_ROWS = 8194 + 36 * 23


def as_bf16(a):
    return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)


def round_to_bf16(a):
    return S.bf16_to_f32(S.f32_to_bf16_trunc(a))


def layer_tensors(prefix, l, norm_dtype):
    t = {}
    for f, name in (("wq", "attention.wq"), ("wk", "attention.wk"), ("wv", "attention.wv"),
                    ("wo", "attention.wo"), ("w1", "feed_forward.w1"), ("w2", "feed_forward.w2"),
                    ("w3", "feed_forward.w3")):
        t[f"{prefix}{name}.weight"] = as_bf16(getattr(l, f))
    for f in ("attention_norm", "ffn_norm"):
        t[f"{prefix}{f}.weight"] = torch.from_numpy(getattr(l, f)).to(norm_dtype)
    return t


def offsets():
    offs = np.zeros(S.CODES, np.int32)
    offs[1] = 8194
    for i in range(2, S.CODES):
        offs[i] = offs[i - 1] + 23
    return offs


def run_session(hip, embeds, x0, codes):
    """A prefill, two decode steps, an acoustic frame and an embedding of codes."""
    out = {}
    out["prefill"] = hip.llm_prefill(embeds[:8], want_x=True)
    out["h0"] = hip.llm_forward(embeds[8])
    out["h1"] = hip.llm_forward(embeds[9])
    out["codes"], out["x"] = hip.acoustic_frame(out["h1"], x0)
    e = np.zeros(S.DIM, np.float32)
    hip.lib.tts_hip_audio_embed(e.ctypes.data, codes.ctypes.data)
    hip.check()
    out["embed"] = e
    return out


def test_file_load_equals_struct_upload(tmp_path):
    layers = [S.Layer(31), S.Layer(32)]
    final_norm = S.norm_weight(S.DIM, 33)
    ac = S.Acoustic(60)
    table = S.bf16_normal((AUDIO_ROWS, S.DIM), 61, 0.05)
    # the backbone's norm vectors go into the file as bf16 (as checkpoints hold them), the
    # acoustic ones as f16 and f32: the struct path gets the values those round to
    for l in layers:
        l.attention_norm = round_to_bf16(l.attention_norm)
        l.ffn_norm = round_to_bf16(l.ffn_norm)
    final_norm = round_to_bf16(final_norm)
    for l in ac.layers:
        l.attention_norm = l.attention_norm.astype(np.float16).astype(np.float32)

    t = {}
    for i, l in enumerate(layers):
        t.update(layer_tensors(f"layers.{i}.", l, torch.bfloat16))
    t["norm.weight"] = torch.from_numpy(final_norm).to(torch.bfloat16)
    for i, l in enumerate(ac.layers):
        lt = layer_tensors(f"acoustic_transformer.layers.{i}.", l, torch.float32)
        key = f"acoustic_transformer.layers.{i}.attention_norm.weight"
        lt[key] = lt[key].to(torch.float16)
        t.update(lt)
    t["acoustic_transformer.input_projection.weight"] = as_bf16(ac.input_proj)
    t["acoustic_transformer.time_projection.weight"] = as_bf16(ac.time_proj)
    t["acoustic_transformer.llm_projection.weight"] = as_bf16(ac.llm_proj)
    t["acoustic_transformer.semantic_codebook_output.weight"] = as_bf16(ac.semantic_out)
    t["acoustic_transformer.semantic_codebook_output.bias"] = torch.from_numpy(ac.semantic_out_bias)
    t["acoustic_transformer.acoustic_codebook_output.weight"] = as_bf16(ac.acoustic_out)
    t["acoustic_transformer.norm.weight"] = torch.from_numpy(ac.norm)
    # time_embedding.inv_freq is left out: the loader then computes the closed form
    t["mm_audio_embeddings.audio_codebook_embeddings.embeddings.weight"] = as_bf16(table)
    path = tmp_path / "consolidated.safetensors"
    save_file(t, str(path), metadata={"format": "pt"})
    del t

    embeds = S.f32_normal((10, S.DIM), 70, 1.0)
    x0 = S.f32_normal(S.ACOUSTIC_DIM, 71, 1.0)
    r = np.random.default_rng(72)
    codes = np.zeros(S.CODES, np.int32)
    codes[0] = r.integers(2, 8194)
    codes[1:] = r.integers(2, 23, S.CODES - 1)

    hip = H.Hip(kv_max=16)
    try:
        hip.upload_decoder(layers, final_norm, 2)
        hip.upload_acoustic(ac)
        assert hip.lib.tts_hip_upload_audio_embeddings(table.ctypes.data, AUDIO_ROWS,
                                                       offsets().ctypes.data) == 0
        want = run_session(hip, embeds, x0, codes)
    finally:
        hip.close()

    hip = H.Hip(kv_max=16)
    try:
        mask = hip.lib.tts_hip_load_safetensors(str(path).encode())
        assert mask == 7, hip.lib.tts_hip_last_error()
        assert hip.pkg.ctx().dec_layers_uploaded == 2
        assert hip.pkg.ctx().ac_layers_uploaded == 3
        hip.n_layers = 2
        got = run_session(hip, embeds, x0, codes)
    finally:
        hip.close()
    for k in want:
        assert np.array_equal(want[k], got[k]), k
    assert np.isfinite(got["h1"]).all() and np.abs(got["h1"]).max() > 0


def test_incomplete_layer_is_an_error(tmp_path):
    l = S.Layer(34)
    t = layer_tensors("layers.0.", l, torch.float32)
    del t["layers.0.feed_forward.w2.weight"]
    t["norm.weight"] = torch.ones(S.DIM)
    path = tmp_path / "broken.safetensors"
    save_file(t, str(path))
    hip = H.Hip(kv_max=8)
    try:
        n0 = hip.lib.tts_hip_error_count()
        assert hip.lib.tts_hip_load_safetensors(str(path).encode()) == -1
        assert hip.lib.tts_hip_error_count() > n0
        assert b"layer 0" in hip.lib.tts_hip_last_error()
        # a wrong shape under a right name
        t["layers.0.feed_forward.w2.weight"] = torch.zeros(S.DIM, 8, dtype=torch.bfloat16)
        save_file(t, str(path))
        assert hip.lib.tts_hip_load_safetensors(str(path).encode()) == -1
        assert hip.pkg.ctx().dec_layers_uploaded == 0
        # an optional tensor of the wrong size is an error too, not "absent"
        t = {"acoustic_transformer.input_projection.weight": torch.zeros(S.DIM, S.ACOUSTIC_DIM, dtype=torch.bfloat16),
             "acoustic_transformer.semantic_codebook_output.bias": torch.zeros(17)}
        save_file(t, str(path))
        assert hip.lib.tts_hip_load_safetensors(str(path).encode()) == -1
        assert b"bias" in hip.lib.tts_hip_last_error() or b"incomplete" in hip.lib.tts_hip_last_error()
    finally:
        hip.close()


def test_codec_file_load_equals_struct_upload(tmp_path):
    """The codec decoder from a file (weight norm folded by the loader, semantic table divided by the
    cluster usage with its floor: voxtral_tts_codec.c:38-57, 196-205) against the struct upload of
    arrays prepared by the oracle's restatement of the same steps: waveforms bit-equal."""
    import ctypes as C

    import codecsupport as K
    from test_gpu_codec import hip_decode

    o = K.bind_oracle()
    hc = K.HostCodec(12, distinct_layers=2)
    usage = (np.abs(S.f32_normal(K.SEM_SIZE, 500, 1.0)) + np.float32(1.0)).astype(np.float32)
    usage[3] = 0.0                               # floor of 1e-5 applies
    hc.emb_sum[3] *= np.float32(1e-5)
    o.orc_codec_semantic_embedding(S.fp(hc.semantic_embedding), S.fp(hc.emb_sum), S.fp(usage))

    t = {"audio_tokenizer.quantizer.semantic_codebook.embedding_sum": torch.from_numpy(hc.emb_sum),
         "audio_tokenizer.quantizer.semantic_codebook.cluster_usage": torch.from_numpy(usage)}

    def conv(prefix, cv, parametrised=True):
        if parametrised:
            shape = (cv.in_ch, cv.out_ch, cv.kernel) if cv.transpose else (cv.out_ch, cv.in_ch, cv.kernel)
            t[f"{prefix}.conv.parametrizations.weight.original0"] = torch.from_numpy(cv.g).reshape(-1, 1, 1)
            t[f"{prefix}.conv.parametrizations.weight.original1"] = torch.from_numpy(cv.v).reshape(shape)
        else:
            t[f"{prefix}.conv.weight"] = torch.from_numpy(cv.weight)
        if cv.bias is not None:
            t[f"{prefix}.conv.bias"] = torch.from_numpy(cv.bias)

    conv("audio_tokenizer.decoder_blocks.0", hc.input_conv)
    conv("audio_tokenizer.output_proj", hc.output_proj, parametrised=False)
    for st in range(3):
        conv(f"audio_tokenizer.decoder_blocks.{2 * st + 2}", hc.stage_convs[st])
    names = dict(wq="attention.wq.weight", wk="attention.wk.weight", wv="attention.wv.weight",
                 wo="attention.wo.weight", q_norm="attention.q_norm.weight", k_norm="attention.k_norm.weight",
                 attention_norm="attention_norm.weight", ffn_norm="ffn_norm.weight", w1="feed_forward.w1.weight",
                 w2="feed_forward.w2.weight", w3="feed_forward.w3.weight", attn_scale="attention_scale",
                 ffn_scale="ffn_scale")
    for i, l in enumerate(hc.layers):
        for field, suffix in names.items():
            t[f"audio_tokenizer.decoder_blocks.{2 * (i // 2) + 1}.layers.{i % 2}.{suffix}"] = \
                torch.from_numpy(getattr(l, field)).clone()     # cycled layers alias: the writer wants copies
    path = tmp_path / "codec.safetensors"
    save_file(t, str(path))
    del t

    codes = K.random_codes(6, 501)
    codes[4, 0] = 5                              # the row whose usage hit the floor
    hip = H.Hip(kv_max=8)
    try:
        cs = hc.struct()
        assert hip.lib.tts_hip_upload_codec_weights(C.addressof(cs)) == 0
        want = hip_decode(hip, codes)
    finally:
        hip.close()
    hip = H.Hip(kv_max=8)
    try:
        assert hip.lib.tts_hip_load_safetensors(str(path).encode()) == 8, hip.lib.tts_hip_last_error()
        got = hip_decode(hip, codes)
    finally:
        hip.close()
    assert np.array_equal(want, got)
    assert np.isfinite(got).all() and np.abs(got).max() > 0
