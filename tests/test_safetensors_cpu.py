"""Header reader of the checkpoint loader (host code, no GPU): files written by the
`safetensors` package itself are the known answers, so the reader is checked against the
format's own writer rather than against a writer of ours (reference reader:
voxtral_tts_safetensors.c:17-300)."""
import ctypes as C
import json
import struct

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import hipsupport as H
import vtsupport as S


def probe(lib, path, name):
    dtype = C.create_string_buffer(8)
    rank = C.c_int(-1)
    shape = (C.c_longlong * 4)()
    nbytes = C.c_longlong(-1)
    rc = lib.tts_hip_safetensors_probe(str(path).encode(), name.encode(), dtype, C.byref(rank),
                                       shape, C.byref(nbytes))
    return rc, dtype.value.decode(), rank.value, list(shape), nbytes.value


@pytest.fixture(scope="module")
def lib():
    return H.load_package().lib()


def test_probe_reads_what_the_format_writer_wrote(lib, tmp_path):
    tensors = {
        "layers.0.attention.wq.weight": torch.zeros(8, 6, dtype=torch.bfloat16),
        "norm.weight": torch.arange(5, dtype=torch.float32),
        "acoustic_transformer.layers.2.ffn_norm.weight": torch.ones(3, dtype=torch.float16),
        "a.scalar": torch.tensor(3.0),
        "cube": torch.zeros(2, 3, 4, 5, dtype=torch.bfloat16),
    }
    path = tmp_path / "m.safetensors"
    save_file(tensors, str(path), metadata={"format": "pt", "note": "braces } ] \" in a string"})
    want = {"layers.0.attention.wq.weight": ("BF16", [8, 6], 96),
            "norm.weight": ("F32", [5], 20),
            "acoustic_transformer.layers.2.ffn_norm.weight": ("F16", [3], 6),
            "a.scalar": ("F32", [], 4),
            "cube": ("BF16", [2, 3, 4, 5], 240)}
    for name, (dt, shp, nb) in want.items():
        rc, dtype, rank, shape, nbytes = probe(lib, path, name)
        assert rc == 0, name
        assert (dtype, rank, shape[:rank], nbytes) == (dt, len(shp), shp, nb), name
    assert probe(lib, path, "layers.0.attention.wq")[0] == 1         # prefix of a name: absent
    assert probe(lib, path, "__metadata__")[0] == 1                  # not a tensor


def test_many_tensors_grow_the_index(lib, tmp_path):
    tensors = {f"t.{i}": torch.full((i % 7 + 1,), float(i)) for i in range(1300)}
    path = tmp_path / "many.safetensors"
    save_file(tensors, str(path))
    for i in (0, 511, 512, 1299):
        rc, dtype, rank, shape, nbytes = probe(lib, path, f"t.{i}")
        assert (rc, dtype, rank, shape[0], nbytes) == (0, "F32", 1, i % 7 + 1, 4 * (i % 7 + 1))


def raw_file(path, header, data=b""):
    h = header if isinstance(header, bytes) else json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(h)) + h + data)


def test_malformed_files_are_errors(lib, tmp_path):
    n0 = lib.tts_hip_error_count()
    assert probe(lib, tmp_path / "absent.safetensors", "x")[0] == -1
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"\x01\x02")
    assert probe(lib, p, "x")[0] == -1
    # header length beyond the file
    p = tmp_path / "len.safetensors"
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    assert probe(lib, p, "x")[0] == -1
    # tensor bytes beyond the data section
    p = tmp_path / "range.safetensors"
    raw_file(p, {"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    assert probe(lib, p, "x")[0] == -1
    # cut-off JSON
    p = tmp_path / "cut.safetensors"
    raw_file(p, b'{"x":{"dtype":"F32","shape":[4],"data_offsets":[0,')
    assert probe(lib, p, "x")[0] == -1
    # an entry without offsets
    p = tmp_path / "nooff.safetensors"
    raw_file(p, {"x": {"dtype": "F32", "shape": [4]}}, b"\0" * 16)
    assert probe(lib, p, "x")[0] == -1
    assert lib.tts_hip_error_count() == n0 + 6
    # and a well-formed hand-written one, keys in another order, unknown keys skipped
    p = tmp_path / "ok.safetensors"
    raw_file(p, b' { "x" : { "data_offsets" : [ 0 , 16 ] , "extra" : {"a":[1,{"b":null}]} ,'
                b' "shape" : [ 2 , 2 ] , "dtype" : "F32" } } ', b"\0" * 16)
    assert probe(lib, p, "x")[:3] == (0, "F32", 2)
    p = tmp_path / "empty.safetensors"
    raw_file(p, b"{}")
    assert probe(lib, p, "x")[0] == 1


def test_hostile_headers_stay_inside_the_file(lib, tmp_path):
    """Numbers are read with every character checked against the end of the header (it is not
    NUL-terminated and may end where the file ends), nesting is bounded, and shapes whose
    product does not fit are not multiplied out."""
    n0 = lib.tts_hip_error_count()
    # the header, and with it the file, ends in the middle of a number
    p = tmp_path / "digits.safetensors"
    raw_file(p, b'{"x":{"dtype":"F32","shape":[4],"data_offsets":[0,1' + b"6" * 4000)
    assert probe(lib, p, "x")[0] == -1
    # a number that does not fit 63 bits
    p = tmp_path / "big.safetensors"
    raw_file(p, b'{"x":{"dtype":"F32","shape":[4],"data_offsets":[0,99999999999999999999999]}}', b"\0" * 16)
    assert probe(lib, p, "x")[0] == -1
    # metadata nested deeper than any writer produces
    p = tmp_path / "deep.safetensors"
    raw_file(p, b'{"__metadata__":' + b"[" * 100000 + b"]" * 100000 + b"}")
    assert probe(lib, p, "x")[0] == -1
    assert lib.tts_hip_error_count() == n0 + 3
    # negative offsets and extents: malformed / a tensor that matches no expected size
    p = tmp_path / "neg.safetensors"
    raw_file(p, {"x": {"dtype": "F32", "shape": [4], "data_offsets": [-16, 0]}}, b"\0" * 16)
    assert probe(lib, p, "x")[0] == -1
    p = tmp_path / "huge.safetensors"
    raw_file(p, {"x": {"dtype": "BF16", "shape": [1 << 40, 1 << 40, -3], "data_offsets": [0, 16]}}, b"\0" * 16)
    rc, dtype, rank, shape, nbytes = probe(lib, p, "x")
    assert (rc, dtype, rank, nbytes) == (0, "BF16", 3, 16)          # the header itself is well-formed


def test_load_needs_an_initialised_backend(lib, tmp_path):
    n0 = lib.tts_hip_error_count()
    p = tmp_path / "e.safetensors"
    raw_file(p, b"{}")
    if not H.load_package().ctx().initialized:
        assert lib.tts_hip_load_safetensors(str(p).encode()) == -1
        assert lib.tts_hip_error_count() == n0 + 1


def test_fallback_time_frequencies_follow_the_closed_form(lib):
    """The table the loader computes when a checkpoint lacks `time_embedding.inv_freq`
    (voxtral_tts_acoustic.c:48-60), checked against the mathematics, not against the oracle."""
    from test_oracle_math import _check_time_inv_freq
    f = np.zeros(S.DIM // 2, np.float32)
    lib.tts_hip_default_time_inv_freq(f.ctypes.data, S.DIM // 2)
    _check_time_inv_freq(f)
