"""CPU-side checks of the boundary: the C-ABI library loads, exports every
symbol include/voxtral_tts_hip.h declares, and fails loudly (0/-1 and an error
text, like the reference's init) when no GPU is present.  No compute calls."""
import ctypes as C
import os
import re

import pytest

import hipsupport as H
import vtsupport as S

pkg = H.load_package()
pytestmark = pytest.mark.skipif(not os.path.exists(pkg.LIB_PATH),
                                reason="library not built (run __graft_entry__.build())")


def declared_symbols(header="voxtral_tts_hip.h"):
    text = open(os.path.join(S.ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tts_hip_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_typed():
    lib = pkg.lib()
    names = declared_symbols()
    assert len(names) >= 37
    for n in names:
        assert hasattr(lib, n), n
        assert n in pkg.SIGNATURES, f"{n} has no ctypes signature"
    assert set(pkg.SIGNATURES) == set(names)
    assert pkg.ctx().initialized in (0, 1)


def test_bench_companion_exports_its_header_and_nothing_of_it_is_in_the_product():
    """Timing loops live in libvoxtral_tts_hip_bench.so (include/voxtral_tts_hip_bench.h); the product
    library's header declares none of them."""
    names = declared_symbols("voxtral_tts_hip_bench.h")
    assert set(names) == set(pkg.BENCH_SIGNATURES)
    bl = pkg.bench_lib()
    product = C.CDLL(pkg.LIB_PATH)
    for n in names:
        assert hasattr(bl, n), n
        assert n not in pkg.SIGNATURES
        assert not hasattr(product, n), f"{n} is still exported by the product library"
    assert not (set(declared_symbols()) & set(names))


def test_host_structs_match_the_reference_layout():
    """Field offsets of tts_decoder_t / tts_acoustic_t (voxtral_tts.h:101-125,
    146-165): pointers only, 9 per layer."""
    assert C.sizeof(pkg.HostLayer) == 9 * 8
    assert pkg.HostDecoder.layers.offset == 8
    assert pkg.HostDecoder.norm.offset == 8 + 26 * 72
    assert pkg.HostAcoustic.layers.offset == 8 * 8
    assert C.sizeof(pkg.HostAcoustic) == 8 * 8 + 3 * 72


@pytest.mark.skipif(H.gpu_present(), reason="only meaningful without a GPU")
def test_init_fails_loudly_without_a_gpu():
    lib = pkg.lib()
    n0 = lib.tts_hip_error_count()
    assert lib.tts_hip_init(64) == -1
    assert lib.tts_hip_available() == 0
    assert lib.tts_hip_error_count() == n0 + 1
    assert lib.tts_hip_last_error()
    # compute entry points are void and record an error instead of computing
    lib.tts_hip_llm_forward(None, None, 0)
    assert lib.tts_hip_error_count() == n0 + 2
    with pytest.raises(pkg.HipError):
        pkg.check_errors(n0)
