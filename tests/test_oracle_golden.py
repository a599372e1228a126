"""The oracle against the committed golden fixtures (tests/golden/*.npz), which
were written by the compiled reference (tests/golden/make_golden.py).
Bit-exact: the reference CPU path is sequential fp32 without contraction."""
import os

import numpy as np
import pytest

import cases
import vtsupport as S


def _load(name):
    return np.load(os.path.join(S.GOLDEN_DIR, name + ".npz"))


def _check(got, gold):
    assert set(got.keys()) == set(gold.files)
    for k in gold.files:
        a, b = np.ascontiguousarray(got[k]), gold[k]
        assert a.shape == b.shape and a.dtype == b.dtype, k
        assert a.tobytes() == b.tobytes(), f"{k}: max|d|={np.max(np.abs(a.astype(np.float64) - b))}"


def test_kernels_match_reference_fixtures():
    _check(cases.kernel_cases(cases.OracleBackend(threads=1)), _load("kernels"))


def test_threads_do_not_change_bits():
    a = cases.kernel_cases(cases.OracleBackend(threads=1))
    b = cases.kernel_cases(cases.OracleBackend(threads=4))
    for k in a:
        assert a[k].tobytes() == b[k].tobytes(), k


def test_llm_decode_and_prefill_match_reference_fixtures():
    _check(cases.llm_cases(cases.OracleBackend(threads=8)), _load("llm"))


def test_acoustic_matches_reference_fixtures():
    _check(cases.acoustic_cases(cases.OracleBackend(threads=8)), _load("acoustic"))


@pytest.mark.skipif(not S.have_ref(), reason="oracle/_ref not built (reference tree absent)")
def test_oracle_equals_compiled_reference_directly():
    """Where the compiled reference is present, rerun the kernel cases on it
    and compare bit-for-bit (the model-level cases are covered by the fixtures,
    which the same library wrote)."""
    a = cases.kernel_cases(cases.RefBackend())
    b = cases.kernel_cases(cases.OracleBackend(threads=1))
    for k in a:
        assert a[k].tobytes() == b[k].tobytes(), k
