#!/usr/bin/env python3
"""Writes the golden fixtures in this directory by running the seeded cases of
cases.py on the COMPILED REFERENCE (oracle/_ref/libvoxtral_ref.so, built from
the reference's own sources by `make -C oracle ref`).  The reference tree
cannot travel, so only the outputs are committed, as .npz data.

    python tests/golden/make_golden.py            # writes kernels/llm/acoustic/codec .npz

Run it only where the reference tree is mounted.  It also cross-checks the
oracle bit-for-bit against what it writes and fails loudly on a mismatch.
"""
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import cases  # noqa: E402
import codec_cases  # noqa: E402
import vtsupport as S  # noqa: E402


def bit_equal(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


def main():
    if not S.have_ref():
        sys.exit("oracle/_ref/libvoxtral_ref.so missing: run `make -C oracle ref` "
                 "where the reference tree is mounted")
    rb, ob = cases.RefBackend(), cases.OracleBackend(threads=8)
    bad = 0
    crb, cob = codec_cases.RefCodecBackend(), codec_cases.OracleCodecBackend(threads=8)
    for name, fn, r, o in (("kernels", cases.kernel_cases, rb, ob), ("llm", cases.llm_cases, rb, ob),
                           ("acoustic", cases.acoustic_cases, rb, ob),
                           ("codec", codec_cases.codec_cases, crb, cob)):
        t0 = time.time()
        got = fn(r)
        t1 = time.time()
        mine = fn(o)
        t2 = time.time()
        for k in got:
            if not bit_equal(got[k], mine[k]):
                bad += 1
                print(f"MISMATCH {name}/{k}: max|d|={np.max(np.abs(got[k].astype(np.float64) - mine[k]))}")
        np.savez_compressed(os.path.join(HERE, f"{name}.npz"), **got)
        print(f"{name}: {len(got)} arrays, reference {t1 - t0:.1f}s, oracle {t2 - t1:.1f}s")
    if bad:
        sys.exit(f"{bad} arrays differ between the oracle and the compiled reference")
    print("oracle == compiled reference, bit for bit, on every case")


if __name__ == "__main__":
    main()
