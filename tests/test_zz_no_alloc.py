"""tts_hip_linear_bf16_noalloc, the entry point for callers that cannot allocate device memory:
the same kernels as tts_hip_linear_bf16 on a fixed work area.  Its output must equal that entry
point's bit for bit (same launches, same summation order), on two calls in a row of which the
second is smaller (the work area keeps the first call's contents), and against the oracle to the
product's own bound; a product beyond the fixed work area is refused with an error."""
import numpy as np
import pytest

import cases
import hipsupport as H
import vtsupport as S

pytestmark = pytest.mark.gpu


def test_noalloc_linear_equals_the_allocating_entry_point_twice_in_a_row():
    hip = H.Hip(kv_max=8)
    lib = hip.lib
    orc = cases.OracleBackend(threads=16)
    try:
        # (rows, out, in): a K cut with partial planes, then a smaller product, then a few rows
        # that take the row kernels (no work area), then the first again
        for m, n, k in ((130, 256, 4096), (24, 128, 192), (3, 56, 3072), (130, 256, 4096)):
            W = S.bf16_normal((n, k), 5000 + m + n)
            x = S.f32_normal((m, k), 5100 + k + m)
            dx, dW = H.DevBuf.from_numpy(lib, x), H.DevBuf.from_numpy(lib, W)
            dy0, dy1 = H.DevBuf(lib, m * n * 4), H.DevBuf(lib, m * n * 4)
            lib.tts_hip_memset(dy0.ptr, 0xff, m * n * 4)
            lib.tts_hip_memset(dy1.ptr, 0xff, m * n * 4)
            lib.tts_hip_linear_bf16(dy0.ptr, dx.ptr, None, m, k, n, dW.ptr)
            assert lib.tts_hip_linear_bf16_noalloc(dy1.ptr, dx.ptr, m, k, n, dW.ptr) == 0, lib.tts_hip_last_error()
            lib.tts_hip_sync()
            hip.check()
            want, got = dy0.to_numpy(np.float32, (m, n)), dy1.to_numpy(np.float32, (m, n))
            assert np.all(np.isfinite(got))
            assert np.array_equal(want, got), (m, n, k, float(np.max(np.abs(want - got))))
            ref = orc.linear(x, W, None, m)
            for r in range(m):
                mx, l2 = S.rel_errors(ref[r], got[r])
                assert mx < 1e-3 and l2 < 1e-3, (m, n, k, r, mx, l2)
            for b in (dx, dW, dy0, dy1):
                b.free()
        # beyond the fixed work area: an error, nothing launched
        m, n, k = 512, 4096, 3072
        dx, dW, dy = H.DevBuf(lib, m * k * 4), H.DevBuf(lib, n * k * 2), H.DevBuf(lib, m * n * 4)
        n0 = lib.tts_hip_error_count()
        assert lib.tts_hip_linear_bf16_noalloc(dy.ptr, dx.ptr, m, k, n, dW.ptr) == -1
        assert lib.tts_hip_error_count() == n0 + 1
        assert b"work area" in lib.tts_hip_last_error()
        assert lib.tts_hip_linear_bf16_noalloc(None, dx.ptr, m, k, n, dW.ptr) == -1
        for b in (dx, dW, dy):
            b.free()
    finally:
        hip.close()
