"""Where the time of a decode step goes, phase by phase, from the instrumented build of the library
(`make -C voxtral-tts.c_amd/csrc trace`, i.e. the same sources with -DVT_TRACE): workgroups 0 and
gridDim.x - 1 of the whole-step kernel stamp the 100 MHz wall clock four times per hand-over (phase
body done, hand-over stores acknowledged, next phase's rows requested, flags complete), and
tts_hip_trace_read copies the stamps out.

    VOXTRAL_TTS_HIP_LIB=$PWD/voxtral-tts.c_amd/csrc/trace/libvoxtral_tts_hip.so \\
        python3 voxtral-tts.c_amd/phase_trace.py [cache position, default 100]

Synthetic weights (three distinct layers in rotation over 26), as in tests/."""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
import hipsupport as H      # noqa: E402
import vtsupport as S       # noqa: E402

N_LAYERS, PHASES = 26, ("q|k|v", "attention", "output", "gate|up", "down")


def main():
    pos = int(sys.argv[1]) if len(sys.argv) > 1 else 100
    hip = H.Hip(kv_max=pos + 64)
    lib = hip.lib
    if not hasattr(lib, "tts_hip_trace_read"):
        raise SystemExit("this library was built without -DVT_TRACE (see the docstring)")
    hip.upload_decoder([S.Layer(1), S.Layer(2), S.Layer(3)], S.norm_weight(S.DIM, 99), N_LAYERS)
    e = H.DevBuf.from_numpy(lib, S.f32_normal(S.DIM, 6))
    h = H.DevBuf(lib, S.DIM * 4)
    for i in range(6):                                   # the stamps of the last launch stay in the buffer
        lib.tts_hip_llm_forward_device(h.ptr, e.ptr, pos + i)
    lib.tts_hip_sync()
    hip.check()
    buf = np.zeros(2 * 4096, np.uint64)
    lib.tts_hip_trace_read.argtypes = [C.c_void_p]
    lib.tts_hip_trace_read(buf.ctypes.data)
    for w, who in enumerate(("workgroup 0", "last workgroup")):
        t = buf[w * 4096:(w + 1) * 4096].astype(np.int64)[:N_LAYERS * 5 * 4].reshape(N_LAYERS, 5, 4)
        released = np.concatenate([[t[0, 0, 0]], t.reshape(-1, 4)[:-1, 3]]).reshape(N_LAYERS, 5)
        parts = {"body": t[:, :, 0] - released, "stores acknowledged": t[:, :, 1] - t[:, :, 0],
                 "rows requested": t[:, :, 2] - t[:, :, 1], "flags complete": t[:, :, 3] - t[:, :, 2]}
        print(f"{who}: {(t[-1, -1, -1] - t[0, 0, 0]) / 100.0:.1f} us per step; mean over layers 1..{N_LAYERS - 1}, us")
        for p, name in enumerate(PHASES):
            print(f"  {name:10s} " + "  ".join(f"{k} {v[1:, p].mean() / 100.0:5.2f}" for k, v in parts.items()))
        print(f"  per layer {sum(v[1:].sum(axis=1).mean() for v in parts.values()) / 100.0:.2f}")
    hip.close()


if __name__ == "__main__":
    main()
