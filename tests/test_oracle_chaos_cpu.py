"""Why decode parity is stated teacher-forced: the randomly initialised 26-layer backbone, with each
hidden state fed back through a random 3072 x 3072 projection (BASELINE.json configs[2]), is a
chaotic map.  Two runs of the SAME CPU oracle (tts_llm_forward, voxtral_tts_llm.c:171-271) whose
first inputs differ by one part in a million separate by about 3 x per step (measured here: 4.2e-5
of a hidden state's rms after the first step, 8.4e-4 after the fourth, 0.19 after the ninth, then
of the order of the signal).  A GPU run differs from the oracle by fp32 summation order (about 2e-4
of a hidden state's rms per step, each step adding its own), so its free-running chain has to leave
the oracle's chain at least that fast whatever its accuracy per step; the full-size GPU test reports
that drift (step 1: 8.5e-4, step 5: 0.3, from step 10 on of the order of the signal)."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import cases
import vtsupport as S

N_LAYERS = 26
STEPS = 12


@pytest.mark.timeout(600)
def test_two_oracle_chains_one_ppm_apart_separate_geometrically():
    with ThreadPoolExecutor(8) as ex:
        layers = list(ex.map(lambda i: S.Layer(1000 + i), range(N_LAYERS)))
    norm = S.norm_weight(S.DIM, 99)
    proj = S.bf16_normal((S.DIM, S.DIM), 31337)
    orc = cases.OracleBackend(threads=8)
    orc.llm_open(layers, norm, STEPS + 4, n_layers=N_LAYERS)

    def chain(e):
        orc.pos = 0                        # rows from `pos` on are never read: the cache needs no clearing
        out = []
        for _ in range(STEPS):
            h = orc.llm_forward(e)
            out.append(h)
            e = orc.linear(h.reshape(1, -1), proj, None, 1)[0]
        return out

    e0 = S.f32_normal(S.DIM, 4242)
    noise = S.f32_normal(S.DIM, 4243)
    a = chain(e0)
    b = chain((e0 * (np.float32(1.0) + np.float32(1e-6) * noise)).astype(np.float32))
    orc.llm_close()
    sep = np.array([S.rel_errors(x, y)[0] for x, y in zip(a, b)])      # max |d| / rms per step
    print("\nseparation of two oracle chains 1e-6 apart at the input, max|d|/rms per step: "
          + ", ".join(f"{s}: {v:.2e}" for s, v in enumerate(sep)))
    assert np.all(np.isfinite(sep))
    # small at first: the map is smooth, one step does not blow a 1e-6 perturbation up beyond 1e-3
    assert sep[0] < 1e-3, sep[0]
    # geometric growth while the chains are still close: 2.9 x per step on average at these seeds
    small = [s for s in range(1, STEPS) if sep[s] < 0.1]
    last = small[-1] if small else 0
    assert last >= 3, sep
    rate = (sep[last] / sep[0]) ** (1.0 / last)
    print(f"growth per step over steps 0..{last}: {rate:.2f} x")
    assert rate >= 2.5, (rate, sep)
    # and of the order of the signal from step 10 on: nothing of the first input is left
    assert sep[10:].min() > 0.5, sep
