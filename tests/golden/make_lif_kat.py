"""Writes tests/golden/lif_kat.json: known-answer LIF traces computed with scalar numpy.float32 arithmetic.

The traces follow the update rule of pengjh0111/triton-snn-fusion runtime/snn_custom_ops.py:384-409 literally, one
scalar at a time (no tensors, no oracle code), so they pin the oracle, the C restatement and the HIP scan kernel
independently of each other:

    h = v + x                     if tau <= 1
    h = v + (x - v) / tau         otherwise          (all operations rounded to float32)
    s = 1 if h >= v_threshold else 0
    v = h - s * v_threshold       if v_reset < 0     (soft reset)
    v = v_reset if s else h       otherwise          (hard reset)

Run from the repository root:  python tests/golden/make_lif_kat.py
"""
import json
import os

import numpy as np

F = np.float32


def trace(xs, v0, v_th, v_reset, tau):
    v = F(v0)
    spikes, hs = [], []
    for x in xs:
        x = F(x)
        if tau <= 1.0:
            h = F(v + x)
        else:
            h = F(v + F(F(x - v) / F(tau)))
        s = 1 if h >= F(v_th) else 0
        if v_reset < 0:
            v = F(h - F(F(s) * F(v_th)))
        else:
            v = F(v_reset) if s else h
        spikes.append(s)
        hs.append(float(h))
    return spikes, hs, float(v)


def main():
    rng = np.random.RandomState(20260101)
    cases = []
    params = [(1.0, 0.0, 2.0), (1.0, -1.0, 2.0), (0.5, 0.0, 1.0), (1.0, 0.25, 4.0), (0.75, 0.0, 1.5), (1.0, -1.0, 3.0),
              (1.0, 0.0, 0.5)]
    for v_th, v_reset, tau in params:
        for T in (1, 2, 4, 8, 16):
            for _ in range(6):
                xs = (rng.randn(T) * 0.9 + 0.4).astype(np.float32)
                v0 = F(rng.randn() * 0.3) if rng.rand() < 0.5 else F(0.0)
                spikes, hs, v = trace(xs, v0, v_th, v_reset, tau)
                cases.append({"v_threshold": v_th, "v_reset": v_reset, "tau": tau, "v0": float(v0),
                              "x": [float(x) for x in xs], "spikes": spikes, "h": hs, "v": v})
    # Closed forms: constant sub-threshold drive b, tau 2, v0 0 -> h_t = b (1 - 2^-t); constant drive 1.5 -> spike every
    # second step.
    b = 0.9375
    spikes, hs, v = trace([b] * 10, 0.0, 1.0, 0.0, 2.0)
    assert spikes == [0] * 10 and all(abs(h - b * (1 - 2.0 ** -(t + 1))) < 1e-7 for t, h in enumerate(hs))
    cases.append({"v_threshold": 1.0, "v_reset": 0.0, "tau": 2.0, "v0": 0.0, "x": [b] * 10, "spikes": spikes, "h": hs, "v": v})
    spikes, hs, v = trace([1.5] * 8, 0.0, 1.0, 0.0, 2.0)
    assert spikes == [0, 1] * 4
    cases.append({"v_threshold": 1.0, "v_reset": 0.0, "tau": 2.0, "v0": 0.0, "x": [1.5] * 8, "spikes": spikes, "h": hs, "v": v})
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lif_kat.json")
    with open(out, "w") as fh:
        json.dump({"cases": cases}, fh)
    print(f"wrote {len(cases)} cases to {out}")


if __name__ == "__main__":
    main()
