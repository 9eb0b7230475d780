"""Shared helpers of the parity tests: seeded operands rounded to the storage dtype, and the oracle comparison."""
from __future__ import annotations

import torch

from oracle import snn_oracle as O

LIF = (1.0, 0.0, 2.0)
DEV = "cuda:0"


def gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def spikes(shape, p, g):
    return (torch.rand(shape, generator=g) < p).to(torch.float32)


def q(t, dtype):
    """fp32 CPU tensor holding `t` after rounding to `dtype` (what the kernel receives)."""
    return O.round_like(t, dtype)


def dev(t, dtype):
    return None if t is None else t.to(DEV, dtype)


def zero_v(dtype=torch.float32):
    return torch.zeros((), device=DEV, dtype=dtype)


def check(got_spikes, got_v, ref, v_threshold=1.0, v_dtype=torch.float32, what="", max_rate=1e-4):
    """Gate: no spike mismatch away from threshold, mismatch rate <= 1e-4 counting only neurons within 1e-3 of the
    threshold, membrane within rtol 1e-3 / atol 1e-4 (widened to the storage rounding when the membrane is stored in a
    16-bit dtype)."""
    rtol, atol = (1e-3, 1e-4) if v_dtype == torch.float32 else ((8e-3, 1e-3) if v_dtype == torch.bfloat16 else (2e-3, 1e-3))
    report = O.parity_report(got_spikes, got_v, ref[0], ref[1], ref[2], v_threshold, rtol=rtol, atol=atol)
    O.assert_parity(report, max_rate=max_rate, what=what)
    return report
