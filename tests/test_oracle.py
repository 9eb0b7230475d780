"""Pins the CPU oracle (oracle/snn_oracle.py, oracle/snn_oracle.c) without the reference, which ships no vectors.

Each check is chosen so that a plausible mistake (dropped term, wrong sign, swapped stride/padding, wrong reset) fails
it: committed known-answer traces computed by scalar arithmetic, exact-sum convolutions computed by Python loops,
closed forms, and cross-checks between the torch restatement and the brute-force C restatement.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import snn_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with open(os.path.join(GOLDEN, name)) as fh:
        return json.load(fh)["cases"]


LIF_KAT = _load("lif_kat.json")
CONV_KAT = _load("conv_kat.json")


def test_lif_known_answer_traces_torch_oracle():
    for case in LIF_KAT:
        x = torch.tensor(case["x"], dtype=torch.float32).reshape(-1, 1)
        v0 = torch.tensor([case["v0"]], dtype=torch.float32)
        s, v, h = O.temporal_lif(x, v0, case["v_threshold"], case["v_reset"], case["tau"])
        assert s.flatten().tolist() == [float(k) for k in case["spikes"]], case
        assert h.flatten().tolist() == case["h"], case
        assert float(v) == case["v"], case


def test_lif_known_answer_traces_c_oracle():
    for case in LIF_KAT:
        x = np.asarray(case["x"], dtype=np.float32).reshape(-1, 1)
        s, v, h = c_oracle.lif_scan(x, np.asarray([case["v0"]], dtype=np.float32), case["v_threshold"], case["v_reset"], case["tau"])
        assert s.flatten().tolist() == [float(k) for k in case["spikes"]], case
        assert h.flatten().tolist() == case["h"], case
        assert float(v[0]) == case["v"], case


def test_lif_closed_forms():
    x = torch.tensor([0.3, 1.9, 2.0, 2.5, -1.0])
    s, v, h = O.lif_step(x, torch.tensor(0.0), 1.0, 0.0, 2.0)
    assert torch.equal(h, x / 2)                      # tau = 2, v = 0: h = x / 2 exactly
    assert s.tolist() == [0, 0, 1, 1, 0]              # fires iff x >= 2 * v_th
    assert torch.equal(v, torch.where(s.bool(), torch.zeros_like(h), h))   # hard reset
    s, v, h = O.lif_step(x, torch.tensor(0.0), 1.0, -1.0, 2.0)
    assert torch.equal(v, h - s * 1.0)                # soft reset
    s, v, h = O.lif_step(x, torch.full_like(x, 0.25), 1.0, 0.5, 1.0)
    assert torch.equal(h, x + 0.25)                   # tau <= 1: integrate-and-fire
    assert torch.equal(v[s.bool()], torch.full((int(s.sum()),), 0.5))
    # mismatched / 0-dim initial membrane means zeros
    assert torch.equal(O.lif_step(x, torch.zeros(3), 1.0, 0.0, 2.0)[2], x / 2)
    # geometric charging toward a constant drive b: h_t = b (1 - 2^-t)
    b = 0.9375
    _, _, h = O.temporal_lif(torch.full((10, 4), b), torch.tensor(0.0), 1.0, 0.0, 2.0)
    expected = torch.tensor([b * (1 - 2.0 ** -(t + 1)) for t in range(10)])
    assert torch.allclose(h[:, 0], expected, atol=1e-7, rtol=0)
    # constant supra-threshold drive 1.5: period-2 spike train
    s, _, _ = O.temporal_lif(torch.full((8, 2), 1.5), torch.tensor(0.0), 1.0, 0.0, 2.0)
    assert s[:, 0].tolist() == [0, 1] * 4


def test_lif_torch_oracle_matches_c_oracle_bit_exact():
    g = torch.Generator().manual_seed(11)
    for (v_th, v_reset, tau) in [(1.0, 0.0, 2.0), (0.7, -1.0, 3.0), (1.0, 0.3, 1.0), (1.2, 0.0, 1.7)]:
        x = torch.randn(6, 500, generator=g) * 0.9 + 0.3
        v0 = torch.randn(500, generator=g) * 0.4
        s, v, h = O.temporal_lif(x, v0, v_th, v_reset, tau)
        cs, cv, ch = c_oracle.lif_scan(x.numpy(), v0.numpy(), v_th, v_reset, tau)
        assert np.array_equal(s.numpy(), cs) and np.array_equal(v.numpy(), cv) and np.array_equal(h.numpy(), ch)


@pytest.mark.parametrize("case", [c for c in CONV_KAT if c["kind"] == "conv2d"], ids=lambda c: f"k{c['KH']}s{c['stride'][0]}g{c['groups']}")
def test_conv_known_answers_exact(case):
    x = torch.tensor(case["x"]).reshape(case["N"], case["Cin"], case["H"], case["W"])
    w = torch.tensor(case["w"]).reshape(case["Cout"], case["Cin"] // case["groups"], case["KH"], case["KW"])
    b = torch.tensor(case["b"])
    want = torch.tensor(case["out"]).reshape(case["N"], case["Cout"], case["Ho"], case["Wo"])
    # the oracle's conv stage: drive LIF with tau <= 1 and a huge threshold so that h == conv output
    _, _, h = O.temporal_conv_lif([x], w, b, torch.tensor(0.0), case["stride"], case["padding"], (1, 1), case["groups"], 1e30, 0.0, 1.0)
    assert torch.equal(h[0], want)
    got_c = c_oracle.conv2d(x.numpy(), w.numpy(), b.numpy(), case["stride"], case["padding"], case["groups"])
    assert np.array_equal(got_c, want.numpy())


@pytest.mark.parametrize("case", [c for c in CONV_KAT if c["kind"] == "linear"], ids=lambda c: f"{c['M']}x{c['Fin']}x{c['Fout']}")
def test_linear_known_answers_exact(case):
    x = torch.tensor(case["x"]).reshape(case["M"], case["Fin"])
    w = torch.tensor(case["w"]).reshape(case["Fout"], case["Fin"])
    b = torch.tensor(case["b"])
    want = torch.tensor(case["out"]).reshape(case["M"], case["Fout"])
    _, _, h = O.temporal_linear_lif([x], w, b, torch.tensor(0.0), 1e30, 0.0, 1.0)
    assert torch.equal(h[0], want)
    assert np.array_equal(c_oracle.linear(x.numpy(), w.numpy(), b.numpy()), want.numpy())


def test_conv_torch_vs_c_bruteforce_random():
    g = torch.Generator().manual_seed(5)
    for (N, Cin, H, W, Cout, k, s, p, groups) in [(2, 6, 9, 11, 8, 3, 1, 1, 1), (1, 8, 12, 12, 8, 3, 2, 1, 8), (2, 3, 17, 17, 4, 7, 2, 3, 1)]:
        x = torch.randn(N, Cin, H, W, generator=g)
        w = torch.randn(Cout, Cin // groups, k, k, generator=g) * 0.2
        b = torch.randn(Cout, generator=g)
        want = c_oracle.conv2d(x.numpy(), w.numpy(), b.numpy(), (s, s), (p, p), groups)
        got = F.conv2d(x, w, b, (s, s), (p, p), (1, 1), groups).numpy()
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_conv_one_hot_input_reads_back_the_weights():
    w = torch.randn(5, 3, 3, 3)
    x = torch.zeros(1, 3, 7, 7)
    x[0, 1, 3, 3] = 1.0
    _, _, h = O.temporal_conv_lif([x], w, None, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, 1e30, 0.0, 1.0)
    # output (oc, 3 + dy, 3 + dx) = w[oc, 1, 1 - dy, 1 - dx]
    assert torch.equal(h[0, 0, :, 2:5, 2:5], w[:, 1].flip(-1, -2))


def test_residual_is_a_plain_add_before_lif():
    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(2, 4, 6, 6, generator=g) for _ in range(3)]
    rs = [torch.randn(2, 5, 6, 6, generator=g) for _ in range(3)]
    w, b = torch.randn(5, 4, 3, 3, generator=g) * 0.3, torch.randn(5, generator=g)
    s, v, h = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, 1.0, 0.0, 2.0, residuals=rs)
    seq = torch.stack([F.conv2d(x, w, b, 1, 1) + r for x, r in zip(xs, rs)])
    s2, v2, h2 = O.temporal_lif(seq, torch.tensor(0.0), 1.0, 0.0, 2.0)
    assert torch.equal(s, s2) and torch.equal(v, v2) and torch.equal(h, h2)


def test_linear_with_binary_inputs_selects_weight_columns():
    g = torch.Generator().manual_seed(8)
    w = torch.randn(6, 40, generator=g)
    x = (torch.rand(4, 40, generator=g) < 0.2).float()
    _, _, h = O.temporal_linear_lif([x], w, None, torch.tensor(0.0), 1e30, 0.0, 1.0)
    want = torch.stack([w[:, x[m].bool()].double().sum(1) for m in range(4)]).float()
    assert torch.allclose(h[0], want, atol=1e-5)


def test_tail_identity_and_c_bruteforce():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(4, 3, 16, 5, 5, generator=g) * 0.75 + 0.15
    w, b = torch.randn(7, 16, generator=g) * 0.1, torch.randn(7, generator=g) * 0.1
    out, v, h, s = O.temporal_lif_avgpool_linear(x, torch.tensor(0.0), w, b, 1.0, 0.0, 2.0)
    s2, v2, _ = O.temporal_lif(x, torch.tensor(0.0), 1.0, 0.0, 2.0)
    assert torch.equal(s, s2) and torch.equal(v, v2)
    pooled_sum = s.mean(dim=(3, 4)).sum(0)               # sum_t mean_hw(s_t)
    assert torch.allclose(out, pooled_sum @ w.t() + 4 * b, atol=1e-5)
    per_step = sum(torch.from_numpy(c_oracle.avgpool_linear(s[t].numpy(), w.numpy(), b.numpy())) for t in range(4))
    assert torch.allclose(out, per_step, atol=1e-5)
    out_nb, *_ = O.temporal_lif_avgpool_linear(x, torch.tensor(0.0), w, torch.empty(0), 1.0, 0.0, 2.0)
    assert torch.allclose(out_nb, pooled_sum @ w.t(), atol=1e-5)   # empty bias means no bias


def test_bn_fold_matches_batch_norm_of_conv():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 5, 8, 8, generator=g)
    w, cb = torch.randn(6, 5, 3, 3, generator=g), torch.randn(6, generator=g)
    mean, var = torch.randn(6, generator=g) * 0.1, torch.rand(6, generator=g) + 0.5
    gamma, beta = torch.rand(6, generator=g) * 0.4 + 0.8, torch.randn(6, generator=g) * 0.1
    want = F.batch_norm(F.conv2d(x, w, cb, 1, 1), mean, var, gamma, beta, False, 0.0, 1e-5)
    fw, fb = O.fold_bn(w, cb, mean, var, gamma, beta, 1e-5)
    assert torch.allclose(F.conv2d(x, fw, fb, 1, 1), want, atol=2e-5, rtol=1e-5)
    fw0, fb0 = O.fold_bn(w, None, mean, var, None, None, 1e-5)
    want0 = F.batch_norm(F.conv2d(x, w, None, 1, 1), mean, var, None, None, False, 0.0, 1e-5)
    assert torch.allclose(F.conv2d(x, fw0, fb0, 1, 1), want0, atol=2e-5, rtol=1e-5)


def test_round_like_is_the_storage_round_trip():
    t = torch.tensor([1.0, 1.00390625, 0.1, -3.14159, 65504.0])
    assert torch.equal(O.round_like(t, torch.bfloat16), t.to(torch.bfloat16).float())
    assert torch.equal(O.round_like(t, torch.float16), t.to(torch.float16).float())
    assert torch.equal(O.round_like(t, torch.float32), t)


def test_parity_gate_accepts_near_threshold_flips_only():
    ref_s = torch.tensor([[0., 1., 0.], [1., 0., 0.]])
    ref_h = torch.tensor([[0.5, 1.0004, 0.2], [1.5, 0.3, 0.9996]])
    ref_v = torch.tensor([0.0, 0.3, 0.9996])
    ok = O.parity_report(ref_s.clone(), ref_v.clone(), ref_s, ref_v, ref_h, 1.0)
    assert ok["hard_mismatches"] == 0 and ok["near_threshold_flips"] == 0 and ok["membrane_out_of_tolerance"] == 0
    flipped = ref_s.clone()
    flipped[0, 1] = 0.0                                   # |h - v_th| = 4e-4: tolerated, neuron drops out of the v check
    rep = O.parity_report(flipped, torch.tensor([0.0, 9.9, 0.9996]), ref_s, ref_v, ref_h, 1.0)
    assert rep["hard_mismatches"] == 0 and rep["near_threshold_flips"] == 1 and rep["membrane_out_of_tolerance"] == 0
    far = ref_s.clone()
    far[0, 0] = 1.0                                       # h = 0.5: a real error
    assert O.parity_report(far, ref_v, ref_s, ref_v, ref_h, 1.0)["hard_mismatches"] == 1
    bad_v = O.parity_report(ref_s, torch.tensor([0.0, 0.31, 0.9996]), ref_s, ref_v, ref_h, 1.0)
    assert bad_v["membrane_out_of_tolerance"] == 1
    with pytest.raises(AssertionError):
        O.assert_parity(bad_v)
