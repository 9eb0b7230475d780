"""CPU oracle for the fused temporal SNN operators. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module, and only as the checker
(or as the timed CPU baseline); the product package never does.

It restates, in plain fp32 PyTorch-CPU ops, the eager path of pengjh0111/triton-snn-fusion
(runtime/snn_custom_ops.py:378-642) and additionally returns the pre-reset membrane h[t] of every step, which the
reference never materialises but which the parity gate needs (spike mismatches only count for |h - v_th| <= 1e-3).

How each function is pinned (the reference ships no golden vectors or tests for this path, see tests/test_oracle.py):
  lif_step               closed forms: tau=2, v=0 gives h = x/2 exactly; hard reset gives v' == v_reset where s == 1
                         and v' == h elsewhere; soft reset gives v' = h - v_th*s; tau <= 1 is the IF neuron; constant
                         drive b with no spike gives h_t = b*(1 - 2^-t); hand-computed 3-step traces.
  temporal_conv_lif      F.conv2d (the routine the reference itself calls) cross-checked against the brute-force
                         direct convolution of oracle/snn_oracle.c in float64, one-hot linearity, residual = plain add.
  temporal_linear_lif    F.linear cross-checked against the C brute force; binary inputs select weight columns.
  temporal_lif_avgpool_linear   identity out_sum == W . sum_t mean_hw(s_t) + T*b, and the C brute force.
  fold_bn                conv(x, W', b') == batch_norm(conv(x, W, b)) in eval mode.
bf16 / fp16 operation of the HIP kernels is checked against this oracle evaluated in fp32 on inputs that were first
rounded to that dtype (round_like), because the kernels keep the membrane and every accumulation in fp32.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


def round_like(t: Optional[torch.Tensor], dtype: torch.dtype) -> Optional[torch.Tensor]:
    """fp32 tensor holding the values `t` takes after a round trip through `dtype`."""
    if t is None:
        return None
    return t.detach().to("cpu").to(dtype).to(torch.float32)


def _initial_membrane(x: torch.Tensor, v_prev: Optional[torch.Tensor]) -> torch.Tensor:
    # runtime/snn_custom_ops.py:378-381: a 0-dim or mismatched v_prev means a zero membrane.
    if v_prev is None or v_prev.dim() == 0 or tuple(v_prev.shape) != tuple(x.shape):
        return torch.zeros_like(x)
    return v_prev.to(x.dtype)


def lif_step(x: torch.Tensor, v_prev: Optional[torch.Tensor], v_threshold: float, v_reset: float, tau: float):
    """One LIF update (runtime/snn_custom_ops.py:384-409). Returns (spike, v_next, h)."""
    v = _initial_membrane(x, v_prev)
    if float(tau) <= 1.0:
        h = v + x
    else:
        h = v + (x - v) / float(tau)
    fired = h >= float(v_threshold)
    spike = fired.to(x.dtype)
    if float(v_reset) < 0:
        v_next = h - spike * float(v_threshold)
    else:
        v_next = torch.where(fired, torch.full_like(h, float(v_reset)), h)
    return spike, v_next, h


def temporal_lif(x_seq: torch.Tensor, v_init, v_threshold, v_reset, tau):
    """runtime/snn_custom_ops.py:521-536. x_seq [T, ...] -> (spikes [T, ...], v_final, h [T, ...])."""
    v = v_init
    spikes, hs = [], []
    for t in range(int(x_seq.shape[0])):
        s, v, h = lif_step(x_seq[t], v, v_threshold, v_reset, tau)
        spikes.append(s)
        hs.append(h)
    return torch.stack(spikes, 0), v, torch.stack(hs, 0)


def temporal_conv_lif(
    xs: Sequence[torch.Tensor],
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    v_init,
    stride,
    padding,
    dilation,
    groups: int,
    v_threshold: float,
    v_reset: float,
    tau: float,
    residuals: Optional[Sequence[torch.Tensor]] = None,
):
    """runtime/snn_custom_ops.py:430-453 (and :491-518 with residuals): conv2d (+ residual) + LIF per step."""
    if len(xs) == 0:
        raise RuntimeError("temporal_conv_lif requires at least one input tensor")
    if residuals is not None and len(residuals) != len(xs):
        raise RuntimeError("xs and residuals must have the same temporal length")
    v = v_init
    spikes, hs = [], []
    for t, x in enumerate(xs):
        cur = F.conv2d(x, weight, bias, stride, padding, dilation, groups)
        if residuals is not None:
            cur = cur + residuals[t]
        s, v, h = lif_step(cur, v, v_threshold, v_reset, tau)
        spikes.append(s)
        hs.append(h)
    return torch.stack(spikes, 0), v, torch.stack(hs, 0)


def temporal_linear_lif(xs, weight, bias, v_init, v_threshold, v_reset, tau):
    """runtime/snn_custom_ops.py:561-611. xs: list of [M, Fin] or a packed [T, ..., Fin] tensor."""
    steps: List[torch.Tensor] = [xs[t] for t in range(int(xs.shape[0]))] if isinstance(xs, torch.Tensor) else list(xs)
    if len(steps) == 0:
        raise RuntimeError("temporal_linear_lif requires at least one input tensor")
    b = bias if isinstance(bias, torch.Tensor) and bias.numel() > 0 else None
    v = v_init
    spikes, hs = [], []
    for x in steps:
        s, v, h = lif_step(F.linear(x, weight, b), v, v_threshold, v_reset, tau)
        spikes.append(s)
        hs.append(h)
    return torch.stack(spikes, 0), v, torch.stack(hs, 0)


def temporal_lif_avgpool_linear(x_seq, v_init, fc_weight, fc_bias, v_threshold, v_reset, tau):
    """runtime/snn_custom_ops.py:539-558. Returns (out_sum [N, K], v_final, h [T, N, C, H, W], spikes)."""
    b = fc_bias if isinstance(fc_bias, torch.Tensor) and fc_bias.numel() > 0 else None
    v = v_init
    out_sum = None
    spikes, hs = [], []
    for t in range(int(x_seq.shape[0])):
        s, v, h = lif_step(x_seq[t], v, v_threshold, v_reset, tau)
        pooled = F.adaptive_avg_pool2d(s, (1, 1)).flatten(1)
        logits = F.linear(pooled, fc_weight, b)
        out_sum = logits if out_sum is None else out_sum + logits
        spikes.append(s)
        hs.append(h)
    return out_sum, v, torch.stack(hs, 0), torch.stack(spikes, 0)


def fold_bn(conv_weight, conv_bias, running_mean, running_var, bn_weight, bn_bias, eps: float):
    """Eval-mode BatchNorm folded into the preceding conv (compiler/fx_lif_rewrite.py:340-353)."""
    if conv_bias is None:
        conv_bias = torch.zeros_like(running_mean)
    if bn_weight is None:
        bn_weight = torch.ones_like(running_mean)
    if bn_bias is None:
        bn_bias = torch.zeros_like(running_mean)
    scale = bn_weight / torch.sqrt(running_var + float(eps))
    w = conv_weight.to(running_mean.dtype) * scale.reshape(-1, 1, 1, 1)
    b = (conv_bias.to(running_mean.dtype) - running_mean) * scale + bn_bias
    return w, b


# -----------------------------------------------------------------------------------------------------------------
# Parity gate
# -----------------------------------------------------------------------------------------------------------------
def parity_report(
    spikes: torch.Tensor,
    v_final: torch.Tensor,
    ref_spikes: torch.Tensor,
    ref_v: torch.Tensor,
    ref_h: torch.Tensor,
    v_threshold: float,
    band: float = 1e-3,
    rtol: float = 1e-3,
    atol: float = 1e-4,
) -> dict:
    """Compares a kernel result with the oracle under the gate:

    * a spike mismatch is tolerated only at its FIRST occurrence for a neuron and only if the oracle's pre-reset
      membrane there is within `band` of the threshold (a rounding-order flip); anything else is a hard mismatch;
    * the mismatch rate counts neuron-steps up to and including each neuron's first flip over all neuron-steps;
    * the final membrane is compared (rtol/atol) only on neurons whose whole spike history agrees, because a flip
      legitimately changes everything downstream of it.
    """
    got = spikes.detach().to("cpu", torch.float32)
    ref = ref_spikes.detach().to("cpu", torch.float32)
    h = ref_h.detach().to("cpu", torch.float32)
    assert got.shape == ref.shape == h.shape, (got.shape, ref.shape, h.shape)
    values_ok = bool(((got == 0) | (got == 1)).all())
    diff = got != ref
    seen_before = (torch.cumsum(diff.to(torch.int32), 0) - diff.to(torch.int32)) > 0
    first = diff & ~seen_before
    near = (h - float(v_threshold)).abs() <= band
    hard = int((first & ~near).sum())
    soft = int((first & near).sum())
    counted = int((~seen_before).sum())
    history_ok = ~diff.any(0)
    gv = v_final.detach().to("cpu", torch.float32)
    rv = ref_v.detach().to("cpu", torch.float32)
    err = (gv - rv).abs()
    tol = atol + rtol * rv.abs()
    bad_v = int(((err > tol) & history_ok).sum())
    max_v_err = float(err[history_ok].max()) if bool(history_ok.any()) else 0.0
    return {
        "spike_values_binary": values_ok,
        "hard_mismatches": hard,
        "near_threshold_flips": soft,
        "mismatch_rate": soft / max(counted, 1),
        "neuron_steps": counted,
        "membrane_out_of_tolerance": bad_v,
        "membrane_max_abs_err": max_v_err,
        "neurons_with_matching_history": int(history_ok.sum()),
        "neurons": int(history_ok.numel()),
    }


def assert_parity(report: dict, max_rate: float = 1e-4, what: str = "") -> None:
    assert report["spike_values_binary"], f"{what}: spikes are not 0/1: {report}"
    assert report["hard_mismatches"] == 0, f"{what}: spike mismatch away from threshold: {report}"
    assert report["mismatch_rate"] <= max_rate, f"{what}: spike mismatch rate too high: {report}"
    assert report["membrane_out_of_tolerance"] == 0, f"{what}: membrane out of tolerance: {report}"
