"""`snn_custom` torch.library operators with the HIP (libsnnf) backend behind them.

Counterpart of the reference's runtime/snn_custom_ops.py: the same operator namespace, names and schema strings
(runtime/snn_custom_ops.py:1963-2073), the same configuration / statistics functions (`configure_fused_op`,
`get_fused_op_call_stats`, `reset_fused_op_call_stats`, `get_kernel_temporal_configs`, :179-272) and the same eager
functions (`*_torch`, :384-642) that serve CPU tensors and the "torch" backend. FX graphs rewritten by the reference
compiler call `torch.ops.snn_custom.<op>.default` and match operators by that string, so names are part of the ABI.

Backend selection: `configure_fused_op("hip")` (or "triton", the name the reference CLIs pass) routes GPU tensors to
the hand-written HIP kernels; "torch" (the default, as in the reference) runs the eager PyTorch ops. When a call is
outside what the kernels implement, it is counted under `fallback_reasons` and evaluated by the eager ops on the same
device, exactly like the reference (:1052-1058) - unless strict mode is on, which raises instead. A missing libsnnf.so
is never papered over: it raises even in non-strict mode.
"""
from __future__ import annotations

import os
from collections import Counter
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from .. import _lib
from .hip_convlif_backend import (
    check_triton_support,
    classify_conv_lif_config,
    get_autotune_best_config,
    kernel_dtype_diagnostics,
    run_triton_fused_conv_lif_state,
    run_triton_fused_temporal_conv_add_lif_state,
    run_triton_fused_temporal_conv_lif_state,
    run_triton_fused_temporal_conv_lif_state_packed_out,
    run_triton_fused_temporal_depthwise_conv_lif_state,
    run_triton_fused_temporal_pointwise_conv_lif_state,
)
from .hip_temporal_lif_avgpool_linear_backend import run_triton_fused_temporal_lif_avgpool_linear
from .hip_temporal_lif_backend import run_hip_lif_forward_state, run_triton_fused_temporal_lif_state
from .hip_temporal_linear_lif_backend import (
    run_triton_fused_temporal_linear_lif_state,
    run_triton_fused_temporal_linear_lif_state_packed,
    run_triton_fused_temporal_linear_lif_state_packed_out,
)

TORCH_LIBRARY_HANDLES: List[Any] = []
NATIVE_BACKENDS = ("triton", "hip")


@dataclass
class FusedOpConfig:
    backend: str = "torch"
    strict_triton: bool = False
    verbose: bool = False
    use_triton_autotune: bool = True


_CONFIG = FusedOpConfig()

_COUNTER_KEYS = (
    "total", "triton", "fallback", "temporal_total", "temporal_triton", "temporal_fallback",
    "single_k1_s1_p0", "single_k3_s1_p1", "single_k3_s2_p1", "single_k5_s1_p2", "single_k7_s2_p3", "single_k11_s4_p2",
    "temporal_k1_s1_p0", "temporal_k3_s1_p1", "temporal_k3_s2_p1", "temporal_k5_s1_p2", "temporal_k7_s2_p3",
    "temporal_k11_s4_p2", "temporal_depthwise_k3_s1_p1", "temporal_depthwise_k3_s2_p1",
    "temporal_residual_depthwise_k3_s1_p1", "temporal_residual_depthwise_k3_s2_p1",
    "temporal_residual_total", "temporal_residual_triton", "temporal_residual_fallback",
    "temporal_lif_total", "temporal_lif_triton", "temporal_lif_fallback",
    "temporal_lif_avgpool_linear_total", "temporal_lif_avgpool_linear_triton", "temporal_lif_avgpool_linear_fallback",
    "temporal_linear_lif_total", "temporal_linear_lif_triton", "temporal_linear_lif_fallback",
    "temporal_linear_lif_packed_total", "temporal_linear_lif_packed_triton", "temporal_linear_lif_packed_fallback",
    "temporal_linear_lif_stack_materialized",
    "temporal_lif_tail_total", "temporal_lif_tail_triton", "temporal_lif_tail_fallback",
    "temporal_batched_output_total", "temporal_batched_output_layout_projection",
)
_TABLE_KEYS = (
    "kernel_temporal_configs", "temporal_conv_lif_runtime_by_signature",
    "temporal_conv_lif_runtime_fallback_by_signature", "temporal_conv_lif_unsupported_configs",
    "temporal_conv_lif_depthwise_configs", "temporal_conv_lif_grouped_configs", "temporal_conv_lif_pointwise_configs",
)


def _fresh_stats() -> Dict[str, Any]:
    stats: Dict[str, Any] = {key: 0 for key in _COUNTER_KEYS}
    stats.update({key: {} for key in _TABLE_KEYS})
    return stats


_CALL_STATS: Dict[str, Any] = _fresh_stats()
_FALLBACK_REASON_STATS: Counter = Counter()


def configure_fused_op(backend: str = "torch", strict_triton: bool = False, verbose: bool = False,
                       use_triton_autotune: bool = True) -> None:
    """Selects the backend of every snn_custom operator (runtime/snn_custom_ops.py:179-190); "hip" == "triton"."""
    if backend not in ("torch",) + NATIVE_BACKENDS:
        raise ValueError(f"unsupported fused op backend: {backend}")
    _CONFIG.backend = backend
    _CONFIG.strict_triton = bool(strict_triton)
    _CONFIG.verbose = bool(verbose)
    _CONFIG.use_triton_autotune = bool(use_triton_autotune)


def reset_fused_op_call_stats() -> None:
    _CALL_STATS.clear()
    _CALL_STATS.update(_fresh_stats())
    _FALLBACK_REASON_STATS.clear()


def get_fused_op_call_stats() -> Dict[str, Any]:
    out = {key: dict(value) if isinstance(value, dict) else value for key, value in _CALL_STATS.items()}
    out["fallback_reasons"] = dict(_FALLBACK_REASON_STATS)
    return out


def get_kernel_temporal_configs() -> Dict[str, int]:
    return dict(_CALL_STATS.get("kernel_temporal_configs", {}))


def _bump(*keys: str) -> None:
    for key in keys:
        _CALL_STATS[key] = _CALL_STATS.get(key, 0) + 1


def _bump_table(name: str, key: str, amount: int = 1) -> None:
    table = _CALL_STATS.setdefault(name, {})
    table[key] = table.get(key, 0) + amount


# -----------------------------------------------------------------------------------------------------------------
# Fallback bookkeeping (reason vocabulary of runtime/snn_custom_ops.py:129-176)
# -----------------------------------------------------------------------------------------------------------------
_REASON_RULES: Tuple[Tuple[Tuple[str, ...], str], ...] = (
    (("not implemented",), "not_implemented"),
    (("stride",), "unsupported_stride"),
    (("padding",), "unsupported_padding"),
    (("3x3", "kernel"), "unsupported_kernel_size"),
    (("dilation",), "unsupported_dilation"),
    (("groups",), "unsupported_groups"),
    (("float32", "dtype"), "unsupported_dtype"),
    (("bias",), "missing_or_unsupported_bias"),
    (("v_prev", "membrane", "v_init"), "unsupported_membrane_state"),
    (("threshold", "V_THRESHOLD"), "unsupported_threshold"),
    (("V_RESET", "v_reset"), "unsupported_reset"),
    (("tau",), "unsupported_tau"),
    (("detach_reset",), "unsupported_detach_reset"),
)


def _reason_key(reasons) -> str:
    if not reasons:
        return "unknown"
    msg = "; ".join(str(r) for r in reasons)
    for needles, key in _REASON_RULES:
        if any(needle in msg for needle in needles):
            return key
    return "other_unsupported"


def _fallback_reason_keys(reasons) -> List[str]:
    keys = set()
    for reason in reasons or ["unknown"]:
        text = str(reason)
        head = text.split(":", 1)[0]
        keys.add(head if ":" in text and head.startswith("unsupported_") else _reason_key([text]))
    return sorted(keys)


def _record_fallback(kind: str, reasons, shape_desc: str) -> None:
    keys = _fallback_reason_keys(reasons)
    for key in keys:
        _FALLBACK_REASON_STATS[f"{kind}:{key}"] += 1
    if _CONFIG.verbose:
        text = "; ".join(str(r) for r in reasons) if reasons else "unknown"
        print(f"[HIP][FALLBACK][{kind}] reason_key={','.join(keys)}; reason={text}; {shape_desc}")


def _as_pair(value) -> Tuple[int, int]:
    if isinstance(value, int):
        return value, value
    return int(value[0]), int(value[1])


class _Lazy:
    """A description that is only formatted if somebody prints it (verbose mode, fallback reports): building the string
    on every operator call costs more host time than the rest of the dispatch."""
    __slots__ = ("fn", "args", "kwargs")

    def __init__(self, fn, *args, **kwargs):
        self.fn, self.args, self.kwargs = fn, args, kwargs

    def __str__(self) -> str:
        return self.fn(*self.args, **self.kwargs)


def _shape_tuple(x):
    return tuple(x.shape) if isinstance(x, torch.Tensor) else None


def _conv_shape_desc(x, weight, bias, v, stride, padding, dilation, groups, temporal_len=None) -> str:
    if not isinstance(x, torch.Tensor) or not isinstance(weight, torch.Tensor) or x.dim() != 4 or weight.dim() != 4:
        return "shape=<unknown>"
    return (
        f"T={temporal_len if temporal_len is not None else 1}, x={tuple(x.shape)}, weight={tuple(weight.shape)}, "
        f"bias={_shape_tuple(bias)}, v={_shape_tuple(v)}, stride={_as_pair(stride)}, padding={_as_pair(padding)}, "
        f"dilation={_as_pair(dilation)}, groups={groups}, dtype={x.dtype}, device={x.device}"
    )


_SIGNATURE_KEYS: Dict[tuple, str] = {}


def _conv_signature_key(x, weight, stride, padding, dilation, groups) -> str:
    """Same key format as runtime/snn_custom_ops.py:275-297 (summaries of reference drivers parse it). Formatted once per
    distinct layer."""
    if not isinstance(weight, torch.Tensor) or weight.dim() != 4:
        return "unknown_conv_signature"
    try:
        memo = (x.shape[1] if isinstance(x, torch.Tensor) and x.dim() >= 2 else None, weight.shape,
                stride if isinstance(stride, int) else tuple(stride), padding if isinstance(padding, int) else tuple(padding),
                dilation if isinstance(dilation, int) else tuple(dilation), groups)
        known = _SIGNATURE_KEYS.get(memo)
    except TypeError:
        memo, known = None, None
    if known is not None:
        return known
    key = _format_conv_signature_key(x, weight, stride, padding, dilation, groups)
    if memo is not None and len(_SIGNATURE_KEYS) < 4096:
        _SIGNATURE_KEYS[memo] = key
    return key


def _format_conv_signature_key(x, weight, stride, padding, dilation, groups) -> str:
    s, p, d = _as_pair(stride), _as_pair(padding), _as_pair(dilation)
    oc, wic, kh, kw = (int(v) for v in weight.shape)
    groups = int(groups)
    ic = int(x.shape[1]) if isinstance(x, torch.Tensor) and x.dim() >= 2 else wic * groups
    tags = ["depthwise" if groups == ic == oc else ("grouped" if groups != 1 else "standard")]
    if (kh, kw) == (1, 1):
        tags.append("pointwise")
    return (f"k{kh}x{kw}_s{s[0]}x{s[1]}_p{p[0]}x{p[1]}_d{d[0]}x{d[1]}_g{groups}_ic{ic}_oc{oc}_" + "_".join(tags))


def _record_temporal_conv_signature(kind: str, signature: str, status: str, reasons=None) -> None:
    entry_key = f"{kind}:{signature}"
    table = _CALL_STATS.setdefault("temporal_conv_lif_runtime_by_signature", {})
    entry = table.setdefault(entry_key, {"total": 0, "triton": 0, "fallback": 0, "fallback_reasons": {}})
    entry["total"] += 1
    if status == "triton":
        entry["triton"] += 1
    else:
        entry["fallback"] += 1
        for reason_key in _fallback_reason_keys(reasons):
            entry["fallback_reasons"][reason_key] = entry["fallback_reasons"].get(reason_key, 0) + 1
            _bump_table("temporal_conv_lif_runtime_fallback_by_signature", f"{entry_key}|{reason_key}")
            if reason_key.startswith("unsupported_"):
                _bump_table("temporal_conv_lif_unsupported_configs", f"{entry_key}|{reason_key}")
    if "depthwise" in signature:
        _bump_table("temporal_conv_lif_depthwise_configs", entry_key)
    elif "grouped" in signature:
        _bump_table("temporal_conv_lif_grouped_configs", entry_key)
    if "pointwise" in signature:
        _bump_table("temporal_conv_lif_pointwise_configs", entry_key)


def _record_kernel_temporal_config(kind: str, kernel_key: str, config, compute_dtype: str = "float32") -> None:
    if not config:
        return
    btile_t, reuse = config.get("BTILE_T"), config.get("REUSE_GROUPS")
    if btile_t is None or reuse is None:
        key = f"{kind}:{kernel_key}:compute_dtype={compute_dtype}:BLOCK_SIZE={config.get('BLOCK_SIZE')}"
    else:
        key = (f"{kind}:{kernel_key}:compute_dtype={compute_dtype}:BTILE_T={btile_t}:REUSE_GROUPS={reuse}:"
               f"window={config.get('kernel_temporal_window')}")
    _bump_table("kernel_temporal_configs", key)


def _strict() -> bool:
    return bool(_CONFIG.strict_triton) or os.environ.get("CHRONOS_STRICT_TEMPORAL_LIF_TRITON", "0") == "1"


def _compute_dtype(dtype: torch.dtype) -> str:
    return "float16" if dtype == torch.float16 else "float32"


def _native(first) -> bool:
    return _CONFIG.backend in NATIVE_BACKENDS and isinstance(first, torch.Tensor) and first.is_cuda


def _dispatch_reason(what: str) -> str:
    return "backend is not triton" if _CONFIG.backend not in NATIVE_BACKENDS else what


_LIBRARY_SEEN = False


def _require_library() -> None:
    global _LIBRARY_SEEN
    if not _LIBRARY_SEEN:
        if not _lib.library_available():
            _lib.lib()  # raises with the build instruction
        _LIBRARY_SEEN = True


# -----------------------------------------------------------------------------------------------------------------
# Eager implementations (CPU tensors, "torch" backend, and calls outside the kernels' coverage)
# -----------------------------------------------------------------------------------------------------------------
def _ensure_v_prev(x: torch.Tensor, v_prev: torch.Tensor, shape=None) -> torch.Tensor:
    """The membrane a step starts from (runtime/snn_custom_ops.py:378-381): `v_prev` when it has the neurons' shape
    (`shape`, default that of `x`), the device of `x` and the membrane dtype of the call (the activation dtype, or
    float32 next to 16-bit activations, which the native kernels honour as well), zeros of that dtype otherwise."""
    shape = tuple(x.shape if shape is None else shape)
    v_dtype = _lib.membrane_dtype(x, v_prev)
    if (not isinstance(v_prev, torch.Tensor) or v_prev.dim() == 0 or tuple(v_prev.shape) != shape
            or v_prev.device != x.device or v_prev.dtype != v_dtype):
        return torch.zeros(shape, dtype=v_dtype, device=x.device)
    return v_prev


def _lif_step_torch(cur, v, spike_dtype, v_threshold: float, v_reset: float, tau: float, detach_reset: bool):
    """One LIF update (runtime/snn_custom_ops.py:384-409) of the input current `cur` on the membrane `v` (same dtype)."""
    h = v + cur if float(tau) <= 1.0 else v + (cur - v) / float(tau)
    spike = (h >= float(v_threshold)).to(spike_dtype)
    gate = spike.detach() if bool(detach_reset) else spike
    if float(v_reset) < 0:
        v_next = h - gate.to(h.dtype) * float(v_threshold)
    else:
        v_next = torch.where(gate.bool(), torch.full_like(h, float(v_reset)), h)
    return spike, v_next


def lif_forward_state_torch(x, v_prev, v_threshold: float, v_reset: float, tau: float, detach_reset: bool):
    v = _ensure_v_prev(x, v_prev)
    cur = x if x.dtype == v.dtype else x.to(v.dtype)     # float32 membrane next to 16-bit activations: step in float32
    return _lif_step_torch(cur, v, x.dtype, v_threshold, v_reset, tau, detach_reset)


def _wide(x, v_prev, *operands):
    """Operands of a layer whose membrane is float32 while its activations are 16 bit, converted to float32: the eager
    path then accumulates and steps in float32 like the kernels (16-bit operands, float32 accumulator and membrane)."""
    if _lib.membrane_dtype(x, v_prev) == x.dtype:
        return (x,) + operands
    return (x.float(),) + tuple(None if t is None else t.float() for t in operands)


def fused_conv_lif_state_torch(x, weight, bias, v_prev, stride, padding, dilation, groups: int, v_threshold: float,
                               v_reset: float, tau: float, detach_reset: bool, residual=None):
    xw, ww, bw, rw = _wide(x, v_prev, weight, bias, residual)
    cur = F.conv2d(xw, ww, bw, stride, padding, dilation, groups)
    if rw is not None:
        cur = cur + rw
    v = _ensure_v_prev(x, v_prev, cur.shape)
    return _lif_step_torch(cur, v, x.dtype, v_threshold, v_reset, tau, detach_reset)


def fused_temporal_conv_lif_state_torch(xs, weight, bias, v_init, stride, padding, dilation, groups: int,
                                        v_threshold: float, v_reset: float, tau: float, detach_reset: bool):
    if len(xs) == 0:
        raise RuntimeError("fused_temporal_conv_lif_state requires at least one input tensor")
    v, spikes = v_init, []
    for x in xs:
        s, v = fused_conv_lif_state_torch(x, weight, bias, v, stride, padding, dilation, groups, v_threshold, v_reset,
                                          tau, detach_reset)
        spikes.append(s)
    return torch.stack(spikes, dim=0), v


def fused_temporal_conv_lif_state_packed_out_torch(x_seq, weight, bias, v_init, stride, padding, dilation, groups: int,
                                                   v_threshold: float, v_reset: float, tau: float, detach_reset: bool,
                                                   spike_out, v_out):
    stack, v = fused_temporal_conv_lif_state_torch([x_seq[t] for t in range(int(x_seq.shape[0]))], weight, bias, v_init,
                                                   stride, padding, dilation, groups, v_threshold, v_reset, tau,
                                                   detach_reset)
    spike_out.copy_(stack)
    v_out.copy_(v)
    return None


def fused_temporal_conv_add_lif_state_torch(xs, residuals, weight, bias, v_init, stride, padding, dilation,
                                            groups: int, v_threshold: float, v_reset: float, tau: float,
                                            detach_reset: bool):
    if len(xs) == 0:
        raise RuntimeError("fused_temporal_conv_add_lif_state requires at least one input tensor")
    if len(xs) != len(residuals):
        raise RuntimeError("xs and residuals must have the same temporal length")
    v, spikes = v_init, []
    for x, residual in zip(xs, residuals):
        s, v = fused_conv_lif_state_torch(x, weight, bias, v, stride, padding, dilation, groups, v_threshold, v_reset, tau,
                                          detach_reset, residual=residual)
        spikes.append(s)
    return torch.stack(spikes, dim=0), v


def fused_temporal_lif_state_torch(x_seq, v_init, v_threshold: float, v_reset: float, tau: float, detach_reset: bool):
    if x_seq.dim() != 5:
        raise RuntimeError(f"fused_temporal_lif_state requires x_seq [T,N,C,H,W], got dim={x_seq.dim()}")
    v, spikes = v_init, []
    for t in range(int(x_seq.shape[0])):
        s, v = lif_forward_state_torch(x_seq[t], v, v_threshold, v_reset, tau, detach_reset)
        spikes.append(s)
    return torch.stack(spikes, dim=0), v


def _optional_bias(bias):
    return bias if isinstance(bias, torch.Tensor) and bias.numel() > 0 else None


def fused_temporal_lif_avgpool_linear_torch(x_seq, v_init, fc_weight, fc_bias, v_threshold: float, v_reset: float,
                                            tau: float, detach_reset: bool):
    if x_seq.dim() != 5:
        raise RuntimeError(f"fused_temporal_lif_avgpool_linear requires x_seq [T,N,C,H,W], got dim={x_seq.dim()}")
    v, out_sum = v_init, None
    for t in range(int(x_seq.shape[0])):
        s, v = lif_forward_state_torch(x_seq[t], v, v_threshold, v_reset, tau, detach_reset)
        logits = F.linear(F.adaptive_avg_pool2d(s, (1, 1)).flatten(1), fc_weight, _optional_bias(fc_bias))
        out_sum = logits if out_sum is None else out_sum + logits
    return out_sum, v


fused_temporal_lif_tail_torch = fused_temporal_lif_avgpool_linear_torch  # deprecated alias kept by the reference


def fused_temporal_linear_lif_state_torch(xs, weight, bias, v_init, v_threshold: float, v_reset: float, tau: float,
                                          detach_reset: bool):
    if len(xs) == 0:
        raise RuntimeError("fused_temporal_linear_lif_state requires at least one input tensor")
    v, spikes = v_init, []
    for x in xs:
        xw, ww, bw = _wide(x, v, weight, _optional_bias(bias))
        cur = F.linear(xw, ww, bw)
        vv = _ensure_v_prev(x, v, cur.shape)
        s, v = _lif_step_torch(cur, vv, x.dtype, v_threshold, v_reset, tau, detach_reset)
        spikes.append(s)
    return torch.stack(spikes, dim=0), v


def _check_packed_linear(x_seq, weight) -> None:
    if x_seq.dim() < 3:
        raise RuntimeError(f"fused_temporal_linear_lif_state_packed requires x_seq [T,...,Fin], got dim={x_seq.dim()}")
    if weight.dim() != 2:
        raise RuntimeError(f"fused_temporal_linear_lif_state_packed requires rank-2 weight, got dim={weight.dim()}")
    if int(x_seq.shape[-1]) != int(weight.shape[1]):
        raise RuntimeError("fused_temporal_linear_lif_state_packed input feature mismatch: "
                           f"x_seq.shape[-1]={int(x_seq.shape[-1])}, weight.shape[1]={int(weight.shape[1])}")


def fused_temporal_linear_lif_state_packed_torch(x_seq, weight, bias, v_init, v_threshold: float, v_reset: float,
                                                 tau: float, detach_reset: bool):
    _check_packed_linear(x_seq, weight)
    return fused_temporal_linear_lif_state_torch([x_seq[t] for t in range(int(x_seq.shape[0]))], weight, bias, v_init,
                                                 v_threshold, v_reset, tau, detach_reset)


def fused_temporal_linear_lif_state_packed_out_torch(x_seq, weight, bias, v_init, v_threshold: float, v_reset: float,
                                                     tau: float, detach_reset: bool, spike_out, v_out):
    stack, v = fused_temporal_linear_lif_state_packed_torch(x_seq, weight, bias, v_init, v_threshold, v_reset, tau,
                                                            detach_reset)
    spike_out.copy_(stack)
    v_out.copy_(v)
    return None


# -----------------------------------------------------------------------------------------------------------------
# Meta (shape) functions (runtime/snn_custom_ops.py:645-875). The membrane output follows v_init's dtype when that is
# float32 or the activation dtype, which is x.dtype in every configuration the reference supports.
# -----------------------------------------------------------------------------------------------------------------
def _v_dtype(x, v_init) -> torch.dtype:
    return _lib.membrane_dtype(x, v_init)


def _conv_out_shape(x, weight, stride, padding, dilation):
    s, p, d = _as_pair(stride), _as_pair(padding), _as_pair(dilation)
    kh, kw = int(weight.shape[2]), int(weight.shape[3])
    ho = (int(x.shape[2]) + 2 * p[0] - d[0] * (kh - 1) - 1) // s[0] + 1
    wo = (int(x.shape[3]) + 2 * p[1] - d[1] * (kw - 1) - 1) // s[1] + 1
    return int(x.shape[0]), int(weight.shape[0]), ho, wo


def _lif_forward_state_meta(x, v_prev, v_threshold, v_reset, tau, detach_reset):
    return x.new_empty(x.shape), x.new_empty(x.shape, dtype=_v_dtype(x, v_prev))


def _fused_conv_lif_state_meta(x, weight, bias, v_prev, stride, padding, dilation, groups, v_threshold, v_reset, tau,
                               detach_reset):
    shape = _conv_out_shape(x, weight, stride, padding, dilation)
    return x.new_empty(shape), x.new_empty(shape, dtype=_v_dtype(x, v_prev))


def _temporal_conv_meta(name: str, batched: bool):
    def meta(xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau, detach_reset):
        if len(xs) == 0:
            raise RuntimeError(f"{name} requires at least one input tensor")
        shape = _conv_out_shape(xs[0], weight, stride, padding, dilation)
        lead = (len(xs) * shape[0],) + tuple(shape[1:]) if batched else (len(xs),) + tuple(shape)
        return xs[0].new_empty(lead), xs[0].new_empty(shape, dtype=_v_dtype(xs[0], v_init))
    return meta


def _temporal_conv_add_meta(name: str, batched: bool):
    inner = _temporal_conv_meta(name, batched)

    def meta(xs, residuals, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau,
             detach_reset):
        return inner(xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau,
                     detach_reset)
    return meta


def _returns_none_meta(*args):
    return None


def _fused_temporal_lif_state_meta(x_seq, v_init, v_threshold, v_reset, tau, detach_reset):
    if x_seq.dim() != 5:
        raise RuntimeError(f"fused_temporal_lif_state requires x_seq [T,N,C,H,W], got dim={x_seq.dim()}")
    return x_seq.new_empty(x_seq.shape), x_seq.new_empty(x_seq.shape[1:], dtype=_v_dtype(x_seq, v_init))


def _fused_temporal_lif_avgpool_linear_meta(x_seq, v_init, fc_weight, fc_bias, v_threshold, v_reset, tau, detach_reset):
    if x_seq.dim() != 5:
        raise RuntimeError(f"fused_temporal_lif_avgpool_linear requires x_seq [T,N,C,H,W], got dim={x_seq.dim()}")
    return (x_seq.new_empty((x_seq.shape[1], fc_weight.shape[0])),
            x_seq.new_empty(x_seq.shape[1:], dtype=_v_dtype(x_seq, v_init)))


def _fused_temporal_linear_lif_state_meta(xs, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset):
    if len(xs) == 0:
        raise RuntimeError("fused_temporal_linear_lif_state requires at least one input tensor")
    first = xs[0]
    if first.dim() != 2:
        raise RuntimeError(f"fused_temporal_linear_lif_state requires rank-2 inputs, got dim={first.dim()}")
    shape = (first.shape[0], weight.shape[0])
    return first.new_empty((len(xs),) + tuple(shape)), first.new_empty(shape, dtype=_v_dtype(first, v_init))


def _fused_temporal_linear_lif_state_packed_meta(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset):
    _check_packed_linear(x_seq, weight)
    lead = tuple(x_seq.shape[1:-1])
    return (x_seq.new_empty((x_seq.shape[0],) + lead + (weight.shape[0],)),
            x_seq.new_empty(lead + (weight.shape[0],), dtype=_v_dtype(x_seq, v_init)))


# -----------------------------------------------------------------------------------------------------------------
# Dispatch
# -----------------------------------------------------------------------------------------------------------------
def _run(first, counters: Sequence[str], fallback_kind: str, shape_desc: str, native: Callable[[], Any],
         eager: Callable[[], Any], on_hit: Optional[Callable[[Any], None]] = None,
         on_miss: Optional[Callable[[List[str]], None]] = None, not_gpu_reason: str = "x is not CUDA",
         strict: Optional[bool] = None):
    """Shared body of every operator: count, try the HIP backend, else count the fallback and run the eager ops.

    `counters` are the stat prefixes of this operator family ("temporal", "temporal_lif", ...): `<p>_total`,
    `<p>_triton`, `<p>_fallback` are bumped next to the global `total` / `triton` / `fallback`.
    """
    _bump("total", *[f"{p}_total" for p in counters])
    if _native(first):
        _require_library()
        try:
            result = native()
        except Exception as exc:  # the reference catches everything (runtime/snn_custom_ops.py:1052)
            _bump("fallback", *[f"{p}_fallback" for p in counters])
            _record_fallback(fallback_kind, [str(exc)], shape_desc)
            if on_miss is not None:
                on_miss([str(exc)])
            if (_strict() if strict is None else strict) or isinstance(exc, _lib.SnnfError) and exc.status == -3:
                raise
        else:
            _bump("triton", *[f"{p}_triton" for p in counters])
            if on_hit is not None:
                on_hit(result)
            return result, True
    else:
        reason = _dispatch_reason(not_gpu_reason)
        _bump("fallback", *[f"{p}_fallback" for p in counters])
        _record_fallback(f"{fallback_kind}_dispatch", [reason], shape_desc)
        if on_miss is not None:
            on_miss([reason])
    return eager(), False


def _lif_forward_state_impl(x, v_prev, v_threshold, v_reset, tau, detach_reset):
    """Single LIF step. The reference keeps this operator on eager ops and counts nothing for it
    (runtime/snn_custom_ops.py:878-879); with the native backend selected a GPU tensor goes through the scan kernel
    (one launch instead of seven elementwise ones), uncounted as well."""
    if _native(x):
        _require_library()
        try:
            return run_hip_lif_forward_state(x, v_prev, v_threshold, v_reset, tau)
        except _lib.SnnfError:
            raise
        except RuntimeError:
            if _strict():
                raise
    return lif_forward_state_torch(x, v_prev, v_threshold, v_reset, tau, detach_reset)


def _fused_conv_lif_state_impl(x, weight, bias, v_prev, stride, padding, dilation, groups, v_threshold, v_reset, tau,
                               detach_reset):
    desc = _Lazy(_conv_shape_desc, x, weight, bias, v_prev, stride, padding, dilation, groups)
    args = (x, weight, bias, v_prev, stride, padding, dilation, groups, v_threshold, v_reset, tau, detach_reset)

    def hit(result):
        _bump(f"single_{result.kernel_key}")
        _record_kernel_temporal_config("single", result.kernel_key, result.kernel_temporal_config, _compute_dtype(x.dtype))
        if _CONFIG.verbose:
            print(f"[HIP][HIT][single][{result.kernel_key}] {desc}")

    out, native = _run(x, (), "single", desc,
                       lambda: run_triton_fused_conv_lif_state(*args, strict=_CONFIG.strict_triton, verbose=_CONFIG.verbose,
                                                               compute_dtype=_compute_dtype(x.dtype)),
                       lambda: fused_conv_lif_state_torch(*args), on_hit=hit, strict=_CONFIG.strict_triton)
    return (out.spikes, out.v_next) if native else out


def _temporal_conv_impl(op_name: str, runner, stats_kind: str):
    """Builds the implementation of one `Tensor[] xs` conv operator (regular / pointwise / depthwise)."""

    def impl(xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau, detach_reset):
        first = xs[0] if len(xs) > 0 else None
        desc = _Lazy(_conv_shape_desc, first, weight, bias, v_init, stride, padding, dilation, groups, temporal_len=len(xs))
        signature = _conv_signature_key(first, weight, stride, padding, dilation, groups)
        args = (xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau, detach_reset)

        def hit(result):
            cd = _compute_dtype(first.dtype)
            _bump(f"temporal_{result.kernel_key}")
            _record_kernel_temporal_config("temporal", result.kernel_key, result.kernel_temporal_config, cd)
            _record_temporal_conv_signature(stats_kind, signature, "triton")
            if _CONFIG.verbose:
                print(f"[HIP][HIT][{stats_kind}][{result.kernel_key}] {desc}")

        out, native = _run(first, ("temporal",), stats_kind if stats_kind != "temporal" else "temporal", desc,
                           lambda: runner(*args, strict=_CONFIG.strict_triton, verbose=_CONFIG.verbose,
                                          compute_dtype=_compute_dtype(first.dtype),
                                          use_autotune=_CONFIG.use_triton_autotune),
                           lambda: fused_temporal_conv_lif_state_torch(*args), on_hit=hit,
                           on_miss=lambda reasons: _record_temporal_conv_signature(stats_kind, signature, "fallback", reasons),
                           not_gpu_reason="first_x is not CUDA or xs is empty")
        return (out.spikes, out.v_next) if native else out

    impl.__name__ = f"_{op_name}_impl"
    return impl


_fused_temporal_conv_lif_state_impl = _temporal_conv_impl(
    "fused_temporal_conv_lif_state", run_triton_fused_temporal_conv_lif_state, "temporal")
_fused_temporal_pointwise_conv_lif_state_impl = _temporal_conv_impl(
    "fused_temporal_pointwise_conv_lif_state", run_triton_fused_temporal_pointwise_conv_lif_state,
    "fused_temporal_pointwise_conv_lif_state")
_fused_temporal_depthwise_conv_lif_state_impl = _temporal_conv_impl(
    "fused_temporal_depthwise_conv_lif_state", run_triton_fused_temporal_depthwise_conv_lif_state,
    "fused_temporal_depthwise_conv_lif_state")


def _fused_temporal_conv_lif_state_packed_out_impl(x_seq, weight, bias, v_init, stride, padding, dilation, groups,
                                                   v_threshold, v_reset, tau, detach_reset, spike_out, v_out):
    first = x_seq[0] if isinstance(x_seq, torch.Tensor) and x_seq.dim() == 5 else None
    T = int(x_seq.shape[0]) if isinstance(x_seq, torch.Tensor) and x_seq.dim() > 0 else None
    desc = _Lazy(_conv_shape_desc, first, weight, bias, v_init, stride, padding, dilation, groups, temporal_len=T)
    signature = _conv_signature_key(first, weight, stride, padding, dilation, groups)
    args = (x_seq, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau, detach_reset,
            spike_out, v_out)

    def hit(result):
        _bump(f"temporal_{result.kernel_key}")
        _record_kernel_temporal_config("temporal", result.kernel_key, result.kernel_temporal_config, _compute_dtype(first.dtype))
        _record_temporal_conv_signature("temporal", signature, "triton")

    _run(first, ("temporal",), "temporal_out", desc,
         lambda: run_triton_fused_temporal_conv_lif_state_packed_out(
             *args, strict=_CONFIG.strict_triton, verbose=_CONFIG.verbose,
             compute_dtype=_compute_dtype(first.dtype), use_autotune=_CONFIG.use_triton_autotune),
         lambda: fused_temporal_conv_lif_state_packed_out_torch(*args), on_hit=hit,
         on_miss=lambda reasons: _record_temporal_conv_signature("temporal", signature, "fallback", reasons),
         not_gpu_reason="x_seq is not CUDA or invalid")
    return None


def _flatten_temporal_stack_to_batched_tn(spike_stack: torch.Tensor) -> torch.Tensor:
    if spike_stack.dim() != 5:
        raise RuntimeError(f"expected spike stack [T,N,C,H,W], got shape={tuple(spike_stack.shape)}")
    _bump("temporal_batched_output_layout_projection")
    return spike_stack.flatten(0, 1)


def _fused_temporal_conv_lif_state_batched_tn_impl(*args):
    _bump("temporal_batched_output_total")
    stack, v = _fused_temporal_conv_lif_state_impl(*args)
    return _flatten_temporal_stack_to_batched_tn(stack), v


def _temporal_conv_add_impl(require_depthwise: bool):
    def impl(xs, residuals, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau,
             detach_reset):
        first = xs[0] if len(xs) > 0 else None
        desc = _Lazy(_conv_shape_desc, first, weight, bias, v_init, stride, padding, dilation, groups, temporal_len=len(xs))
        signature = _conv_signature_key(first, weight, stride, padding, dilation, groups)
        args = (xs, residuals, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau,
                detach_reset)

        def native():
            result = run_triton_fused_temporal_conv_add_lif_state(
                *args, strict=_CONFIG.strict_triton, verbose=_CONFIG.verbose,
                compute_dtype=_compute_dtype(first.dtype), use_autotune=_CONFIG.use_triton_autotune)
            if require_depthwise and not result.kernel_key.startswith("depthwise_"):
                raise RuntimeError(f"depthwise residual op requires depthwise kernel, got {result.kernel_key}")
            return result

        def hit(result):
            key = result.kernel_key
            _bump(f"temporal_residual_{key}" if key.startswith("depthwise_") else f"temporal_{key}")
            _record_kernel_temporal_config("temporal_residual", key, result.kernel_temporal_config, _compute_dtype(first.dtype))
            _record_temporal_conv_signature("temporal_residual", signature, "triton")
            if _CONFIG.verbose:
                print(f"[HIP][HIT][temporal_residual][{key}] {desc}")

        out, was_native = _run(first, ("temporal", "temporal_residual"), "temporal_residual", desc, native,
                               lambda: fused_temporal_conv_add_lif_state_torch(*args), on_hit=hit,
                               on_miss=lambda reasons: _record_temporal_conv_signature("temporal_residual", signature, "fallback", reasons),
                               not_gpu_reason="first_x is not CUDA or xs is empty")
        return (out.spikes, out.v_next) if was_native else out
    return impl


_fused_temporal_conv_add_lif_state_impl = _temporal_conv_add_impl(False)
_fused_temporal_conv_add_lif_state_depthwise_impl = _temporal_conv_add_impl(True)


def _fused_temporal_conv_add_lif_state_batched_tn_impl(*args):
    _bump("temporal_batched_output_total")
    stack, v = _fused_temporal_conv_add_lif_state_impl(*args)
    return _flatten_temporal_stack_to_batched_tn(stack), v


def _lif_shape_desc(x_seq, v_init) -> str:
    if not isinstance(x_seq, torch.Tensor):
        return "shape=<unknown>"
    return f"x_seq={tuple(x_seq.shape)}, v={_shape_tuple(v_init)}, dtype={x_seq.dtype}, device={x_seq.device}"


def _fused_temporal_lif_state_impl(x_seq, v_init, v_threshold, v_reset, tau, detach_reset):
    desc = _Lazy(_lif_shape_desc, x_seq, v_init)
    args = (x_seq, v_init, v_threshold, v_reset, tau, detach_reset)

    def hit(result):
        _record_kernel_temporal_config("temporal_lif", result.kernel_key, result.kernel_temporal_config,
                                       _compute_dtype(x_seq.dtype))
        if _CONFIG.verbose:
            print(f"[HIP][HIT][temporal_lif] {result.kernel_diagnostics} {desc}")

    out, native = _run(x_seq, ("temporal", "temporal_lif"), "temporal_lif", desc,
                       lambda: run_triton_fused_temporal_lif_state(*args, strict=_CONFIG.strict_triton,
                                                                   verbose=_CONFIG.verbose,
                                                                   use_autotune=_CONFIG.use_triton_autotune),
                       lambda: fused_temporal_lif_state_torch(*args), on_hit=hit, not_gpu_reason="x_seq is not CUDA",
                       strict=_CONFIG.strict_triton)
    return (out.spikes, out.v_next) if native else out


def _fused_temporal_lif_avgpool_linear_impl(x_seq, v_init, fc_weight, fc_bias, v_threshold, v_reset, tau, detach_reset):
    desc = _Lazy(_lif_shape_desc, x_seq, v_init)
    args = (x_seq, v_init, fc_weight, fc_bias, v_threshold, v_reset, tau, detach_reset)
    out, native = _run(x_seq, ("temporal", "temporal_lif_avgpool_linear", "temporal_lif_tail"),
                       "temporal_lif_avgpool_linear", desc,
                       lambda: run_triton_fused_temporal_lif_avgpool_linear(*args, strict=_CONFIG.strict_triton,
                                                                            verbose=_CONFIG.verbose,
                                                                            use_autotune=_CONFIG.use_triton_autotune),
                       lambda: fused_temporal_lif_avgpool_linear_torch(*args), not_gpu_reason="x_seq is not CUDA",
                       strict=_CONFIG.strict_triton)
    return (out.out_sum, out.v_next) if native else out


def _linear_shape_desc(xs, weight, bias, v_init) -> str:
    if isinstance(xs, torch.Tensor):
        x_shape, dtype, device = tuple(xs.shape), xs.dtype, xs.device
    elif isinstance(xs, (list, tuple)) and len(xs) > 0 and isinstance(xs[0], torch.Tensor):
        x_shape, dtype, device = (len(xs),) + tuple(xs[0].shape), xs[0].dtype, xs[0].device
    else:
        return "shape=<unknown>"
    return (f"x={x_shape}, weight={_shape_tuple(weight)}, bias={_shape_tuple(bias)}, v={_shape_tuple(v_init)}, "
            f"dtype={dtype}, device={device}")


def _linear_hit(kind: str, dtype):
    def hit(result):
        if result.kernel_diagnostics and result.kernel_diagnostics.get("stack_materialized"):
            _bump("temporal_linear_lif_stack_materialized")
        _record_kernel_temporal_config(kind, result.kernel_key, result.kernel_temporal_config, _compute_dtype(dtype))
        if _CONFIG.verbose:
            print(f"[HIP][HIT][{kind}] {result.kernel_diagnostics}")
    return hit


def _fused_temporal_linear_lif_state_impl(xs, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset):
    first = xs[0] if isinstance(xs, torch.Tensor) or (isinstance(xs, (tuple, list)) and len(xs) > 0) else None
    args = (xs, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset)
    out, native = _run(first, ("temporal", "temporal_linear_lif"), "temporal_linear_lif",
                       _Lazy(_linear_shape_desc, xs, weight, bias, v_init),
                       lambda: run_triton_fused_temporal_linear_lif_state(*args, strict=_CONFIG.strict_triton,
                                                                          verbose=_CONFIG.verbose),
                       lambda: fused_temporal_linear_lif_state_torch(*args),
                       on_hit=_linear_hit("temporal_linear_lif", getattr(first, "dtype", torch.float32)),
                       not_gpu_reason="first_x is not CUDA or xs is empty", strict=_CONFIG.strict_triton)
    return (out.spikes, out.v_next) if native else out


def _fused_temporal_linear_lif_state_packed_impl(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset):
    args = (x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset)
    out, native = _run(x_seq, ("temporal", "temporal_linear_lif", "temporal_linear_lif_packed"),
                       "temporal_linear_lif_packed", _Lazy(_linear_shape_desc, x_seq, weight, bias, v_init),
                       lambda: run_triton_fused_temporal_linear_lif_state_packed(*args, strict=_CONFIG.strict_triton,
                                                                                 verbose=_CONFIG.verbose),
                       lambda: fused_temporal_linear_lif_state_packed_torch(*args),
                       on_hit=_linear_hit("temporal_linear_lif_packed", getattr(x_seq, "dtype", torch.float32)),
                       not_gpu_reason="x_seq is not CUDA", strict=_CONFIG.strict_triton)
    return (out.spikes, out.v_next) if native else out


def _fused_temporal_linear_lif_state_packed_out_impl(x_seq, weight, bias, v_init, v_threshold, v_reset, tau,
                                                     detach_reset, spike_out, v_out):
    args = (x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset, spike_out, v_out)
    _run(x_seq, ("temporal", "temporal_linear_lif", "temporal_linear_lif_packed"), "temporal_linear_lif_packed_out",
         _Lazy(_linear_shape_desc, x_seq, weight, bias, v_init),
         lambda: run_triton_fused_temporal_linear_lif_state_packed_out(*args, strict=_CONFIG.strict_triton,
                                                                       verbose=_CONFIG.verbose,
                                                                       use_autotune=_CONFIG.use_triton_autotune),
         lambda: fused_temporal_linear_lif_state_packed_out_torch(*args),
         on_hit=_linear_hit("temporal_linear_lif_packed", getattr(x_seq, "dtype", torch.float32)),
         not_gpu_reason="x_seq is not CUDA", strict=_CONFIG.strict_triton)
    return None


# -----------------------------------------------------------------------------------------------------------------
# Registration: schema strings identical to runtime/snn_custom_ops.py:1966-2073.
# -----------------------------------------------------------------------------------------------------------------
_CONV = "int[] stride, int[] padding, int[] dilation, int groups"
_LIF = "float v_threshold, float v_reset, float tau, bool detach_reset"
_XS_CONV = f"Tensor[] xs, Tensor weight, Tensor bias, Tensor v_init, {_CONV}, {_LIF}"
_XS_ADD_CONV = f"Tensor[] xs, Tensor[] residuals, Tensor weight, Tensor bias, Tensor v_init, {_CONV}, {_LIF}"

# name -> (schema, gpu/cpu implementation, cpu-only implementation or None, meta implementation)
OPERATORS: Dict[str, Tuple[str, Callable, Optional[Callable], Callable]] = {
    "lif_forward_state": (f"(Tensor x, Tensor v_prev, {_LIF}) -> (Tensor, Tensor)",
                          _lif_forward_state_impl, None, _lif_forward_state_meta),
    "fused_conv_lif_state": (f"(Tensor x, Tensor weight, Tensor bias, Tensor v_prev, {_CONV}, {_LIF}) -> (Tensor, Tensor)",
                             _fused_conv_lif_state_impl, None, _fused_conv_lif_state_meta),
    "fused_temporal_conv_lif_state": (f"({_XS_CONV}) -> (Tensor, Tensor)", _fused_temporal_conv_lif_state_impl, None,
                                      _temporal_conv_meta("fused_temporal_conv_lif_state", False)),
    "fused_temporal_pointwise_conv_lif_state": (f"({_XS_CONV}) -> (Tensor, Tensor)",
                                                _fused_temporal_pointwise_conv_lif_state_impl,
                                                _fused_temporal_conv_lif_state_impl,
                                                _temporal_conv_meta("fused_temporal_pointwise_conv_lif_state", False)),
    "fused_temporal_depthwise_conv_lif_state": (f"({_XS_CONV}) -> (Tensor, Tensor)",
                                                _fused_temporal_depthwise_conv_lif_state_impl,
                                                _fused_temporal_conv_lif_state_impl,
                                                _temporal_conv_meta("fused_temporal_depthwise_conv_lif_state", False)),
    "fused_temporal_conv_lif_state_depthwise": (f"({_XS_CONV}) -> (Tensor, Tensor)",
                                                _fused_temporal_depthwise_conv_lif_state_impl,
                                                _fused_temporal_conv_lif_state_impl,
                                                _temporal_conv_meta("fused_temporal_conv_lif_state_depthwise", False)),
    "fused_temporal_conv_lif_state_packed_out": (
        f"(Tensor x_seq, Tensor weight, Tensor bias, Tensor v_init, {_CONV}, {_LIF}, "
        "Tensor(a!) spike_out, Tensor(b!) v_out) -> ()",
        _fused_temporal_conv_lif_state_packed_out_impl, None, _returns_none_meta),
    "fused_temporal_conv_lif_state_batched_tn": (f"({_XS_CONV}) -> (Tensor, Tensor)",
                                                 _fused_temporal_conv_lif_state_batched_tn_impl, None,
                                                 _temporal_conv_meta("fused_temporal_conv_lif_state_batched_tn", True)),
    "fused_temporal_conv_add_lif_state": (f"({_XS_ADD_CONV}) -> (Tensor, Tensor)",
                                          _fused_temporal_conv_add_lif_state_impl, None,
                                          _temporal_conv_add_meta("fused_temporal_conv_add_lif_state", False)),
    "fused_temporal_conv_add_lif_state_depthwise": (f"({_XS_ADD_CONV}) -> (Tensor, Tensor)",
                                                    _fused_temporal_conv_add_lif_state_depthwise_impl,
                                                    _fused_temporal_conv_add_lif_state_impl,
                                                    _temporal_conv_add_meta("fused_temporal_conv_add_lif_state_depthwise", False)),
    "fused_temporal_conv_add_lif_state_batched_tn": (f"({_XS_ADD_CONV}) -> (Tensor, Tensor)",
                                                     _fused_temporal_conv_add_lif_state_batched_tn_impl, None,
                                                     _temporal_conv_add_meta("fused_temporal_conv_add_lif_state_batched_tn", True)),
    "fused_temporal_lif_state": (f"(Tensor x_seq, Tensor v_init, {_LIF}) -> (Tensor, Tensor)",
                                 _fused_temporal_lif_state_impl, None, _fused_temporal_lif_state_meta),
    "fused_temporal_lif_avgpool_linear": (
        f"(Tensor x_seq, Tensor v_init, Tensor fc_weight, Tensor fc_bias, {_LIF}) -> (Tensor, Tensor)",
        _fused_temporal_lif_avgpool_linear_impl, None, _fused_temporal_lif_avgpool_linear_meta),
    "fused_temporal_linear_lif_state": (
        f"(Tensor[] xs, Tensor weight, Tensor? bias, Tensor v_init, {_LIF}) -> (Tensor, Tensor)",
        _fused_temporal_linear_lif_state_impl, None, _fused_temporal_linear_lif_state_meta),
    "fused_temporal_linear_lif_state_packed": (
        f"(Tensor x_seq, Tensor weight, Tensor? bias, Tensor v_init, {_LIF}) -> (Tensor, Tensor)",
        _fused_temporal_linear_lif_state_packed_impl, None, _fused_temporal_linear_lif_state_packed_meta),
    "fused_temporal_linear_lif_state_packed_out": (
        f"(Tensor x_seq, Tensor weight, Tensor? bias, Tensor v_init, {_LIF}, "
        "Tensor(a!) spike_out, Tensor(b!) v_out) -> ()",
        _fused_temporal_linear_lif_state_packed_out_impl, None, _returns_none_meta),
    "fused_temporal_lif_tail": (
        f"(Tensor x_seq, Tensor v_init, Tensor fc_weight, Tensor fc_bias, {_LIF}) -> (Tensor, Tensor)",
        _fused_temporal_lif_avgpool_linear_impl, None, _fused_temporal_lif_avgpool_linear_meta),
}


def register_snn_custom_ops() -> None:
    """Defines and implements the `snn_custom` library once per process (a second definition is ignored, like the
    reference's try/except around registration, runtime/snn_custom_ops.py:1964-2076)."""
    try:
        def_lib = torch.library.Library("snn_custom", "DEF")
        for name, (schema, _, _, _) in OPERATORS.items():
            def_lib.define(name + schema)
        TORCH_LIBRARY_HANDLES.append(def_lib)
    except RuntimeError:
        pass
    try:
        impl_lib = torch.library.Library("snn_custom", "IMPL")
        for name, (_, gpu_impl, cpu_impl, meta_impl) in OPERATORS.items():
            impl_lib.impl(name, cpu_impl if cpu_impl is not None else gpu_impl, "CPU")
            impl_lib.impl(name, gpu_impl, "CUDA")
            impl_lib.impl(name, meta_impl, "Meta")
        TORCH_LIBRARY_HANDLES.append(impl_lib)
    except RuntimeError:
        pass


register_snn_custom_ops()
