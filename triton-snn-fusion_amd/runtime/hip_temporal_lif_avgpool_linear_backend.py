"""LIF -> AvgPool -> Linear backend on libsnnf: drop-in for runtime/triton_temporal_lif_avgpool_linear_backend.py.

Keeps the reference's names (including the deprecated `*_tail` aliases of
runtime/triton_temporal_lif_avgpool_linear_backend.py:111-115) and accepts the `use_autotune` keyword the reference
operator layer passes (runtime/snn_custom_ops.py:1695-1707).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .. import _lib

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)
MAX_TIMESTEPS = _lib.SNNF_MAX_T_PER_LAUNCH
MAX_PLANE_ELEMENTS = 1 << 24


@dataclass
class TritonTemporalLIFAvgPoolLinearResult:
    """Same fields as runtime/triton_temporal_lif_avgpool_linear_backend.py:8-15."""

    out_sum: torch.Tensor
    v_next: torch.Tensor
    used_triton: bool
    kernel_key: str = "temporal_lif_avgpool_linear"
    fallback_reason: str = ""
    kernel_diagnostics: Optional[Dict] = None


def strict_temporal_lif_avgpool_linear_enabled(strict: bool = False) -> bool:
    return bool(strict) or os.environ.get("CHRONOS_STRICT_TEMPORAL_LIF_AVGPOOL_LINEAR_TRITON", "0") == "1"


def _same_place_and_dtype(t: torch.Tensor, like: torch.Tensor) -> bool:
    return t.device == like.device and t.dtype == like.dtype


def _input_reasons(x_seq: torch.Tensor) -> List[str]:
    """What the pooling kernel needs of its input: a [T, N, C, H, W] tensor on the GPU in one of the three dtypes, T within
    one launch, planes that a workgroup can walk."""
    found: List[str] = []
    if x_seq.device.type != "cuda":
        found.append("unsupported_device: x_seq is not CUDA")
    if x_seq.dtype not in SUPPORTED_DTYPES:
        found.append(f"unsupported_dtype: x_seq dtype must be float32, bfloat16 or float16, got {x_seq.dtype}")
    if x_seq.dim() != 5:
        found.append(f"unsupported_rank: x_seq.dim must be 5, got {x_seq.dim()}")
        return found
    T, _, _, H, W = (int(d) for d in x_seq.shape)
    if T < 1 or T > MAX_TIMESTEPS:
        found.append(f"unsupported_temporal_length: T must be in 1..{MAX_TIMESTEPS}, got {T}")
    if H * W > MAX_PLANE_ELEMENTS:
        found.append(f"unsupported_shape: H*W must be at most {MAX_PLANE_ELEMENTS}, got {H * W}")
    return found


def _classifier_reasons(x_seq: torch.Tensor, fc_weight, fc_bias) -> List[str]:
    """[classes, C] weights (and an optional [classes] bias) stored like the activations."""
    if not isinstance(fc_weight, torch.Tensor) or fc_weight.dim() != 2:
        return ["fc_weight must be a 2D tensor"]
    found: List[str] = []
    classes, features = (int(d) for d in fc_weight.shape)
    if x_seq.dim() == 5 and features != int(x_seq.shape[2]):
        found.append(f"unsupported_linear: fc in_features {features} must match channels {int(x_seq.shape[2])}")
    if not _same_place_and_dtype(fc_weight, x_seq):
        found.append("unsupported_dtype: fc_weight device/dtype must match x_seq")
    if isinstance(fc_bias, torch.Tensor) and fc_bias.numel() > 0:      # None or an empty tensor: no bias
        if fc_bias.numel() != classes:
            found.append("unsupported_linear: fc_bias shape does not match out_features")
        if not _same_place_and_dtype(fc_bias, x_seq):
            found.append("unsupported_dtype: fc_bias device/dtype must match x_seq")
    return found


def _state_reasons(x_seq: torch.Tensor, v_init) -> List[str]:
    """A 0-dim `v_init` stands for zeros; a full one must have the neurons' shape, in the activation dtype or float32."""
    if not isinstance(v_init, torch.Tensor):
        return ["v_init must be a tensor"]
    if v_init.dim() == 0:
        return []
    found: List[str] = []
    if x_seq.dim() == 5 and v_init.shape != x_seq.shape[1:]:
        found.append(f"unsupported_membrane_state: v_init shape {tuple(v_init.shape)} does not match {tuple(x_seq.shape[1:])}")
    if v_init.device != x_seq.device or v_init.dtype not in (x_seq.dtype, torch.float32):
        found.append("unsupported_dtype: v_init device/dtype must match x_seq (or be float32)")
    return found


def check_temporal_lif_avgpool_linear_support(x_seq, v_init, fc_weight, fc_bias, tau) -> List[str]:
    """Counterpart of runtime/triton_temporal_lif_avgpool_linear_backend.py:22-55: the reasons (each with the
    `unsupported_*:` prefix the operator layer turns into a statistics key) why a call cannot run on the HIP tail kernels;
    empty when it can. Wider than the reference's: bfloat16, any T up to one launch window, float32 membranes next to
    16-bit activations."""
    if not isinstance(x_seq, torch.Tensor):
        return ["x_seq must be a tensor"]
    reasons = _input_reasons(x_seq) + _state_reasons(x_seq, v_init) + _classifier_reasons(x_seq, fc_weight, fc_bias)
    if float(tau) == 0.0:
        reasons.append("unsupported_tau: tau must be nonzero")
    return reasons


def run_triton_fused_temporal_lif_avgpool_linear(x_seq, v_init, fc_weight, fc_bias, v_threshold: float, v_reset: float,
                                                 tau: float, detach_reset: bool, strict: bool = False,
                                                 verbose: bool = False,
                                                 use_autotune: bool = True) -> TritonTemporalLIFAvgPoolLinearResult:
    reasons = check_temporal_lif_avgpool_linear_support(x_seq, v_init, fc_weight, fc_bias, tau)
    strict = strict_temporal_lif_avgpool_linear_enabled(strict)
    if reasons:
        if verbose:
            print(f"[HIP][FALLBACK][temporal_lif_avgpool_linear] {'; '.join(reasons)}")
        if strict:
            raise RuntimeError("[HIP][STRICT][temporal_lif_avgpool_linear] " + "; ".join(reasons))
        raise RuntimeError("; ".join(reasons))

    lib = _lib.lib()
    x = x_seq if x_seq.is_contiguous() else x_seq.contiguous()
    T, N, C, H, W = (int(d) for d in x.shape)
    K = int(fc_weight.shape[0])
    v_dtype = _lib.membrane_dtype(x, v_init)
    vi = None
    if v_init.dim() != 0:
        vi = v_init if v_init.is_contiguous() else v_init.contiguous()
    w = fc_weight if fc_weight.is_contiguous() else fc_weight.contiguous()
    b = None
    if isinstance(fc_bias, torch.Tensor) and fc_bias.numel() > 0:
        b = fc_bias if fc_bias.is_contiguous() else fc_bias.contiguous()
    out_sum = torch.empty((N, K), dtype=x.dtype, device=x.device)
    v_next = torch.empty((N, C, H, W), dtype=v_dtype, device=x.device)
    ws_bytes = int(lib.snnf_lif_pool_linear_workspace_bytes(N, C))
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    _lib.check("snnf_lif_pool_linear", lib.snnf_lif_pool_linear(
        _lib.packed_step_pointers(x), T, N, C, H, W, _lib.dtype_code(x.dtype), _lib.ptr(vi), _lib.dtype_code(v_dtype),
        w.data_ptr(), _lib.ptr(b), K, _lib.dtype_code(w.dtype), out_sum.data_ptr(), v_next.data_ptr(),
        workspace.data_ptr(), ws_bytes, float(v_threshold), float(v_reset), float(tau), _lib.current_stream(x.device)))
    one_launch = int(lib.snnf_lif_pool_linear_launches(T, N, C, H, W, K)) == 1
    diagnostics = {
        "kernel_kind": "temporal_lif_avgpool_linear",
        # small tails: a workgroup per sample and class range runs the scan, counts in LDS and applies its classifier rows
        "launches": (["lif_scan_counts_and_classifier_per_sample"] if one_launch
                     else ["lif_scan_with_spike_counts_per_plane", "classifier_on_summed_counts"]),
        "workspace": "unused (counts stay in LDS)" if one_launch else f"int32 spike counts [{N}, {C}]",
        "membrane_dtype": str(v_dtype),
        "accumulator_dtype": "float32",
        "timesteps": T,
        "plane": (H, W),
        "classes": K,
    }
    return TritonTemporalLIFAvgPoolLinearResult(out_sum, v_next, True, kernel_diagnostics=diagnostics)


# Deprecated compatibility aliases (runtime/triton_temporal_lif_avgpool_linear_backend.py:111-115).
TritonTemporalLIFTailResult = TritonTemporalLIFAvgPoolLinearResult
strict_temporal_lif_tail_enabled = strict_temporal_lif_avgpool_linear_enabled
check_temporal_lif_tail_support = check_temporal_lif_avgpool_linear_support
run_triton_fused_temporal_lif_tail = run_triton_fused_temporal_lif_avgpool_linear
