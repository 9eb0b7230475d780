"""Temporal Linear + LIF backend on libsnnf: drop-in for runtime/triton_temporal_linear_lif_backend.py.

The list form consumes the T input tensors in place (no torch.stack, runtime/triton_temporal_linear_lif_backend.py:105);
`stack_materialized` in the diagnostics is therefore always False.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .. import _lib

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


@dataclass
class TritonTemporalLinearLIFResult:
    """Same fields as runtime/triton_temporal_linear_lif_backend.py:8-16."""

    spikes: torch.Tensor
    v_next: torch.Tensor
    used_triton: bool
    kernel_key: str = "temporal_linear_lif"
    fallback_reason: str = ""
    kernel_temporal_config: Optional[Dict] = None
    kernel_diagnostics: Optional[Dict] = None


def strict_temporal_linear_lif_enabled(strict: bool = False) -> bool:
    return bool(strict) or os.environ.get("CHRONOS_STRICT_TEMPORAL_LINEAR_LIF_TRITON", "0") == "1"


def _support_reasons(rank: int, T: int, M: int, Fin: int, dtype, device, weight, bias, v_init, tau) -> List[str]:
    reasons: List[str] = []
    if device.type != "cuda":
        reasons.append("unsupported_device: x_seq is not CUDA")
    if rank != 3:
        reasons.append(f"unsupported_rank: x_seq.dim must be 3, got {rank}")
    if dtype not in SUPPORTED_DTYPES:
        reasons.append(f"unsupported_dtype: x_seq dtype must be float32, bfloat16 or float16, got {dtype}")
    if T < 1:
        reasons.append(f"unsupported_temporal_length: T must be at least 1, got {T}")
    if not isinstance(weight, torch.Tensor):
        reasons.append("weight must be a tensor")
    elif weight.dim() != 2:
        reasons.append(f"unsupported_weight_rank: weight.dim must be 2, got {weight.dim()}")
    elif weight.device != device or weight.dtype != dtype:
        reasons.append(f"unsupported_dtype: weight device/dtype must match x_seq, got {weight.device}/{weight.dtype}")
    elif rank == 3 and int(weight.shape[1]) != Fin:
        reasons.append(f"unsupported_shape: weight in_features {int(weight.shape[1])} != x_seq {Fin}")
    if isinstance(bias, torch.Tensor) and bias.numel() > 0:
        if isinstance(weight, torch.Tensor) and weight.dim() == 2 and (bias.dim() != 1 or int(bias.shape[0]) != int(weight.shape[0])):
            reasons.append(f"unsupported_bias: bias shape {tuple(bias.shape)} does not match out_features")
        if bias.device != device or bias.dtype != dtype:
            reasons.append(f"unsupported_dtype: bias device/dtype must match x_seq, got {bias.device}/{bias.dtype}")
    if not isinstance(v_init, torch.Tensor):
        reasons.append("v_init must be a tensor")
    elif v_init.dim() != 0:
        if rank == 3 and isinstance(weight, torch.Tensor) and weight.dim() == 2:
            expected = (M, int(weight.shape[0]))
            if tuple(v_init.shape) != expected:
                reasons.append(f"unsupported_membrane_state: v_init shape {tuple(v_init.shape)} does not match {expected}")
        if v_init.device != device or v_init.dtype not in (dtype, torch.float32):
            reasons.append(
                f"unsupported_dtype: v_init device/dtype must match x_seq (or be float32), got {v_init.device}/{v_init.dtype}")
    if float(tau) == 0.0:
        reasons.append("unsupported_tau: tau must be nonzero")
    return reasons


def check_temporal_linear_lif_support(x_seq, weight, bias, v_init, v_threshold: float, v_reset: float, tau: float,
                                      detach_reset: bool) -> List[str]:
    """Counterpart of runtime/triton_temporal_linear_lif_backend.py:23-71 for a packed [T, M, Fin] input.

    Any T >= 1 is accepted, bfloat16 is accepted, and v_init may be float32 next to 16-bit activations.
    """
    if not isinstance(x_seq, torch.Tensor):
        return ["x_seq must be a tensor"]
    rank = x_seq.dim()
    T = int(x_seq.shape[0]) if rank >= 1 else 0
    M = int(x_seq.shape[1]) if rank == 3 else 0
    Fin = int(x_seq.shape[2]) if rank == 3 else 0
    return _support_reasons(rank, T, M, Fin, x_seq.dtype, x_seq.device, weight, bias, v_init, tau)


def _reject(reasons: List[str], strict: bool, verbose: bool) -> None:
    if not reasons:
        return
    if verbose:
        print(f"[HIP][FALLBACK][temporal_linear_lif] {'; '.join(reasons)}")
    if strict:
        raise RuntimeError("[HIP][STRICT][temporal_linear_lif] " + "; ".join(reasons))
    raise RuntimeError("; ".join(reasons))


def _run_steps(steps: List[torch.Tensor], weight, bias, v_init, v_threshold, v_reset, tau, spike_out, v_out,
               lead_shape) -> TritonTemporalLinearLIFResult:
    """`steps`: T tensors [M, Fin] with unit inner stride. Outputs are [T, M, Fout] / [M, Fout] (reshaped by caller)."""
    lib = _lib.lib()
    first = steps[0]
    T = len(steps)
    M, Fin = int(first.shape[0]), int(first.shape[1])
    Fout = int(weight.shape[0])
    v_dtype = _lib.membrane_dtype(first, v_init)
    row_stride = int(first.stride(0)) if M > 1 else Fin
    fixed = []
    for s in steps:
        ok = s.stride(1) == 1 and (M == 1 or int(s.stride(0)) == row_stride) and row_stride >= Fin
        fixed.append(s if ok else s.contiguous())
    if any(f is not s for f, s in zip(fixed, steps)):
        fixed = [s.contiguous() for s in steps]
        row_stride = Fin
    w = weight if weight.is_contiguous() else weight.contiguous()
    b = None
    if isinstance(bias, torch.Tensor) and bias.numel() > 0:
        b = bias if bias.is_contiguous() else bias.contiguous()
    vi = None
    if v_init.dim() != 0:
        vi = v_init.reshape(M, Fout)
        vi = vi if vi.is_contiguous() else vi.contiguous()
    if spike_out is None:
        spikes = torch.empty((T, M, Fout), dtype=first.dtype, device=first.device)
        v_next = torch.empty((M, Fout), dtype=v_dtype, device=first.device)
    else:
        # Same contract as kernels/generated_temporal_linear_lif_kernel.py:265-282.
        if tuple(spike_out.shape) != (T, M, Fout) or tuple(v_out.shape) != (M, Fout):
            raise RuntimeError(f"spike_out/v_out shapes {tuple(spike_out.shape)}/{tuple(v_out.shape)} do not match {(T, M, Fout)}/{(M, Fout)}")
        if spike_out.dtype != first.dtype or v_out.dtype != v_dtype or spike_out.device != first.device or v_out.device != first.device:
            raise RuntimeError("spike_out/v_out dtype or device mismatch")
        if not spike_out.is_contiguous() or not v_out.is_contiguous():
            raise RuntimeError("spike_out and v_out must be contiguous")
        spikes, v_next = spike_out, v_out
    workspace = _split_workspace(lib, first.device, T, M, Fin, Fout)
    # The library runs more than 16 timesteps as windows that hand the membrane over through `v_out`. A 16-bit membrane
    # would be rounded at every hand-over; the reference's kernel rounds once, after the last step. So such a call
    # computes with a float32 membrane and rounds the result.
    wide = v_dtype != torch.float32 and T > _lib.SNNF_MAX_T_PER_LAUNCH
    v_work = torch.empty((M, Fout), dtype=torch.float32, device=first.device) if wide else v_next
    if wide and vi is not None:
        vi = vi.float()
    _lib.check("snnf_linear_lif_ws", lib.snnf_linear_lif_ws(
        _lib.step_pointers(fixed), T, M, Fin, row_stride, _lib.dtype_code(first.dtype), w.data_ptr(), _lib.ptr(b), Fout,
        _lib.dtype_code(w.dtype), _lib.ptr(vi), _lib.dtype_code(v_work.dtype), spikes.data_ptr(), M * Fout,
        v_work.data_ptr(), float(v_threshold), float(v_reset), float(tau), _lib.ptr(workspace),
        0 if workspace is None else workspace.numel(), _lib.current_stream(first.device)))
    if wide:
        v_next.copy_(v_work)
    diagnostics = {
        "kernel_kind": "temporal_linear_lif",
        "compute_dtype": "float16" if first.dtype == torch.float16 else "float32",
        "matrix_operand_dtype": "float16" if first.dtype == torch.float16 else "bfloat16",
        "accumulator_dtype": "float32",
        "BLOCK_M": 16, "BLOCK_N": 16, "BLOCK_K": 32, "BTILE_T": min(T, 16), "REUSE_GROUPS": 1,
        "kernel_temporal_window": min(T, 16),
        "membrane_dtype": str(v_dtype),
        "spike_dtype": str(first.dtype),
        "stack_materialized": False,
        "flattened_leading_dims": lead_shape is not None,
    }
    if lead_shape is not None and spike_out is None:
        spikes = spikes.reshape((T,) + tuple(lead_shape) + (Fout,))
        v_next = v_next.reshape(tuple(lead_shape) + (Fout,))
    return TritonTemporalLinearLIFResult(spikes=spikes, v_next=v_next, used_triton=True,
                                         kernel_key="temporal_linear_lif", kernel_temporal_config=diagnostics,
                                         kernel_diagnostics=diagnostics)


# Workspaces that let the kernel split K over workgroups: one per (device, stream), zeroed when allocated (the kernel
# leaves its counters zero). A call under stream capture cannot allocate, and its stream exists only for the capture, so
# captured calls share one workspace per device that the eager calls before the capture (the warm-up every capture
# needs anyway) have prepared; without one they run unsplit. Graphs that share it must not replay concurrently.
# A captured graph holds the raw address of the workspace it was captured with, so a workspace that a larger layer
# outgrows is never handed back to the allocator: it moves to `_RETIRED_WORKSPACES` and lives as long as the process.
_WORKSPACES: Dict = {}
_RETIRED_WORKSPACES: list = []


def _split_workspace(lib, device, T: int, M: int, Fin: int, Fout: int):
    need = int(lib.snnf_linear_lif_workspace_bytes(T, M, Fin, Fout))
    if need == 0:
        return None
    capturing = torch.cuda.is_current_stream_capturing()
    graph_key = (device.index, "captured")
    key = graph_key if capturing else (device.index, int(torch.cuda.current_stream(device).cuda_stream))
    keys = (key,) if capturing else (key, graph_key)
    for k in keys:
        have = _WORKSPACES.get(k)
        if have is None or have.numel() < need:
            if capturing:
                return None
            if have is not None:
                _RETIRED_WORKSPACES.append(have)     # an earlier capture may still replay on it
            _WORKSPACES[k] = torch.zeros(need, dtype=torch.uint8, device=device)
    return _WORKSPACES[key]


def _run_packed(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset, strict, verbose,
                spike_out=None, v_out=None) -> TritonTemporalLinearLIFResult:
    lead_shape = None
    if isinstance(x_seq, torch.Tensor) and x_seq.dim() > 3:
        # Leading dims fold into rows (runtime/triton_temporal_linear_lif_backend.py:201-214).
        if not isinstance(weight, torch.Tensor) or weight.dim() != 2:
            raise RuntimeError("temporal Linear+LIF flatten path requires rank-2 weight")
        lead_shape = tuple(x_seq.shape[1:-1])
        x_seq = x_seq.contiguous().reshape(int(x_seq.shape[0]), -1, int(x_seq.shape[-1]))
        if isinstance(v_init, torch.Tensor) and v_init.dim() > 0:
            v_init = v_init.contiguous().reshape(-1, int(weight.shape[0]))
        if isinstance(spike_out, torch.Tensor):
            spike_out = spike_out.reshape(int(x_seq.shape[0]), -1, int(weight.shape[0]))
        if isinstance(v_out, torch.Tensor):
            v_out = v_out.reshape(-1, int(weight.shape[0]))
    strict = strict_temporal_linear_lif_enabled(strict)
    _reject(check_temporal_linear_lif_support(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset),
            strict, verbose)
    steps = [x_seq[t] for t in range(int(x_seq.shape[0]))]
    return _run_steps(steps, weight, bias, v_init, v_threshold, v_reset, tau, spike_out, v_out, lead_shape)


def run_triton_fused_temporal_linear_lif_state(xs, weight, bias, v_init, v_threshold: float, v_reset: float,
                                               tau: float, detach_reset: bool, strict: bool = False,
                                               verbose: bool = False,
                                               use_autotune: bool = True) -> TritonTemporalLinearLIFResult:
    """List form (runtime/triton_temporal_linear_lif_backend.py:74-118); a packed tensor is accepted too."""
    if isinstance(xs, torch.Tensor):
        return _run_packed(xs, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset, strict, verbose)
    if not isinstance(xs, (tuple, list)) or len(xs) == 0:
        raise RuntimeError("fused temporal linear LIF requires a non-empty Tensor list or [T,N,F] tensor")
    steps = list(xs)
    first = steps[0]
    strict = strict_temporal_linear_lif_enabled(strict)
    reasons: List[str] = []
    for index, x in enumerate(steps):
        if not isinstance(x, torch.Tensor):
            reasons.append(f"xs[{index}] is not a tensor")
        elif tuple(x.shape) != tuple(first.shape) or x.dtype != first.dtype or x.device != first.device:
            reasons.append(f"xs[{index}] shape/dtype/device differs from first tensor")
    if not reasons and first.dim() != 2:
        reasons.append(f"unsupported_rank: xs tensors must have rank 2, got {first.dim()}")
    _reject(reasons, strict, verbose)
    _reject(_support_reasons(3, len(steps), int(first.shape[0]), int(first.shape[1]), first.dtype, first.device,
                             weight, bias, v_init, tau), strict, verbose)
    return _run_steps(steps, weight, bias, v_init, v_threshold, v_reset, tau, None, None, None)


def run_triton_fused_temporal_linear_lif_state_packed(x_seq, weight, bias, v_init, v_threshold: float, v_reset: float,
                                                      tau: float, detach_reset: bool, strict: bool = False,
                                                      verbose: bool = False,
                                                      use_autotune: bool = True) -> TritonTemporalLinearLIFResult:
    """runtime/triton_temporal_linear_lif_backend.py:121-149."""
    return _run_packed(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset, strict, verbose)


def run_triton_fused_temporal_linear_lif_state_packed_out(x_seq, weight, bias, v_init, v_threshold: float,
                                                          v_reset: float, tau: float, detach_reset: bool, spike_out,
                                                          v_out, strict: bool = False, verbose: bool = False,
                                                          use_autotune: bool = True) -> TritonTemporalLinearLIFResult:
    """runtime/triton_temporal_linear_lif_backend.py:152-182."""
    return _run_packed(x_seq, weight, bias, v_init, v_threshold, v_reset, tau, detach_reset, strict, verbose,
                       spike_out=spike_out, v_out=v_out)
