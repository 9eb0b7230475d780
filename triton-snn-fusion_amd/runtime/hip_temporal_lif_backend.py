"""Standalone temporal LIF backend on libsnnf: drop-in for the reference's runtime/triton_temporal_lif_backend.py.

`run_triton_fused_temporal_lif_state` keeps the reference's name and arguments and additionally accepts the
`use_autotune` keyword that the reference operator layer passes (runtime/snn_custom_ops.py:1623-1633) but the reference
backend does not accept.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from .. import _lib

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


@dataclass
class TritonTemporalLIFResult:
    """Same fields as runtime/triton_temporal_lif_backend.py:8-16."""

    spikes: torch.Tensor
    v_next: torch.Tensor
    used_triton: bool
    kernel_key: str = "temporal_lif"
    fallback_reason: str = ""
    kernel_temporal_config: Optional[Dict] = None
    kernel_diagnostics: Optional[Dict] = None


HipTemporalLIFResult = TritonTemporalLIFResult


def strict_temporal_lif_enabled(strict: bool = False) -> bool:
    return bool(strict) or os.environ.get("CHRONOS_STRICT_TEMPORAL_LIF_TRITON", "0") == "1"


def check_temporal_lif_support(x_seq, v_init, v_threshold: float, v_reset: float, tau: float,
                               detach_reset: bool) -> List[str]:
    """Counterpart of runtime/triton_temporal_lif_backend.py:23-54. Any T >= 1 and any rank >= 2 are accepted."""
    if not isinstance(x_seq, torch.Tensor):
        return ["x_seq must be a tensor"]
    reasons: List[str] = []
    if not x_seq.is_cuda:
        reasons.append("unsupported_device: x_seq is not CUDA")
    if x_seq.dim() != 5:
        reasons.append(f"unsupported_rank: x_seq.dim must be 5, got {x_seq.dim()}")
    if x_seq.dtype not in SUPPORTED_DTYPES:
        reasons.append(f"unsupported_dtype: x_seq dtype must be float32, bfloat16 or float16, got {x_seq.dtype}")
    if x_seq.dim() >= 1 and int(x_seq.shape[0]) < 1:
        reasons.append(f"unsupported_temporal_length: T must be at least 1, got {int(x_seq.shape[0])}")
    if not isinstance(v_init, torch.Tensor):
        reasons.append("v_init must be a tensor")
    elif v_init.dim() != 0:
        if x_seq.dim() == 5 and tuple(v_init.shape) != tuple(x_seq.shape[1:]):
            reasons.append(
                f"unsupported_membrane_state: v_init shape {tuple(v_init.shape)} does not match {tuple(x_seq.shape[1:])}")
        if v_init.device != x_seq.device or v_init.dtype not in (x_seq.dtype, torch.float32):
            reasons.append(
                f"unsupported_dtype: v_init device/dtype must match x_seq (or be float32), got {v_init.device}/{v_init.dtype}")
    if float(tau) == 0.0:
        reasons.append("unsupported_tau: tau must be nonzero")
    return reasons


def get_temporal_lif_best_config(T: int, total_elements: int, dtype: torch.dtype) -> Dict:
    """Launch shape of the scan kernel (counterpart of kernels/generated_temporal_lif_kernel.py's autotune record)."""
    vec = 16 // torch.empty((), dtype=dtype).element_size()
    return {"BLOCK_SIZE": 256 * vec, "elements_per_thread": vec, "T": int(T)}


def run_triton_fused_temporal_lif_state(x_seq, v_init, v_threshold: float, v_reset: float, tau: float,
                                        detach_reset: bool, strict: bool = False, verbose: bool = False,
                                        use_autotune: bool = True) -> TritonTemporalLIFResult:
    reasons = check_temporal_lif_support(x_seq, v_init, v_threshold, v_reset, tau, detach_reset)
    strict = strict_temporal_lif_enabled(strict)
    if reasons:
        if verbose:
            print(f"[HIP][FALLBACK][temporal_lif] {'; '.join(reasons)}")
        if strict:
            raise RuntimeError("[HIP][STRICT][temporal_lif] " + "; ".join(reasons))
        raise RuntimeError("; ".join(reasons))

    lib = _lib.lib()
    x = x_seq if x_seq.is_contiguous() else x_seq.contiguous()
    T = int(x.shape[0])
    numel = int(x[0].numel())
    v_dtype = _lib.membrane_dtype(x, v_init)
    vi = None
    if v_init.dim() != 0:
        vi = v_init if v_init.is_contiguous() else v_init.contiguous()
    spikes = torch.empty_like(x)
    v_next = torch.empty(x.shape[1:], dtype=v_dtype, device=x.device)
    # More than 16 steps run as windows that hand the membrane over through `v_out`; a 16-bit membrane would be rounded
    # at every hand-over, so such a call keeps it in float32 and rounds once at the end.
    wide = v_dtype != torch.float32 and T > _lib.SNNF_MAX_T_PER_LAUNCH
    v_work = torch.empty(x.shape[1:], dtype=torch.float32, device=x.device) if wide else v_next
    if wide and vi is not None:
        vi = vi.float()
    _lib.check("snnf_lif_scan", lib.snnf_lif_scan(
        _lib.packed_step_pointers(x), T, numel, _lib.dtype_code(x.dtype), _lib.ptr(vi), _lib.dtype_code(v_work.dtype),
        spikes.data_ptr(), numel, v_work.data_ptr(), float(v_threshold), float(v_reset), float(tau),
        _lib.current_stream(x.device)))
    if wide:
        v_next.copy_(v_work)
    config = get_temporal_lif_best_config(T=T, total_elements=numel, dtype=x.dtype)
    diagnostics = {
        "kernel_kind": "standalone_temporal_lif",
        "compute_dtype": "float16" if x.dtype == torch.float16 else "float32",
        "membrane_dtype": str(v_dtype),
        "spike_dtype": str(x.dtype),
        "T": T,
        "numel_per_step": numel,
        "kernel_temporal_config": config,
    }
    return TritonTemporalLIFResult(spikes=spikes, v_next=v_next, used_triton=True, kernel_key="temporal_lif",
                                   kernel_temporal_config=config, kernel_diagnostics=diagnostics)


def run_hip_lif_forward_state(x, v_prev, v_threshold: float, v_reset: float, tau: float):
    """One LIF step on a tensor of any rank (the single-step operator `lif_forward_state`, which the reference always
    evaluates with eager ops, runtime/snn_custom_ops.py:878-879): snnf_lif_scan with T = 1. A `v_prev` that is not a
    membrane of x's shape on x's device starts from zeros (runtime/snn_custom_ops.py:378-381). Returns (spikes, v_next);
    raises RuntimeError for tensors the kernel does not take."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype not in SUPPORTED_DTYPES or x.numel() == 0:
        raise RuntimeError("unsupported_device: lif_forward_state on the HIP kernels needs a non-empty fp32/bf16/fp16 GPU tensor")
    if float(tau) == 0.0:
        raise RuntimeError("unsupported_tau: tau must be nonzero")
    xc = x if x.is_contiguous() else x.contiguous()
    v_dtype = _lib.membrane_dtype(xc, v_prev)
    vi = None
    if (isinstance(v_prev, torch.Tensor) and v_prev.dim() != 0 and tuple(v_prev.shape) == tuple(x.shape)
            and v_prev.device == x.device and v_prev.dtype == v_dtype):
        vi = v_prev if v_prev.is_contiguous() else v_prev.contiguous()
    spikes = torch.empty_like(xc)
    v_next = torch.empty(xc.shape, dtype=v_dtype, device=x.device)
    numel = int(xc.numel())
    _lib.check("snnf_lif_scan", _lib.lib().snnf_lif_scan(
        _lib.step_pointers([xc]), 1, numel, _lib.dtype_code(x.dtype), _lib.ptr(vi), _lib.dtype_code(v_dtype),
        spikes.data_ptr(), numel, v_next.data_ptr(), float(v_threshold), float(v_reset), float(tau),
        _lib.current_stream(x.device)))
    return spikes, v_next
