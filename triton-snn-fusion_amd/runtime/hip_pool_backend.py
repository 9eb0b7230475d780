"""Pooling between fused operators on the HIP kernel `snnf_pool2d` (max 3x3/2, max 2x2/2, average 2x2/2).

The reference has no operator for this: pooling layers stay framework calls in its graphs. The fused executors use this
backend so that a whole forward stays on NCHW spike tensors without layout changes; anything the kernel does not
implement raises RuntimeError("unsupported_...") and the caller keeps the framework's pooling.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import _lib


def pool_config(module: nn.Module):
    """(is_max, kernel, stride, padding) when `module` is a pooling layer snnf_pool2d implements, else None."""
    def one(v):
        if isinstance(v, (tuple, list)):
            return int(v[0]) if len(set(v)) == 1 else None
        return int(v)

    if isinstance(module, nn.MaxPool2d):
        k, s, p = one(module.kernel_size), one(module.stride if module.stride is not None else module.kernel_size), one(module.padding)
        if None in (k, s, p) or module.ceil_mode or one(module.dilation) != 1 or module.return_indices:
            return None
        return (True, k, s, p) if (k, s) in ((3, 2), (2, 2)) and 2 * p <= k else None
    if isinstance(module, nn.AvgPool2d):
        k, s, p = one(module.kernel_size), one(module.stride if module.stride is not None else module.kernel_size), one(module.padding)
        if None in (k, s, p) or module.ceil_mode or module.divisor_override is not None:
            return None
        return (False, k, s, p) if (k, s, p) == (2, 2, 0) else None
    return None


def run_hip_pool2d(x: torch.Tensor, is_max: bool, kernel: int, stride: int, padding: int) -> torch.Tensor:
    """Pools the last two dimensions of a contiguous [..., H, W] tensor; returns [..., Ho, Wo] in the same dtype."""
    if not x.is_cuda or x.dtype not in (torch.float32, torch.bfloat16, torch.float16) or x.dim() < 3:
        raise RuntimeError("unsupported_device: snnf_pool2d needs an fp32 / bf16 / fp16 tensor [..., H, W] on the GPU")
    xc = x if x.is_contiguous() else x.contiguous()
    h, w = int(xc.shape[-2]), int(xc.shape[-1])
    ho, wo = (h + 2 * padding - kernel) // stride + 1, (w + 2 * padding - kernel) // stride + 1
    if ho < 1 or wo < 1:
        raise RuntimeError("unsupported_kernel: pooling window larger than the padded plane")
    planes = xc.numel() // (h * w)
    y = torch.empty(tuple(xc.shape[:-2]) + (ho, wo), dtype=xc.dtype, device=xc.device)
    _lib.check("snnf_pool2d", _lib.lib().snnf_pool2d(xc.data_ptr(), y.data_ptr(), planes, h, w, kernel, stride, padding,
                                                     1 if is_max else 0, _lib.dtype_code(xc.dtype), _lib.current_stream(xc.device)))
    return y
