"""ctypes binding of libsnnf.so (the C ABI declared in include/snnf.h).

The library is loaded from triton-snn-fusion_amd/lib/. If it has not been built the loader raises: there is no
Python or CPU substitute for the HIP kernels.
"""
from __future__ import annotations

import ctypes
from pathlib import Path
from typing import Optional, Sequence

import torch

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "lib" / "libsnnf.so"

SNNF_F32, SNNF_BF16, SNNF_F16 = 0, 1, 2
SNNF_LAYOUT_NCHW, SNNF_LAYOUT_C8, SNNF_LAYOUT_BITS = 0, 1, 2
SNNF_MAX_T_PER_LAUNCH = 16

_DTYPE_CODES = {torch.float32: SNNF_F32, torch.bfloat16: SNNF_BF16, torch.float16: SNNF_F16}

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float
_sz = ctypes.c_size_t
_pp = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes); must list every function declared in include/snnf.h.
SIGNATURES = {
    "snnf_abi_version": (_i, []),
    "snnf_status_string": (ctypes.c_char_p, [_i]),
    "snnf_last_error": (ctypes.c_char_p, []),
    "snnf_conv_last_plan": (ctypes.c_char_p, []),
    "snnf_lif_scan": (_i, [_pp, _i, _i64, _i, _vp, _i, _vp, _i64, _vp, _f, _f, _f, _vp]),
    "snnf_dwconv3x3_lif": (_i, [_pp, _pp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _i, _vp, _i64, _vp,
                                _f, _f, _f, _vp]),
    "snnf_dwconv3x3_lif_rowbits": (_i, [_pp, _pp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i64, _vp, _f, _f, _f, _vp]),
    "snnf_rowbits_unpack": (_i, [_vp, _vp, _i64, _i, _vp]),
    "snnf_rowbits_pack": (_i, [_vp, _vp, _i64, _i, _vp]),
    "snnf_pwconv_lif_rowbits": (_i, [_pp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i64, _vp, _f, _f, _f, _vp]),
    "snnf_lif_pool_linear_workspace_bytes": (_sz, [_i, _i]),
    "snnf_lif_pool_linear_launches": (_i, [_i, _i, _i, _i, _i, _i]),
    "snnf_lif_pool_linear": (_i, [_pp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _vp, _vp, _vp, _sz,
                                  _f, _f, _f, _vp]),
    "snnf_lif_pool_linear_static": (_i, [_pp, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _vp, _vp, _f, _f, _f, _vp]),
    "snnf_linear_lif": (_i, [_pp, _i, _i, _i, _i64, _i, _vp, _vp, _i, _i, _vp, _i, _vp, _i64, _vp, _f, _f, _f, _vp]),
    "snnf_linear_lif_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "snnf_linear_lif_ws": (_i, [_pp, _i, _i, _i, _i64, _i, _vp, _vp, _i, _i, _vp, _i, _vp, _i64, _vp, _f, _f, _f, _vp, _sz, _vp]),
    "snnf_conv_packed_weight_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "snnf_conv_pack_weight": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "snnf_conv_lif": (_i, [_pp, _pp, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _i64,
                           _vp, _f, _f, _f, _vp]),
    "snnf_layout_bytes": (_sz, [_i, _i64, _i, _i, _i, _i]),
    "snnf_layout_convert": (_i, [_vp, _i, _vp, _i, _i64, _i, _i, _i, _i, _vp]),
    "snnf_pool2d_blocked": (_i, [_vp, _i, _vp, _i, _i64, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "snnf_conv_blocked_tune": (_i, [_i] * 16),
    "snnf_conv_lif_blocked": (_i, [_pp, _i, _pp, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _i64,
                                   _vp, _i, _f, _f, _f, _vp]),
    "snnf_conv_lif_blocked_shortcut": (_i, [_pp, _pp, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                                            _vp, _vp, _i, _i64, _vp, _i, _f, _f, _f, _vp]),
    "snnf_conv_lif_blocked_avgpool": (_i, [_pp, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp, _f, _f, _f, _vp]),
    "snnf_spike_pool_linear": (_i, [_pp, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _vp, _f, _vp]),
    "snnf_linear_lif_bits": (_i, [_pp, _i, _i, _i, _i, _i64, _i, _vp, _vp, _i, _vp, _vp, _i64, _vp, _f, _f, _f, _vp, _sz, _vp]),
    "snnf_pool2d": (_i, [_vp, _vp, _i64, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "snnf_conv_bias": (_i, [_pp, _pp, _i, _i, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp]),
}

_LIB: Optional[ctypes.CDLL] = None


class SnnfError(RuntimeError):
    """A libsnnf entry point returned a non-zero status."""

    def __init__(self, func: str, status: int, detail: str):
        super().__init__(detail if detail else f"{func} failed with status {status}")
        self.func = func
        self.status = status


def library_available() -> bool:
    return LIB_PATH.exists()


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"libsnnf.so not found at {LIB_PATH}; build it with `python triton-snn-fusion_amd/build.py` "
                "(the fused SNN operators have no non-HIP implementation)"
            )
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here means header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = handle
    return _LIB


def membrane_dtype(x: torch.Tensor, v_init) -> torch.dtype:
    """dtype of the membrane an operator call returns. A `v_init` on the activations' device whose dtype is float32 or
    the activation dtype chooses it (a full-shape state to continue from, or a 0-dim zero placed there on purpose:
    16-bit activations with a float32 membrane); anything else - in particular the host-side 0-dim `torch.tensor(0.0)`
    placeholder the reference's rewriter emits (compiler/fx_lif_temporal_rewrite.py:2593) - gives the activation dtype,
    as in the reference (runtime/snn_custom_ops.py:378-381). Native kernels, eager functions and meta functions all
    use this one rule."""
    if (isinstance(v_init, torch.Tensor) and v_init.dtype in (torch.float32, x.dtype) and v_init.device == x.device):
        return v_init.dtype
    return x.dtype


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise RuntimeError(f"unsupported_dtype: libsnnf handles float32, bfloat16 and float16, got {dtype}") from None


def check(func: str, status: int) -> None:
    if status != 0:
        detail = lib().snnf_last_error().decode("utf-8", "replace")
        raise SnnfError(func, status, detail)


def step_pointers(tensors: Sequence[torch.Tensor]):
    """Host array of per-timestep device pointers."""
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def packed_step_pointers(x_seq: torch.Tensor):
    """Per-timestep pointers into a [T, ...] tensor whose steps are individually contiguous."""
    T = int(x_seq.shape[0])
    arr = (ctypes.c_void_p * T)()
    base = x_seq.data_ptr()
    step = int(x_seq.stride(0)) * x_seq.element_size()
    for t in range(T):
        arr[t] = base + t * step
    return arr


_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> ctypes.c_void_p:
    """The stream PyTorch would launch on for `device` right now, as a raw hipStream_t."""
    if _raw_current_stream is not None:     # the handle without a Stream object around it: a few microseconds per operator call
        index = device.index
        return ctypes.c_void_p(_raw_current_stream(torch.cuda.current_device() if index is None else index))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
