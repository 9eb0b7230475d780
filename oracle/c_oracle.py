"""ctypes bindings for oracle/snn_oracle.c (brute-force C loops). TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path
from typing import Optional

import numpy as np

_DIR = Path(__file__).resolve().parent
LIB_PATH = _DIR / "_build" / "libsnn_oracle.so"
_LIB = None

_F = ctypes.POINTER(ctypes.c_float)


def build(force: bool = False) -> Path:
    if force or not LIB_PATH.exists():
        if force:
            subprocess.run(["make", "-C", str(_DIR), "clean"], check=True, capture_output=True)
        subprocess.run(["make", "-C", str(_DIR)], check=True, capture_output=True)
    return LIB_PATH


def lib():
    global _LIB
    if _LIB is None:
        build()
        _LIB = ctypes.CDLL(str(LIB_PATH))
        _LIB.oracle_lif_scan.argtypes = [_F, ctypes.c_int, ctypes.c_long, _F, ctypes.c_float, ctypes.c_float,
                                         ctypes.c_float, _F, _F, _F]
        _LIB.oracle_lif_scan.restype = None
        _LIB.oracle_conv2d.argtypes = [_F] + [ctypes.c_int] * 4 + [_F] + [ctypes.c_int] * 3 + [_F] + [ctypes.c_int] * 5 + [_F]
        _LIB.oracle_conv2d.restype = None
        _LIB.oracle_linear.argtypes = [_F, ctypes.c_int, ctypes.c_int, _F, ctypes.c_int, _F, _F]
        _LIB.oracle_linear.restype = None
        _LIB.oracle_avgpool_linear.argtypes = [_F, ctypes.c_int, ctypes.c_int, ctypes.c_int, _F, ctypes.c_int, _F, _F]
        _LIB.oracle_avgpool_linear.restype = None
    return _LIB


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(_F)


def _c(a) -> Optional[np.ndarray]:
    return None if a is None else np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def lif_scan(x_seq, v_init, v_threshold, v_reset, tau):
    x = _c(x_seq)
    T = x.shape[0]
    numel = int(np.prod(x.shape[1:]))
    vi = _c(v_init)
    spikes = np.empty_like(x)
    h = np.empty_like(x)
    v = np.empty(x.shape[1:], dtype=np.float32)
    lib().oracle_lif_scan(_p(x), T, numel, _p(vi), v_threshold, v_reset, tau, _p(spikes), _p(v), _p(h))
    return spikes, v, h


def conv2d(x, w, bias, stride, padding, groups=1):
    x, w, bias = _c(x), _c(w), _c(bias)
    N, Cin, H, W = x.shape
    Cout, _, KH, KW = w.shape
    Ho = (H + 2 * padding[0] - (KH - 1) - 1) // stride[0] + 1
    Wo = (W + 2 * padding[1] - (KW - 1) - 1) // stride[1] + 1
    out = np.empty((N, Cout, Ho, Wo), dtype=np.float32)
    lib().oracle_conv2d(_p(x), N, Cin, H, W, _p(w), Cout, KH, KW, _p(bias), stride[0], stride[1], padding[0],
                        padding[1], groups, _p(out))
    return out


def linear(x, w, bias):
    x, w, bias = _c(x), _c(w), _c(bias)
    out = np.empty((x.shape[0], w.shape[0]), dtype=np.float32)
    lib().oracle_linear(_p(x), x.shape[0], x.shape[1], _p(w), w.shape[0], _p(bias), _p(out))
    return out


def avgpool_linear(s, w, bias):
    s, w, bias = _c(s), _c(w), _c(bias)
    N, C = s.shape[:2]
    HW = int(np.prod(s.shape[2:]))
    out = np.empty((N, w.shape[0]), dtype=np.float32)
    lib().oracle_avgpool_linear(_p(s), N, C, HW, _p(w), w.shape[0], _p(bias), _p(out))
    return out
