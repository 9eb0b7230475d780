"""Conv (+BN folded) + LIF backend on libsnnf: drop-in for the reference's runtime/triton_convlif_backend.py.

Exports the names the reference operator layer imports (runtime/snn_custom_ops.py:9-18) with the same positional
arguments and keyword arguments (strict, verbose, use_autotune, compute_dtype): `check_triton_support`,
`classify_conv_lif_config`, `run_triton_fused_conv_lif_state`, `run_triton_fused_temporal_conv_lif_state`,
`run_triton_fused_temporal_pointwise_conv_lif_state`, `run_triton_fused_temporal_depthwise_conv_lif_state`,
`run_triton_fused_temporal_conv_lif_state_packed_out`, `run_triton_fused_temporal_conv_add_lif_state`. The "triton" in
the names is kept only so that the reference's import lines keep working; every call lands in a hand-written HIP kernel.

Differences from the reference backend, all supersets of it:
  * bfloat16 is accepted next to float32/float16, and the membrane (v_init / v_out) may be float32 while activations
    are 16 bit; the membrane dtype follows v_init.dtype (which equals x.dtype in everything the reference supports).
  * any LIF (v_threshold, v_reset, tau) is accepted, not only (1, 0, 2); any dense kernel/stride/padding with
    dilation 1 and 2*padding <= kernel is accepted, not only the six named kernel keys.
  * the T input tensors are consumed in place through per-timestep pointers: there is no torch.stack copy
    (runtime/triton_convlif_backend.py:579) and no membrane zero-fill / clone before the launch.
"""
from __future__ import annotations

import weakref
from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import _lib


@dataclass
class TritonConvLIFResult:
    """Same fields as runtime/triton_convlif_backend.py:7-15."""

    spikes: torch.Tensor
    v_next: torch.Tensor
    used_triton: bool
    kernel_key: str = "unsupported"
    fallback_reason: str = ""
    kernel_temporal_config: Optional[Dict] = None
    kernel_diagnostics: Optional[Dict] = None


HipConvLIFResult = TritonConvLIFResult

_NAMED_KEYS = {
    ((1, 1), (1, 1), (0, 0)): "k1_s1_p0",
    ((3, 3), (1, 1), (1, 1)): "k3_s1_p1",
    ((3, 3), (2, 2), (1, 1)): "k3_s2_p1",
    ((5, 5), (1, 1), (2, 2)): "k5_s1_p2",
    ((7, 7), (2, 2), (3, 3)): "k7_s2_p3",
    ((11, 11), (4, 4), (2, 2)): "k11_s4_p2",
}

# Same table as runtime/triton_convlif_backend.py:96-115 (the configurations the reference names explicitly).
SUPPORTED_CONV_LIF_CONFIGS = {
    (1, 1): {((1, 1), (0, 0)): "k1_s1_p0"},
    (3, 3): {
        ((1, 1), (1, 1)): "k3_s1_p1",
        ((2, 2), (1, 1)): "k3_s2_p1",
        ((1, 1), (1, 1), "depthwise"): "depthwise_k3_s1_p1",
        ((2, 2), (1, 1), "depthwise"): "depthwise_k3_s2_p1",
    },
    (5, 5): {((1, 1), (2, 2)): "k5_s1_p2"},
    (7, 7): {((2, 2), (3, 3)): "k7_s2_p3"},
    (11, 11): {((4, 4), (2, 2)): "k11_s4_p2"},
}

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)
MAX_TIMESTEPS_PER_LAUNCH = 4


def _as_pair(value) -> Tuple[int, int]:
    if isinstance(value, int):
        return value, value
    return int(value[0]), int(value[1])


def _conv2d_output_shape(x, weight, stride, padding, dilation) -> Tuple[int, int, int, int]:
    sh, sw = _as_pair(stride)
    ph, pw = _as_pair(padding)
    dh, dw = _as_pair(dilation)
    kh, kw = int(weight.shape[2]), int(weight.shape[3])
    ho = (int(x.shape[2]) + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    wo = (int(x.shape[3]) + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    return int(x.shape[0]), int(weight.shape[0]), ho, wo


def _is_depthwise_weight(weight, groups) -> bool:
    return int(groups) == int(weight.shape[0]) and int(weight.shape[1]) == 1 and int(groups) > 1


def classify_conv_lif_config(weight, stride, padding, dilation, groups) -> str:
    """Kernel key of a configuration (runtime/triton_convlif_backend.py:50-82), "unsupported" if no HIP kernel covers it.

    The six dense keys and two depthwise keys of the reference keep their names; other dense shapes the implicit-GEMM
    kernel covers get a key of the form k{kh}x{kw}_s{sh}x{sw}_p{ph}x{pw}.
    """
    if weight is None or not isinstance(weight, torch.Tensor) or weight.dim() != 4:
        return "unsupported"
    if tuple(_as_pair(dilation)) != (1, 1):
        return "unsupported"
    s, p = tuple(_as_pair(stride)), tuple(_as_pair(padding))
    k = (int(weight.shape[2]), int(weight.shape[3]))
    groups = int(groups)
    if groups == int(weight.shape[0]) and int(weight.shape[1]) == 1 and not (groups == 1):
        if k == (3, 3) and p == (1, 1) and s in ((1, 1), (2, 2)):
            return f"depthwise_k3_s{s[0]}_p1"
        return "unsupported"
    if groups != 1:
        return "unsupported"
    named = _NAMED_KEYS.get((k, s, p))
    if named is not None:
        return named
    if 2 * p[0] > k[0] or 2 * p[1] > k[1] or min(s) < 1:
        return "unsupported"
    return f"k{k[0]}x{k[1]}_s{s[0]}x{s[1]}_p{p[0]}x{p[1]}"


def classify_conv_lif_runtime_kind(weight, stride, padding, dilation, groups) -> str:
    key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    if key.startswith("depthwise_"):
        return "depthwise"
    if key == "k1_s1_p0":
        return "pointwise"
    return "regular" if key != "unsupported" else "unsupported"


def check_triton_support(x, weight, bias, v_prev, stride, padding, dilation, groups,
                         v_threshold, v_reset, tau, detach_reset) -> List[str]:
    """Reasons why the HIP path cannot take this call (empty list = supported).

    Counterpart of runtime/triton_convlif_backend.py:118-211; reason strings keep the `unsupported_*:` prefixes that the
    operator layer turns into statistics keys.
    """
    reasons: List[str] = []
    if not x.is_cuda:
        reasons.append("unsupported_device: x is not CUDA")
    if bias is None:
        reasons.append("missing_or_unsupported_bias: bias must be a Tensor")
    if x.dtype not in SUPPORTED_DTYPES:
        reasons.append(f"unsupported_dtype: x dtype must be float32, bfloat16 or float16, got {x.dtype}")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        reasons.append(
            "unsupported_dtype: x/weight/bias dtypes must match, got "
            f"x={x.dtype}, weight={weight.dtype}, bias={getattr(bias, 'dtype', None)}"
        )
    if isinstance(v_prev, torch.Tensor) and v_prev.dtype not in (x.dtype, torch.float32):
        reasons.append(f"unsupported_dtype: v_prev dtype must be x dtype or float32, got v_prev={v_prev.dtype}, x={x.dtype}")
    if x.dim() != 4:
        reasons.append(f"unsupported_rank: x.dim must be 4, got {x.dim()}")
    if weight.dim() != 4:
        reasons.append(f"unsupported_rank: weight.dim must be 4, got {weight.dim()}")
    if x.dim() != 4 or weight.dim() != 4:
        return reasons
    groups = int(groups)
    depthwise = int(weight.shape[1]) == 1 and groups == int(x.shape[1]) == int(weight.shape[0]) and groups > 1
    if groups != 1 and not depthwise:
        reasons.append(f"unsupported_groups: groups must be 1 or depthwise, got {groups}")
    if groups == 1 and int(weight.shape[1]) != int(x.shape[1]):
        reasons.append(f"unsupported_shape: weight in_channels {int(weight.shape[1])} != x channels {int(x.shape[1])}")
    if tuple(_as_pair(dilation)) != (1, 1):
        reasons.append(f"unsupported_dilation: dilation must be (1, 1), got {tuple(_as_pair(dilation))}")
    s, p = tuple(_as_pair(stride)), tuple(_as_pair(padding))
    k = (int(weight.shape[2]), int(weight.shape[3]))
    if depthwise:
        if k != (3, 3):
            reasons.append(f"unsupported_kernel: depthwise kernel must be (3, 3), got {k}")
        elif s not in ((1, 1), (2, 2)):
            reasons.append(f"unsupported_stride: 3x3 depthwise kernel supports stride [(1, 1), (2, 2)], got {s}")
        elif p != (1, 1):
            reasons.append(f"unsupported_padding: 3x3 depthwise kernel supports padding [(1, 1)], got {p}")
    elif groups == 1:
        if 2 * p[0] > k[0] or 2 * p[1] > k[1]:
            reasons.append(f"unsupported_padding: {k[0]}x{k[1]} kernel supports padding up to half the kernel, got {p}")
        if int(x.shape[2]) + 2 * p[0] < k[0] or int(x.shape[3]) + 2 * p[1] < k[1]:
            reasons.append(f"unsupported_kernel: kernel {k} larger than padded input {tuple(x.shape[2:])}")
    if float(tau) == 0.0:
        reasons.append("unsupported_tau: tau must be nonzero")
    if isinstance(v_prev, torch.Tensor) and v_prev.dim() != 0:
        out_shape = _conv2d_output_shape(x, weight, stride, padding, dilation)
        if tuple(v_prev.shape) != tuple(out_shape):
            reasons.append(f"v_prev shape {tuple(v_prev.shape)} does not match conv output shape {out_shape}")
    return reasons


def _unsupported(reasons: List[str], strict: bool, verbose: bool) -> None:
    if reasons and verbose:
        print(f"[HIP][FALLBACK] {'; '.join(reasons)}")
    if reasons and strict:
        raise RuntimeError("[HIP][STRICT] " + "; ".join(reasons))


def _validate_temporal_conv_kind(kind: str, kernel_key: str) -> None:
    # The depthwise / pointwise operators insist on their own kernel family (runtime/triton_convlif_backend.py:285-293);
    # the regular operator takes any dense kernel here.
    if kind == "pointwise" and kernel_key != "k1_s1_p0":
        raise RuntimeError(f"pointwise conv op requires k1_s1_p0 kernel, got {kernel_key}")
    if kind == "depthwise" and not kernel_key.startswith("depthwise_"):
        raise RuntimeError(f"depthwise conv op requires depthwise kernel, got {kernel_key}")
    if kind == "regular" and kernel_key.startswith("depthwise_"):
        raise RuntimeError(f"regular conv op cannot dispatch depthwise kernel {kernel_key}")


def _compute_dtype_name(dtype: torch.dtype) -> str:
    return "float16" if dtype == torch.float16 else "float32"


def _check_compute_dtype(compute_dtype, dtype: torch.dtype) -> None:
    expected = _compute_dtype_name(dtype)
    if compute_dtype is not None and compute_dtype != expected:
        raise RuntimeError(f"compute_dtype={compute_dtype} does not match input dtype path {expected}")


def kernel_dtype_diagnostics(dtype: torch.dtype) -> Dict:
    """Counterpart of kernels/benchmark_conv_lif_temporal_general.py:264-293 for the HIP kernels."""
    operand = "float16" if dtype == torch.float16 else "bfloat16"
    if dtype == torch.float32:
        # fp32 tensors: value = hi + lo with both terms bf16; w_hi x_hi + w_lo x_hi + w_hi x_lo accumulated in fp32
        operand = "bfloat16 hi + lo terms (3 products per fp32 product)"
    return {
        "compute_dtype": _compute_dtype_name(dtype),
        "matrix_operand_dtype": operand,
        "accumulator_dtype": "float32",
        "membrane_dtype": "float32 (on chip)",
        "tf32_enabled": False,
        "tensor_core_usage_mode": f"mfma_f32_32x32x16_{'f16' if dtype == torch.float16 else 'bf16'}",
        "stack_materialized": False,
    }


def get_autotune_best_config(kernel_key: str, residual_add: bool = False, T: int = MAX_TIMESTEPS_PER_LAUNCH) -> Dict:
    """Shape of kernels/benchmark_conv_lif_temporal_general.py:1332-1369: the temporal schedule a launch uses.

    The HIP kernels have a fixed schedule: up to 4 timesteps are accumulated side by side against one weight fragment
    load (the role of BTILE_T), with no extra accumulator groups.
    """
    window = max(1, min(int(T), MAX_TIMESTEPS_PER_LAUNCH))
    if kernel_key.startswith("depthwise_"):
        return {"BTILE_T": 1, "REUSE_GROUPS": 1, "kernel_temporal_window": int(T), "residual_add": bool(residual_add)}
    return {"BTILE_T": window, "REUSE_GROUPS": 1, "kernel_temporal_window": window, "residual_add": bool(residual_add)}


def last_conv_plan() -> Dict:
    """What the planner selected for this thread's most recent matrix-core convolution launch (snnf_conv_last_plan):
    kernel family, timesteps per launch, tile and wave decomposition, LDS bytes and grid, as a dict."""
    text = _lib.lib().snnf_conv_last_plan().decode("ascii", "replace")
    plan: Dict = {}
    for item in text.split():
        key, _, value = item.partition("=")
        plan[key] = int(value) if value.lstrip("-").isdigit() else value
    return plan


# The temporal configuration of a launch depends only on the layer (shapes, dtypes, window); the planner's answer is read
# back and parsed once per distinct layer.
_TEMPORAL_CONFIGS: Dict[tuple, Dict] = {}


def _planned_temporal_config(kernel_key: str, residual_add: bool, T: int, memo: Optional[tuple] = None) -> Dict:
    if memo is not None:
        known = _TEMPORAL_CONFIGS.get(memo)
        if known is not None:
            return dict(known)
    config = _read_planned_temporal_config(kernel_key, residual_add, T)
    if memo is not None and len(_TEMPORAL_CONFIGS) < 4096:
        _TEMPORAL_CONFIGS[memo] = dict(config)
    return config


def _read_planned_temporal_config(kernel_key: str, residual_add: bool, T: int) -> Dict:
    config = get_autotune_best_config(kernel_key, residual_add=residual_add, T=T)
    if kernel_key.startswith("depthwise_"):
        return config
    plan = last_conv_plan()
    if plan:
        variant = int(plan.get("variant", 0))
        # Timesteps accumulated side by side against one weight fragment load: the matrix kernels encode it in the
        # variant number (10 + n general, 20 + n fast, 30 + n fast with 4-wave workgroups), the 4-wave T-in-M kernel uses the variant itself, the time-outer and
        # pointwise kernels take one step at a time with the weights resident.
        side_by_side = variant % 10 if variant >= 10 else max(1, variant)
        config.update({"BTILE_T": side_by_side, "kernel_temporal_window": int(plan.get("window", config["kernel_temporal_window"])),
                       "plan": plan})
    return config


# ---------------------------------------------------------------------------------------------------------------
# Packed-weight cache: the implicit-GEMM kernel reads weights in matrix-core fragment order; the repack runs once per
# (weight tensor object, version) and is reused by every later call with the same tensors.
# ---------------------------------------------------------------------------------------------------------------
_PACK_CACHE: "OrderedDict[tuple, tuple]" = OrderedDict()
_PACK_CACHE_LIMIT = 512


def clear_packed_weight_cache() -> None:
    _PACK_CACHE.clear()


def _packed_weight(weight: torch.Tensor, bias: Optional[torch.Tensor], x_dtype: torch.dtype) -> torch.Tensor:
    key = (id(weight), id(bias), x_dtype)
    hit = _PACK_CACHE.get(key)
    if hit is not None:
        w_ref, b_ref, w_ver, b_ver, w_ptr, b_ptr, packed = hit
        if (w_ref() is weight and (bias is None or b_ref() is bias) and w_ver == weight._version
                and (bias is None or b_ver == bias._version) and w_ptr == weight.data_ptr()
                and (bias is None or b_ptr == bias.data_ptr())):
            _PACK_CACHE.move_to_end(key)
            return packed
        del _PACK_CACHE[key]
    lib = _lib.lib()
    cout, cin, kh, kw = (int(d) for d in weight.shape)
    w = weight if weight.is_contiguous() else weight.contiguous()
    b = None if bias is None else (bias if bias.is_contiguous() else bias.contiguous())
    nbytes = int(lib.snnf_conv_packed_weight_bytes(cout, cin, kh, kw, _lib.dtype_code(x_dtype)))
    packed = torch.empty(nbytes, dtype=torch.uint8, device=weight.device)
    _lib.check("snnf_conv_pack_weight", lib.snnf_conv_pack_weight(
        w.data_ptr(), _lib.ptr(b), _lib.dtype_code(weight.dtype), cout, cin, kh, kw, _lib.dtype_code(x_dtype),
        packed.data_ptr(), nbytes, _lib.current_stream(weight.device)))
    _PACK_CACHE[key] = (weakref.ref(weight), weakref.ref(bias) if bias is not None else None, weight._version,
                        None if bias is None else bias._version, weight.data_ptr(),
                        None if bias is None else bias.data_ptr(), packed)
    while len(_PACK_CACHE) > _PACK_CACHE_LIMIT:
        _PACK_CACHE.popitem(last=False)
    return packed


def _membrane_dtype(x: torch.Tensor, v_init) -> torch.dtype:
    return _lib.membrane_dtype(x, v_init)


def _v_init_pointer(v_init, out_shape, v_dtype, device):
    """None for a zero membrane (0-dim v_init), else a contiguous tensor of the output shape."""
    if not isinstance(v_init, torch.Tensor) or v_init.dim() == 0:
        return None
    if tuple(v_init.shape) != tuple(out_shape):
        raise RuntimeError(f"unsupported_membrane_state: v_init shape {tuple(v_init.shape)} does not match {tuple(out_shape)}")
    if v_init.dtype != v_dtype or v_init.device != device:
        raise RuntimeError(f"unsupported_dtype: v_init device/dtype must be {device}/{v_dtype}, got {v_init.device}/{v_init.dtype}")
    return v_init if v_init.is_contiguous() else v_init.contiguous()


def _launch(kernel_key: str, steps: Sequence[torch.Tensor], residuals: Optional[Sequence[torch.Tensor]], weight, bias,
            v_init, stride, padding, v_threshold, v_reset, tau, spikes: torch.Tensor, v_out: torch.Tensor) -> None:
    """Enqueues the HIP kernel(s) for one fused conv+LIF call. `steps` are T contiguous [N, C, H, W] tensors."""
    lib = _lib.lib()
    first = steps[0]
    T = len(steps)
    n, cin, h, w = (int(d) for d in first.shape)
    cout, _, kh, kw = (int(d) for d in weight.shape)
    sh, sw = _as_pair(stride)
    ph, pw = _as_pair(padding)
    xs = _lib.step_pointers(steps)
    rs = _lib.step_pointers(residuals) if residuals is not None else None
    x_code = _lib.dtype_code(first.dtype)
    v_code = _lib.dtype_code(v_out.dtype)
    vi = _v_init_pointer(v_init, v_out.shape, v_out.dtype, first.device)
    stream = _lib.current_stream(first.device)
    step_stride = int(spikes.stride(0)) if spikes.dim() == 5 else int(spikes.numel() // T)
    if kernel_key.startswith("depthwise_"):
        wc = weight if weight.is_contiguous() else weight.contiguous()
        bc = bias if bias.is_contiguous() else bias.contiguous()
        _lib.check("snnf_dwconv3x3_lif", lib.snnf_dwconv3x3_lif(
            xs, rs, T, n, cin, h, w, sh, x_code, wc.data_ptr(), bc.data_ptr(), _lib.dtype_code(weight.dtype),
            _lib.ptr(vi), v_code, spikes.data_ptr(), step_stride, v_out.data_ptr(),
            float(v_threshold), float(v_reset), float(tau), stream))
    else:
        packed = _packed_weight(weight, bias, first.dtype)
        _lib.check("snnf_conv_lif", lib.snnf_conv_lif(
            xs, rs, T, n, cin, h, w, x_code, packed.data_ptr(), cout, kh, kw, sh, sw, ph, pw,
            _lib.ptr(vi), v_code, spikes.data_ptr(), step_stride, v_out.data_ptr(),
            float(v_threshold), float(v_reset), float(tau), stream))


def run_hip_temporal_conv_bias(xs: Sequence[torch.Tensor], weight, bias, stride, padding,
                               residuals: Optional[Sequence[torch.Tensor]] = None) -> torch.Tensor:
    """Neuron-free convolution + bias (+ residual) of T independent frames on the matrix kernel (snnf_conv_bias):
    returns [T, N, Cout, Ho, Wo] in the activation dtype. For the LIF-free Conv+BN layers between fused operators
    (ResNet shortcuts, whose output feeds `fused_temporal_conv_add_lif_state` as `residuals`); the reference leaves
    those to the framework's convolution. Raises RuntimeError("unsupported_...") for layers the kernel does not take."""
    steps = _contiguous_steps(xs)
    first = steps[0]
    if not first.is_cuda or first.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise RuntimeError("unsupported_device: snnf_conv_bias needs fp32 / bf16 / fp16 tensors on the GPU")
    if any(s.shape != first.shape or s.dtype != first.dtype for s in steps):
        raise RuntimeError("unsupported_shape: frames must share shape and dtype")
    T = len(steps)
    n, cin, h, w = (int(d) for d in first.shape)
    cout, wcin, kh, kw = (int(d) for d in weight.shape)
    if wcin != cin:
        raise RuntimeError(f"unsupported_groups: weight has {wcin} input channels, frames have {cin}")
    sh, sw = _as_pair(stride)
    ph, pw = _as_pair(padding)
    ho, wo = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
    res = None
    if residuals is not None:
        res = _contiguous_steps(residuals)
        if len(res) != T or any(tuple(r.shape) != (n, cout, ho, wo) or r.dtype != first.dtype for r in res):
            raise RuntimeError("unsupported_residual_shape: residuals must be T tensors of the output shape and dtype")
    if bias is None:
        bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    out = torch.empty((T, n, cout, ho, wo), dtype=first.dtype, device=first.device)
    packed = _packed_weight(weight, bias, first.dtype)
    _lib.check("snnf_conv_bias", _lib.lib().snnf_conv_bias(
        _lib.step_pointers(steps), _lib.step_pointers(res) if res is not None else None, T, n, cin, h, w,
        _lib.dtype_code(first.dtype), packed.data_ptr(), cout, kh, kw, sh, sw, ph, pw,
        out.data_ptr(), int(out.stride(0)), _lib.current_stream(first.device)))
    return out


def _contiguous_steps(xs: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    return [x if x.is_contiguous() else x.contiguous() for x in xs]


def _validate_step_list(xs, name: str = "xs") -> List[str]:
    reasons: List[str] = []
    if not isinstance(xs, (list, tuple)) or len(xs) == 0:
        return [f"{name} must be a non-empty list/tuple of tensors"]
    first = xs[0]
    for index, x in enumerate(xs):
        if not isinstance(x, torch.Tensor):
            reasons.append(f"{name}[{index}] is not a tensor")
            continue
        if tuple(x.shape) != tuple(first.shape):
            reasons.append(f"{name}[{index}] shape {tuple(x.shape)} differs from first shape {tuple(first.shape)}")
        if x.device != first.device or x.dtype != first.dtype:
            reasons.append(f"{name}[{index}] device/dtype differs from first tensor")
    return reasons


def _raise_if(reasons: List[str], strict: bool, verbose: bool) -> None:
    if reasons:
        _unsupported(reasons, strict=strict, verbose=verbose)
        raise RuntimeError("; ".join(reasons))


def _run_temporal(kind: str, xs, residuals, weight, bias, v_init, stride, padding, dilation, groups,
                  v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype,
                  spike_out=None, v_out=None) -> TritonConvLIFResult:
    first = xs[0]
    _raise_if(check_triton_support(first, weight, bias, v_init, stride, padding, dilation, groups,
                                   v_threshold, v_reset, tau, detach_reset), strict, verbose)
    _check_compute_dtype(compute_dtype, first.dtype)
    kernel_key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    if kernel_key == "unsupported":
        raise RuntimeError("unsupported dispatch key after support check")
    _validate_temporal_conv_kind(kind, kernel_key)
    if verbose:
        print(f"[CHRONOS_DISPATCH] op={kind} backend={kernel_key} x_shape={(len(xs),) + tuple(first.shape)} "
              f"w_shape={tuple(weight.shape)} stride={tuple(_as_pair(stride))} padding={tuple(_as_pair(padding))} "
              f"groups={int(groups)}")
    T = len(xs)
    out_shape = _conv2d_output_shape(first, weight, stride, padding, dilation)
    v_dtype = _membrane_dtype(first, v_init)
    if spike_out is None:
        spikes = torch.empty((T,) + tuple(out_shape), dtype=first.dtype, device=first.device)
        v_next = torch.empty(out_shape, dtype=v_dtype, device=first.device)
    else:
        _check_output_buffers(spike_out, v_out, (T,) + tuple(out_shape), out_shape, first, v_dtype)
        spikes, v_next = spike_out, v_out
    steps = _contiguous_steps(xs)
    res = _contiguous_steps(residuals) if residuals is not None else None
    memo = (kernel_key, residuals is not None, T, first.shape, weight.shape, tuple(_as_pair(stride)), tuple(_as_pair(padding)),
            first.dtype, v_dtype, isinstance(v_init, torch.Tensor) and v_init.dim() > 0)
    # A call of more timesteps than one launch takes hands the membrane from launch to launch through `v_out`. A 16-bit
    # membrane would be rounded at every hand-over, where the reference's kernel rounds once after the last step
    # (kernels/benchmark_conv_lif_temporal_general.py:707-716). How many launches the matrix kernels take depends on the
    # membrane dtype itself (their one-launch variant needs a float32 membrane), so every multi-step call with a 16-bit
    # membrane computes with a float32 working membrane and rounds the result once: the same arithmetic on every call.
    wide = v_dtype != torch.float32 and T > 1 and _takes_several_launches(kernel_key, T)
    v_work = torch.empty(out_shape, dtype=torch.float32, device=first.device) if wide else v_next
    if wide and isinstance(v_init, torch.Tensor) and v_init.dim() > 0:
        v_init = v_init.float()
    _launch(kernel_key, steps, res, weight, bias, v_init, stride, padding, v_threshold, v_reset, tau, spikes, v_work)
    if wide:
        v_next.copy_(v_work)
    diagnostics = kernel_dtype_diagnostics(first.dtype)
    if residuals is not None:
        diagnostics["residual_add"] = True
        diagnostics["kernel_kind"] = "temporal_residual"
    return TritonConvLIFResult(
        spikes, v_next, True, kernel_key=kernel_key,
        kernel_temporal_config=_planned_temporal_config(kernel_key, residuals is not None, T, memo),
        kernel_diagnostics=diagnostics,
    )


def _takes_several_launches(kernel_key: str, T: int) -> bool:
    if kernel_key.startswith("depthwise_"):
        return T > _lib.SNNF_MAX_T_PER_LAUNCH     # the depthwise kernel holds up to 16 steps per launch
    return True                                   # matrix kernels: windows of 2 or 4 steps, chosen per membrane dtype


def _check_output_buffers(spike_out, v_out, spike_shape, v_shape, like: torch.Tensor, v_dtype) -> None:
    # Same contract as kernels/benchmark_conv_lif_temporal_general.py:458-477.
    if tuple(spike_out.shape) != tuple(spike_shape):
        raise RuntimeError(f"spike_out shape {tuple(spike_out.shape)} does not match {tuple(spike_shape)}")
    if tuple(v_out.shape) != tuple(v_shape):
        raise RuntimeError(f"v_out shape {tuple(v_out.shape)} does not match {tuple(v_shape)}")
    if spike_out.dtype != like.dtype or spike_out.device != like.device:
        raise RuntimeError("spike_out dtype/device must match the input")
    if v_out.dtype != v_dtype or v_out.device != like.device:
        raise RuntimeError(f"v_out dtype/device must be {v_dtype}/{like.device}")
    if not spike_out.is_contiguous() or not v_out.is_contiguous():
        raise RuntimeError("spike_out and v_out must be contiguous")


def run_triton_fused_conv_lif_state(x, weight, bias, v_prev, stride: Sequence[int], padding: Sequence[int],
                                    dilation: Sequence[int], groups: int, v_threshold: float, v_reset: float,
                                    tau: float, detach_reset: bool, strict: bool = False, verbose: bool = False,
                                    use_autotune: bool = True, compute_dtype: str = None) -> TritonConvLIFResult:
    """Single-step conv + LIF = the temporal kernel with T = 1 (runtime/triton_convlif_backend.py:331-390)."""
    _raise_if(check_triton_support(x, weight, bias, v_prev, stride, padding, dilation, groups,
                                   v_threshold, v_reset, tau, detach_reset), strict, verbose)
    kernel_key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    kind = "depthwise" if kernel_key.startswith("depthwise_") else ("pointwise" if kernel_key == "k1_s1_p0" else "regular")
    result = _run_temporal(kind, [x], None, weight, bias, v_prev, stride, padding, dilation, groups,
                           v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype)
    result.spikes = result.spikes[0]
    return result


def _run_kind(kind, xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset, tau,
              detach_reset, strict, verbose, compute_dtype) -> TritonConvLIFResult:
    _raise_if(_validate_step_list(xs), strict, verbose)
    return _run_temporal(kind, list(xs), None, weight, bias, v_init, stride, padding, dilation, groups,
                         v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype)


def run_triton_fused_temporal_conv_lif_state(xs, weight, bias, v_init, stride, padding, dilation, groups: int,
                                             v_threshold: float, v_reset: float, tau: float, detach_reset: bool,
                                             strict: bool = False, verbose: bool = False, use_autotune: bool = True,
                                             compute_dtype: str = None) -> TritonConvLIFResult:
    """runtime/triton_convlif_backend.py:393-430. Also takes 1x1 and depthwise weights (routed to their kernels)."""
    _raise_if(_validate_step_list(xs), strict, verbose)
    key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    kind = "depthwise" if key.startswith("depthwise_") else ("pointwise" if key == "k1_s1_p0" else "regular")
    return _run_temporal(kind, list(xs), None, weight, bias, v_init, stride, padding, dilation, groups,
                         v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype)


def run_triton_fused_temporal_pointwise_conv_lif_state(xs, weight, bias, v_init, stride, padding, dilation,
                                                       groups: int, v_threshold: float, v_reset: float, tau: float,
                                                       detach_reset: bool, strict: bool = False, verbose: bool = False,
                                                       use_autotune: bool = True,
                                                       compute_dtype: str = None) -> TritonConvLIFResult:
    """runtime/triton_convlif_backend.py:433-470."""
    return _run_kind("pointwise", xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset,
                     tau, detach_reset, strict, verbose, compute_dtype)


def run_triton_fused_temporal_depthwise_conv_lif_state(xs, weight, bias, v_init, stride, padding, dilation,
                                                       groups: int, v_threshold: float, v_reset: float, tau: float,
                                                       detach_reset: bool, strict: bool = False, verbose: bool = False,
                                                       use_autotune: bool = True,
                                                       compute_dtype: str = None) -> TritonConvLIFResult:
    """runtime/triton_convlif_backend.py:473-510."""
    return _run_kind("depthwise", xs, weight, bias, v_init, stride, padding, dilation, groups, v_threshold, v_reset,
                     tau, detach_reset, strict, verbose, compute_dtype)


def run_triton_fused_temporal_conv_lif_state_packed_out(x_seq, weight, bias, v_init, stride, padding, dilation,
                                                        groups: int, v_threshold: float, v_reset: float, tau: float,
                                                        detach_reset: bool, spike_out, v_out, strict: bool = False,
                                                        verbose: bool = False, use_autotune: bool = True,
                                                        compute_dtype: str = None) -> TritonConvLIFResult:
    """Packed [T, N, C, H, W] input, caller-owned outputs (runtime/triton_convlif_backend.py:601-686)."""
    reasons: List[str] = []
    if not isinstance(x_seq, torch.Tensor):
        reasons.append("x_seq must be a tensor")
    elif x_seq.dim() != 5:
        reasons.append(f"x_seq must have rank 5 [T,N,C,H,W], got {x_seq.dim()}")
    elif not x_seq.is_contiguous():
        reasons.append("x_seq must be contiguous; create the packed stack in FX before calling the out op")
    if not isinstance(spike_out, torch.Tensor) or not isinstance(v_out, torch.Tensor):
        reasons.append("spike_out and v_out must be tensors")
    _raise_if(reasons, strict, verbose)
    steps = [x_seq[t] for t in range(int(x_seq.shape[0]))]
    key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    kind = "depthwise" if key.startswith("depthwise_") else ("pointwise" if key == "k1_s1_p0" else "regular")
    return _run_temporal(kind, steps, None, weight, bias, v_init, stride, padding, dilation, groups,
                         v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype,
                         spike_out=spike_out, v_out=v_out)


def run_triton_fused_temporal_conv_add_lif_state(xs, residuals, weight, bias, v_init, stride, padding, dilation,
                                                 groups: int, v_threshold: float, v_reset: float, tau: float,
                                                 detach_reset: bool, strict: bool = False, verbose: bool = False,
                                                 use_autotune: bool = True,
                                                 compute_dtype: str = None) -> TritonConvLIFResult:
    """conv + residual add + LIF (runtime/triton_convlif_backend.py:689-817); residuals are consumed in place."""
    reasons = _validate_step_list(xs)
    reasons += _validate_step_list(residuals, "residuals")
    if not reasons and len(xs) != len(residuals):
        reasons.append(f"xs and residuals length mismatch: {len(xs)} vs {len(residuals)}")
    if not reasons:
        first = xs[0]
        out_shape = _conv2d_output_shape(first, weight, stride, padding, dilation)
        for index, residual in enumerate(residuals):
            if tuple(residual.shape) != tuple(out_shape):
                reasons.append(f"residuals[{index}] shape {tuple(residual.shape)} does not match conv output shape {out_shape}")
            if residual.device != first.device or residual.dtype != first.dtype:
                reasons.append(f"residuals[{index}] device/dtype differs from first tensor")
    _raise_if(reasons, strict, verbose)
    key = classify_conv_lif_config(weight, stride, padding, dilation, groups)
    kind = "depthwise" if key.startswith("depthwise_") else ("pointwise" if key == "k1_s1_p0" else "regular")
    return _run_temporal(kind, list(xs), list(residuals), weight, bias, v_init, stride, padding, dilation, groups,
                         v_threshold, v_reset, tau, detach_reset, strict, verbose, compute_dtype)
