"""Internal activation layouts between consecutive fused operators of one network, on libsnnf.

The reference hands dense [T, N, C, H, W] tensors of 0/1 elements from one fused operator to the next
(kernels/benchmark_conv_lif_temporal_general.py:707-708), stacks a layer's T inputs into one tensor
(runtime/triton_convlif_backend.py:579) and, in its executor's fast path, writes into pooled caller-owned buffers
(runtime/fx_standalone_executor.py:900-952). This module is the counterpart of that producer-consumer plumbing for a
network executor that owns both ends of a tensor: spikes travel at one bit each (`BITS`: [T, N, ceil(C/8), H, W] bytes,
bit j = channel 8*c8 + j), analog activations channel-blocked (`C8`: [T, N, ceil(C/8), H, W, 8] elements), which is the
operand order of the matrix instruction. Tensors at the operator boundary (`torch.ops.snn_custom.*`) stay dense NCHW.

Everything here raises when libsnnf.so is missing or a call is outside what the kernels take (RuntimeError with an
`unsupported_*:` reason): there is no eager substitute.
"""
from __future__ import annotations

import json
import weakref
from collections import OrderedDict
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Optional, Sequence, Tuple

import torch

from .. import _lib
from .hip_convlif_backend import _as_pair, _packed_weight
from .hip_convlif_backend import last_conv_plan as _library_conv_plan

NCHW, C8, BITS = _lib.SNNF_LAYOUT_NCHW, _lib.SNNF_LAYOUT_C8, _lib.SNNF_LAYOUT_BITS
LAYOUT_NAMES = {NCHW: "nchw", C8: "c8", BITS: "bits"}


@dataclass
class Blocked:
    """T x N frames of [C, H, W] in one of the layouts. `data` is [T, N, C, H, W] (NCHW), [T, N, C8, H, W, 8] (C8) in the
    activation dtype, or [T, N, C8, H, W] uint8 (BITS). `shared`: every timestep is the same frame (data holds one)."""

    data: torch.Tensor
    layout: int
    T: int
    N: int
    C: int
    H: int
    W: int
    dtype: torch.dtype
    shared: bool = False

    @property
    def shape(self) -> Tuple[int, int, int, int, int]:
        return (self.T, self.N, self.C, self.H, self.W)

    def step_pointers(self):
        if self.shared:
            return _lib.step_pointers([self.data[0]] * self.T)
        return _lib.packed_step_pointers(self.data)

    def step_stride_bytes(self) -> int:
        return int(self.data.stride(0)) * self.data.element_size()


def _check_dtype(dtype: torch.dtype) -> None:
    if dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError(f"unsupported_dtype: the internal layouts hold bfloat16 or float16 activations, got {dtype}")


def empty_blocked(layout: int, T: int, N: int, C: int, H: int, W: int, dtype: torch.dtype, device) -> Blocked:
    _check_dtype(dtype)
    c8 = (C + 7) // 8
    if layout == NCHW:
        data = torch.empty((T, N, C, H, W), dtype=dtype, device=device)
    elif layout == C8:
        data = torch.empty((T, N, c8, H, W, 8), dtype=dtype, device=device)
    elif layout == BITS:
        data = torch.empty((T, N, c8, H, W), dtype=torch.uint8, device=device)
    else:
        raise RuntimeError(f"unknown layout code {layout}")
    return Blocked(data, layout, T, N, C, H, W, dtype)


def from_dense(x_seq: torch.Tensor, layout: int = BITS, shared: bool = False) -> Blocked:
    """Dense [T, N, C, H, W] (or one [N, C, H, W] frame with `shared`) -> the layout (BITS: element != 0)."""
    if shared and x_seq.dim() == 4:
        x_seq = x_seq.unsqueeze(0)
    if x_seq.dim() != 5 or not x_seq.is_cuda:
        raise RuntimeError("unsupported_rank: from_dense takes a [T, N, C, H, W] tensor on the GPU")
    _check_dtype(x_seq.dtype)
    x = x_seq if x_seq.is_contiguous() else x_seq.contiguous()
    T, N, C, H, W = (int(d) for d in x.shape)
    src = Blocked(x, NCHW, T, N, C, H, W, x.dtype, shared)
    return src if layout == NCHW else convert(src, layout)


def convert(x: Blocked, layout: int) -> Blocked:
    if x.layout == layout:
        return x
    frames = int(x.data.shape[0]) * x.N
    out = empty_blocked(layout, int(x.data.shape[0]), x.N, x.C, x.H, x.W, x.dtype, x.data.device)
    out.T, out.shared = x.T, x.shared
    _lib.check("snnf_layout_convert", _lib.lib().snnf_layout_convert(
        x.data.data_ptr(), x.layout, out.data.data_ptr(), layout, frames, x.C, x.H, x.W, _lib.dtype_code(x.dtype),
        _lib.current_stream(x.data.device)))
    return out


def to_dense(x: Blocked) -> torch.Tensor:
    """The dense [T, N, C, H, W] tensor (spikes as 0 / 1 in the activation dtype)."""
    d = convert(x, NCHW).data
    return d.expand(x.T, -1, -1, -1, -1) if x.shared and d.shape[0] == 1 else d


def pool_blocked(x: Blocked, is_max: bool, kernel: int, stride: int, padding: int, out_layout: Optional[int] = None) -> Blocked:
    """Max (2x2 or 3x3, stride 2) or average (2x2 / 2) pooling of every frame. Max pooling keeps the layout (BITS: a bitwise
    OR); average pooling of BITS yields C8 (quarters)."""
    if x.layout == NCHW:
        raise RuntimeError("unsupported_layout: pool_blocked takes C8 or BITS tensors (dense ones go to snnf_pool2d)")
    if out_layout is None:
        out_layout = x.layout if is_max else C8
    ho = (x.H + 2 * padding - kernel) // stride + 1
    wo = (x.W + 2 * padding - kernel) // stride + 1
    frames_t = int(x.data.shape[0])
    out = empty_blocked(out_layout, frames_t, x.N, x.C, ho, wo, x.dtype, x.data.device)
    out.T, out.shared = x.T, x.shared
    _lib.check("snnf_pool2d_blocked", _lib.lib().snnf_pool2d_blocked(
        x.data.data_ptr(), x.layout, out.data.data_ptr(), out_layout, frames_t * x.N, x.C, x.H, x.W, int(kernel), int(stride),
        int(padding), 1 if is_max else 0, _lib.dtype_code(x.dtype), _lib.current_stream(x.data.device)))
    return out


# ---------------------------------------------------------------------------------------------------------------
# Measured launch choices (the role of the reference's autotune table, kernels/benchmark_conv_lif_temporal_general.py:
# 524-558,1332-1369): tuned_blocked_plans.json next to this module holds, per layer shape, the patch width, channel
# groups per LDS stage and K-sharing waves that measured fastest on an MI355X (written by tune_blocked.py); shapes
# that are not in it run on the library's planner. The table is handed to the library once per process.
# ---------------------------------------------------------------------------------------------------------------
TUNED_PLANS_PATH = Path(__file__).resolve().parent / "tuned_blocked_plans.json"
_TUNED: Optional[Dict[tuple, Dict]] = None


def _plan_key(T, N, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, shared) -> tuple:
    return (int(T), int(N), int(Cin), int(H), int(W), int(Cout), int(kh), int(kw), int(sh), int(sw), int(ph), int(pw), 1 if shared else 0)


def register_tuned_plan(key: tuple, patch_cols: int, stage_groups: int, k_waves: int) -> None:
    """Registers (all three 0: removes) a launch choice for one layer shape with the library."""
    _lib.check("snnf_conv_blocked_tune", _lib.lib().snnf_conv_blocked_tune(*key, int(patch_cols), int(stage_groups), int(k_waves)))


def load_tuned_plans(path: Optional[Path] = None) -> Dict[tuple, Dict]:
    """Reads the table and registers every entry; returns it keyed by layer shape. Called on the first convolution."""
    global _TUNED
    table: Dict[tuple, Dict] = {}
    source = TUNED_PLANS_PATH if path is None else Path(path)
    if source.exists():
        for entry in json.loads(source.read_text()).get("layers", []):
            key = _plan_key(entry["T"], entry["N"], entry["Cin"], entry["H"], entry["W"], entry["Cout"], *entry["kernel"],
                            *entry["stride"], *entry["padding"], entry["shared_frame"])
            register_tuned_plan(key, entry["patch_cols"], entry["stage_groups"], entry["k_waves"])
            table[key] = entry
    _TUNED = table
    return table


def get_autotune_best_config(T, N, Cin, H, W, weight_shape, stride, padding, shared_frame: bool = False) -> Dict:
    """The measured launch choice of a layer ({} when the layer is not in the table and runs on the planner)."""
    if _TUNED is None:
        load_tuned_plans()
    _forget_plane_matrix()
    cout, _, kh, kw = (int(d) for d in weight_shape)
    key = _plan_key(T, N, Cin, H, W, cout, kh, kw, *_as_pair(stride), *_as_pair(padding), shared_frame)
    return dict(_TUNED.get(key, {}))


_NEEDS_MEMBRANE_BUFFER: set = set()


def _is_input_frame(x: Blocked) -> bool:
    """One dense frame of at most 8 channels for all timesteps (a network's input): the convolution kernel reads it as it is."""
    return x.layout == NCHW and x.shared and x.C <= 8


def input_frame(frame: torch.Tensor, T: int) -> Blocked:
    """A network's analog input [N, C, H, W], the same for all T timesteps, as the operand of the first convolution: dense
    as it is when it has at most 8 channels, channel-blocked otherwise."""
    _check_dtype(frame.dtype)
    if frame.dim() != 4 or not frame.is_cuda:
        raise RuntimeError("unsupported_rank: input_frame takes an [N, C, H, W] tensor on the GPU")
    x = from_dense(frame.contiguous(), NCHW if int(frame.shape[1]) <= 8 else C8, shared=True)
    x.T = int(T)
    return x


# ---------------------------------------------------------------------------------------------------------------
# Convolutions on planes of a few pixels as matrix products. A stride-1 "same" convolution on a plane of at most four
# pixels connects every output pixel to every input pixel through one tap, so a sample's whole frame goes through one
# [Cout H W] x [Cin H W] matrix, and the layer is Linear + LIF over the batch: no padding taps multiplied, no tile of 32
# pixels half empty (the last stage of a VGG on 32 x 32 inputs: 512 -> 512 on 2 x 2 planes, 20.9 -> 9.5 us per layer).
# Features run in the order (channel / 8, row, column, channel % 8), which is how a C8 frame holds its elements and a
# BITS frame its bits, so the frames are the matrix rows as they lie in memory.
# ---------------------------------------------------------------------------------------------------------------
_PLANE_MATRIX_CACHE: "OrderedDict" = OrderedDict()
_LAST_PLANE_MATRIX: Optional[Dict] = None      # set by the most recent convolution of this module when it ran as a matrix product


def last_conv_plan() -> Dict:
    """What ran the most recent convolution launched through this module: the library planner's answer (kernel family,
    tile, waves, ...: hip_convlif_backend.last_conv_plan), or {"kernel": "plane_matrix", ...} for a layer on a plane of a few
    pixels that went through the Linear + LIF kernel."""
    return dict(_LAST_PLANE_MATRIX) if _LAST_PLANE_MATRIX is not None else _library_conv_plan()
_PLANE_MATRIX_LIMIT = 16
PLANE_MATRIX_MAX_PIXELS = 4
PLANE_MATRIX_MAX_ELEMENTS = 4096 * 4096


def _plane_matrix(weight: torch.Tensor, bias: torch.Tensor, H: int, W: int, ph: int, pw: int):
    """([Cout H W, Cin H W] matrix, [Cout H W] bias) of a stride-1 convolution with padding (ph, pw) on H x W planes, features
    in the order (channel / 8, row, column, channel % 8); kept per weight tensor (same rules as the packed weights)."""
    key = (id(weight), id(bias), H, W, ph, pw)
    hit = _PLANE_MATRIX_CACHE.get(key)
    if hit is not None:
        w_ref, b_ref, w_ver, b_ver, w_ptr, b_ptr, matrix, bias_row = hit
        if w_ref() is weight and b_ref() is bias and w_ver == weight._version and b_ver == bias._version \
                and w_ptr == weight.data_ptr() and b_ptr == bias.data_ptr():
            _PLANE_MATRIX_CACHE.move_to_end(key)
            return matrix, bias_row
        del _PLANE_MATRIX_CACHE[key]
    cout, cin, kh, kw = (int(d) for d in weight.shape)
    full = torch.zeros((cout, H, W, cin, H, W), dtype=weight.dtype, device=weight.device)
    for oy in range(H):
        for ox in range(W):
            for iy in range(H):
                for ix in range(W):
                    ty, tx = iy - oy + ph, ix - ox + pw
                    if 0 <= ty < kh and 0 <= tx < kw:
                        full[:, oy, ox, :, iy, ix] = weight[:, :, ty, tx]
    matrix = full.reshape(cout // 8, 8, H, W, cin // 8, 8, H, W).permute(0, 2, 3, 1, 4, 6, 7, 5).reshape(cout * H * W, cin * H * W).contiguous()
    bias_row = bias.reshape(cout // 8, 1, 1, 8).expand(cout // 8, H, W, 8).reshape(cout * H * W).contiguous()
    _PLANE_MATRIX_CACHE[key] = (weakref.ref(weight), weakref.ref(bias), weight._version, bias._version, weight.data_ptr(), bias.data_ptr(),
                                matrix, bias_row)
    while len(_PLANE_MATRIX_CACHE) > _PLANE_MATRIX_LIMIT:
        _PLANE_MATRIX_CACHE.popitem(last=False)
    return matrix, bias_row


def _forget_plane_matrix() -> None:
    global _LAST_PLANE_MATRIX
    _LAST_PLANE_MATRIX = None


def _runs_as_plane_matrix(x: Blocked, cout: int, kh: int, kw: int, sh: int, sw: int, ph: int, pw: int, lif, residual, out_layout,
                          v_init, want_v) -> bool:
    return (lif is not None and residual is None and out_layout == BITS and not want_v and x.layout in (C8, BITS) and not x.shared
            and not (isinstance(v_init, torch.Tensor) and v_init.dim() != 0)
            and 3 <= x.T <= 8 and (sh, sw) == (1, 1) and 2 * ph == kh - 1 and 2 * pw == kw - 1
            and x.H * x.W <= PLANE_MATRIX_MAX_PIXELS and x.C % 8 == 0 and cout % 8 == 0 and (cout * x.H * x.W) % 32 == 0
            and (cout * x.H * x.W) * (x.C * x.H * x.W) <= PLANE_MATRIX_MAX_ELEMENTS)


def _conv_lif_plane_matrix(x: Blocked, weight: torch.Tensor, bias: torch.Tensor, ph: int, pw: int, lif: Sequence[float]) -> Blocked:
    from .hip_temporal_linear_lif_backend import _split_workspace
    cout = int(weight.shape[0])
    fin, fout = x.C * x.H * x.W, cout * x.H * x.W
    global _LAST_PLANE_MATRIX
    matrix, bias_row = _plane_matrix(weight, bias, x.H, x.W, ph, pw)
    out = empty_blocked(BITS, x.T, x.N, cout, x.H, x.W, x.dtype, x.data.device)
    bits_in = x.layout == BITS
    _LAST_PLANE_MATRIX = {"kernel": "plane_matrix", "window": x.T, "rows": x.N, "features_in": fin, "features_out": fout,
                          "x": "bits" if bits_in else "c8"}
    lib = _lib.lib()
    workspace = _split_workspace(lib, x.data.device, x.T, x.N, fin, fout)
    _lib.check("snnf_linear_lif_bits", lib.snnf_linear_lif_bits(
        x.step_pointers(), 1 if bits_in else 0, x.T, x.N, fin, fin // 8 if bits_in else fin, _lib.dtype_code(x.dtype), matrix.data_ptr(),
        bias_row.data_ptr(), fout, None, out.data.data_ptr(), out.step_stride_bytes(), None, float(lif[0]), float(lif[1]), float(lif[2]),
        _lib.ptr(workspace), 0 if workspace is None else workspace.numel(), _lib.current_stream(x.data.device)))
    return out


def conv_lif_blocked(x: Blocked, weight: torch.Tensor, bias: Optional[torch.Tensor], stride, padding,
                     lif: Optional[Sequence[float]], residual: Optional[Blocked] = None, out_layout: int = BITS,
                     v_init: Optional[torch.Tensor] = None, want_v: bool = False):
    """Dense convolution + bias (+ residual) + LIF over the T steps of `x` (C8 or BITS), or without a neuron when `lif` is
    None (output C8 or NCHW). Returns (Blocked output, final membrane [N, Cout, Ho, Wo] fp32 or None). The membrane is
    only written when asked for (`want_v`) or when the timesteps take more than one window of the kernel."""
    if x.layout not in (C8, BITS) and not _is_input_frame(x):
        raise RuntimeError("unsupported_layout: conv_lif_blocked takes inputs in C8 or BITS layout (or one dense frame of at most 8 channels)")
    if weight.dim() != 4 or int(weight.shape[1]) != x.C:
        raise RuntimeError(f"unsupported_groups: weight {tuple(weight.shape)} does not match {x.C} input channels (dense convolutions only)")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise RuntimeError("unsupported_dtype: weight / bias dtype must be the activation dtype")
    cout, _, kh, kw = (int(d) for d in weight.shape)
    sh, sw = _as_pair(stride)
    ph, pw = _as_pair(padding)
    ho, wo = (x.H + 2 * ph - kh) // sh + 1, (x.W + 2 * pw - kw) // sw + 1
    dev = x.data.device
    if bias is None:
        bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    if _runs_as_plane_matrix(x, cout, kh, kw, sh, sw, ph, pw, lif, residual, out_layout, v_init, want_v):
        return _conv_lif_plane_matrix(x, weight, bias, ph, pw, lif), None
    if _TUNED is None:
        load_tuned_plans()
    _forget_plane_matrix()
    packed = _packed_weight(weight, bias, x.dtype)
    out = empty_blocked(out_layout, x.T, x.N, cout, ho, wo, x.dtype, dev)
    neuron = lif is not None
    # The kernel needs `v_out` to carry the membrane when it runs the steps as several windows. More than 4 steps always
    # do; whether a shorter call does (windows of 2 for layers whose accumulators would not fit otherwise) is the planner's
    # answer, learnt from its refusal the first time such a layer is called without a membrane buffer.
    layer = (x.layout, x.shared, x.T, x.N, x.C, x.H, x.W, cout, kh, kw, sh, sw, ph, pw, x.dtype)
    windows = 1 if (x.shared or x.T <= 4) and layer not in _NEEDS_MEMBRANE_BUFFER else 2
    v_out = torch.empty((x.N, cout, ho, wo), dtype=torch.float32, device=dev) if neuron and (want_v or windows > 1) else None
    if residual is not None and (residual.shape != (x.T, x.N, cout, ho, wo) or residual.dtype != x.dtype or residual.shared):
        raise RuntimeError(f"unsupported_residual_shape: residual {residual.shape} does not match the output {(x.T, x.N, cout, ho, wo)}")
    vi = None
    if v_init is not None and isinstance(v_init, torch.Tensor) and v_init.dim() != 0:
        if tuple(v_init.shape) != (x.N, cout, ho, wo) or v_init.dtype != torch.float32 or v_init.device != dev:
            raise RuntimeError("unsupported_membrane_state: v_init must be a float32 [N, Cout, Ho, Wo] tensor on the activations' device")
        vi = v_init if v_init.is_contiguous() else v_init.contiguous()
    v_th, v_reset, tau = (float(lif[0]), float(lif[1]), float(lif[2])) if neuron else (1.0, 0.0, 2.0)
    def launch(v_buffer):
        return _lib.lib().snnf_conv_lif_blocked(
            x.step_pointers(), x.layout, residual.step_pointers() if residual is not None else None,
            residual.layout if residual is not None else 0, x.T, x.N, x.C, x.H, x.W, _lib.dtype_code(x.dtype),
            packed.data_ptr(), cout, kh, kw, sh, sw, ph, pw, _lib.ptr(vi), out.data.data_ptr(), out_layout, out.step_stride_bytes(),
            _lib.ptr(v_buffer), 1 if neuron else 0, v_th, v_reset, tau, _lib.current_stream(dev))

    status = launch(v_out)
    if status != 0 and neuron and v_out is None and b"v_out is required" in _lib.lib().snnf_last_error():
        _NEEDS_MEMBRANE_BUFFER.add(layer)            # refused before anything was enqueued
        status = launch(torch.empty((x.N, cout, ho, wo), dtype=torch.float32, device=dev))
    _lib.check("snnf_conv_lif_blocked", status)
    return out, v_out


def conv_lif_blocked_shortcut(x: Blocked, weight: torch.Tensor, bias: Optional[torch.Tensor], padding,
                              shortcut_x: Blocked, shortcut_weight: torch.Tensor, shortcut_bias: Optional[torch.Tensor], shortcut_stride,
                              lif: Optional[Sequence[float]], out_layout: int = BITS, want_v: bool = False):
    """The second convolution of a residual block with the block's projection shortcut in the same accumulators:
    LIF(conv(x) + bias + conv1x1(shortcut_x, stride) + shortcut bias), both inputs bit-packed, the main convolution keeping
    its plane (stride 1, "same" padding). One launch instead of two, and the shortcut's output never exists in memory.
    Raises RuntimeError("unsupported_shortcut: ...") for layers the kernel does not take in this form (the caller then
    runs the shortcut as a convolution of its own and hands its output to conv_lif_blocked as the residual).
    Returns (Blocked output, final membrane or None)."""
    if x.layout != BITS or shortcut_x.layout != BITS:
        raise RuntimeError("unsupported_shortcut: both inputs must be bit-packed")
    if weight.dim() != 4 or shortcut_weight.dim() != 4 or int(weight.shape[1]) != x.C or int(shortcut_weight.shape[1]) != shortcut_x.C or \
            tuple(shortcut_weight.shape[2:]) != (1, 1) or int(shortcut_weight.shape[0]) != int(weight.shape[0]):
        raise RuntimeError(f"unsupported_shortcut: weights {tuple(weight.shape)} / {tuple(shortcut_weight.shape)} do not match the inputs")
    if weight.dtype != x.dtype or shortcut_weight.dtype != x.dtype or shortcut_x.dtype != x.dtype:
        raise RuntimeError("unsupported_dtype: weight dtypes must be the activation dtype")
    if (shortcut_x.T, shortcut_x.N) != (x.T, x.N) or x.shared or shortcut_x.shared:
        raise RuntimeError("unsupported_shortcut: the two inputs must have the same timesteps and batch, one frame per timestep")
    cout, _, kh, kw = (int(d) for d in weight.shape)
    ph, pw = _as_pair(padding)
    ssh, ssw = _as_pair(shortcut_stride)
    dev = x.data.device
    if bias is None:
        bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    if shortcut_bias is None:
        shortcut_bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    if _TUNED is None:
        load_tuned_plans()
    _forget_plane_matrix()
    packed = _packed_weight(weight, bias, x.dtype)
    packed_sc = _packed_weight(shortcut_weight, shortcut_bias, x.dtype)
    out = empty_blocked(out_layout, x.T, x.N, cout, x.H, x.W, x.dtype, dev)
    neuron = lif is not None
    v_out = torch.empty((x.N, cout, x.H, x.W), dtype=torch.float32, device=dev) if neuron and (want_v or x.T > 4) else None
    v_th, v_reset, tau = (float(lif[0]), float(lif[1]), float(lif[2])) if neuron else (1.0, 0.0, 2.0)
    _lib.check("snnf_conv_lif_blocked_shortcut", _lib.lib().snnf_conv_lif_blocked_shortcut(
        x.step_pointers(), shortcut_x.step_pointers(), x.T, x.N, x.C, x.H, x.W, _lib.dtype_code(x.dtype), packed.data_ptr(), cout, kh, kw,
        ph, pw, shortcut_x.C, shortcut_x.H, shortcut_x.W, ssh, ssw, packed_sc.data_ptr(), None, out.data.data_ptr(), out_layout,
        out.step_stride_bytes(), _lib.ptr(v_out), 1 if neuron else 0, v_th, v_reset, tau, _lib.current_stream(dev)))
    return out, v_out


def conv_lif_blocked_avgpool(x: Blocked, weight: torch.Tensor, bias: Optional[torch.Tensor], stride, padding, lif: Sequence[float],
                             want_v: bool = False):
    """Convolution + bias + LIF and the 2x2 / stride 2 average pool of its spikes in one launch: returns (the pooled tensor,
    channel-blocked quarters at half the plane; final membrane of the unpooled neurons or None). The result of
    `pool_blocked(conv_lif_blocked(...), False, 2, 2, 0)` without the spikes ever being stored (bit for bit where both launches
    share K among waves in the same way; this form plans patches of even extents, which can change the summation order). Raises
    RuntimeError("unsupported_pool: ...") where the kernel does not take the layer in this form."""
    if x.layout not in (C8, BITS) and not _is_input_frame(x):
        raise RuntimeError("unsupported_layout: conv_lif_blocked_avgpool takes inputs in C8 or BITS layout (or one dense frame of at most 8 channels)")
    if weight.dim() != 4 or int(weight.shape[1]) != x.C:
        raise RuntimeError(f"unsupported_groups: weight {tuple(weight.shape)} does not match {x.C} input channels (dense convolutions only)")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise RuntimeError("unsupported_dtype: weight / bias dtype must be the activation dtype")
    cout, _, kh, kw = (int(d) for d in weight.shape)
    sh, sw = _as_pair(stride)
    ph, pw = _as_pair(padding)
    ho, wo = (x.H + 2 * ph - kh) // sh + 1, (x.W + 2 * pw - kw) // sw + 1
    if ho % 2 or wo % 2:
        raise RuntimeError(f"unsupported_pool: the {ho}x{wo} output plane is not even")
    dev = x.data.device
    if bias is None:
        bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    if _TUNED is None:
        load_tuned_plans()
    _forget_plane_matrix()
    packed = _packed_weight(weight, bias, x.dtype)
    out = empty_blocked(C8, x.T, x.N, cout, ho // 2, wo // 2, x.dtype, dev)
    v_out = torch.empty((x.N, cout, ho, wo), dtype=torch.float32, device=dev) if want_v else None
    _lib.check("snnf_conv_lif_blocked_avgpool", _lib.lib().snnf_conv_lif_blocked_avgpool(
        x.step_pointers(), x.layout, x.T, x.N, x.C, x.H, x.W, _lib.dtype_code(x.dtype), packed.data_ptr(), cout, kh, kw, sh, sw, ph, pw,
        out.data.data_ptr(), out.step_stride_bytes(), _lib.ptr(v_out), float(lif[0]), float(lif[1]), float(lif[2]), _lib.current_stream(dev)))
    return out, v_out


def spike_pool_linear(x: Blocked, fc_weight: torch.Tensor, fc_bias: Optional[torch.Tensor], scale: float = 1.0) -> torch.Tensor:
    """scale * sum_t (fc_weight . mean_hw(spikes_t) + fc_bias) of bit-packed spikes: [N, K] in the activation dtype. What is
    left of the LIF -> average pool -> Linear tail when the network's last neuron has fired inside the convolution in front of
    it; `scale = 1 / T` gives the mean over the timesteps."""
    if x.layout != BITS or x.shared:
        raise RuntimeError("unsupported_layout: spike_pool_linear takes bit-packed spikes, one frame per timestep")
    if fc_weight.dim() != 2 or int(fc_weight.shape[1]) != x.C or fc_weight.dtype != x.dtype or (fc_bias is not None and fc_bias.dtype != x.dtype):
        raise RuntimeError(f"unsupported_shape: classifier {tuple(fc_weight.shape)} {fc_weight.dtype} does not match {x.C} channels of {x.dtype}")
    w = fc_weight if fc_weight.is_contiguous() else fc_weight.contiguous()
    out = torch.empty((x.N, int(w.shape[0])), dtype=x.dtype, device=x.data.device)
    _lib.check("snnf_spike_pool_linear", _lib.lib().snnf_spike_pool_linear(
        x.step_pointers(), x.T, x.N, x.C, x.H, x.W, w.data_ptr(), _lib.ptr(fc_bias), int(w.shape[0]), _lib.dtype_code(x.dtype),
        out.data_ptr(), float(scale), _lib.current_stream(x.data.device)))
    return out


def conv_lif_dense_on_blocked(x: Blocked, weight: torch.Tensor, bias: torch.Tensor, stride, padding, lif: Optional[Sequence[float]],
                              residual: Optional[Blocked] = None, out_layout: int = BITS):
    """The same layer through the dense entry points on unpacked tensors, for a layer the internal-layout kernel refuses
    (large kernels on many channels): unpack, `snnf_conv_lif` / `snnf_conv_bias` through the operator layer, and the result
    back into `out_layout`. Returns (Blocked output, final membrane or None)."""
    from .hip_convlif_backend import run_hip_temporal_conv_bias
    _forget_plane_matrix()
    dense = to_dense(x)
    xs = [dense[0]] * x.T if x.shared else list(dense.unbind(0))
    rs = None if residual is None else list(to_dense(residual).unbind(0))
    geometry = ([int(s) for s in _as_pair(stride)], [int(p) for p in _as_pair(padding)], [1, 1], 1)
    if lif is not None:
        zero_v = torch.zeros((), dtype=torch.float32, device=dense.device)
        S = torch.ops.snn_custom
        if rs is None:
            y, v = S.fused_temporal_conv_lif_state(xs, weight, bias, zero_v, *geometry, *lif, False)
        else:
            y, v = S.fused_temporal_conv_add_lif_state(xs, rs, weight, bias, zero_v, *geometry, *lif, False)
    else:
        v = None
        try:
            y = run_hip_temporal_conv_bias(xs, weight, bias, geometry[0], geometry[1], rs)
        except RuntimeError as exc:
            if "unsupported" not in str(exc):
                raise
            y = torch.nn.functional.conv2d(torch.stack(xs).flatten(0, 1), weight, bias, geometry[0], geometry[1])
            y = y.view(x.T, x.N, *y.shape[1:])
            if rs is not None:
                y = y + torch.stack(rs)
    return from_dense(y.contiguous(), out_layout), v


def conv_lif_blocked_or_dense(x: Blocked, weight: torch.Tensor, bias: torch.Tensor, stride, padding, lif: Optional[Sequence[float]],
                              residual: Optional[Blocked] = None, out_layout: int = BITS, want_v: bool = False):
    """conv_lif_blocked, and for a layer it refuses (`unsupported_*`) the dense entry points on unpacked tensors."""
    try:
        return conv_lif_blocked(x, weight, bias, stride, padding, lif, residual=residual, out_layout=out_layout, want_v=want_v)
    except RuntimeError as exc:
        if "unsupported" not in str(exc):
            raise
    return conv_lif_dense_on_blocked(x, weight, bias, stride, padding, lif, residual=residual, out_layout=out_layout)


# ---------------------------------------------------------------------------------------------------------------
# Depthwise 3x3 + LIF with row-packed spikes: one byte = the spikes of 8 consecutive pixels of a row (bit j = pixel 8 x + j).
# A depthwise lane owns such a strip, so its spikes of a timestep leave as one byte instead of eight 16-bit elements.
# ---------------------------------------------------------------------------------------------------------------
def depthwise_conv_lif_rowbits(xs: Sequence[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor, lif: Sequence[float],
                               residuals: Optional[Sequence[torch.Tensor]] = None, v_init: Optional[torch.Tensor] = None,
                               want_v: bool = True):
    """Depthwise 3x3 (stride 1, padding 1) + bias (+ residual) + LIF over the dense steps `xs` ([N, C, H, W] each, bf16 or
    fp16, W % 8 == 0), or over row-packed spikes (`xs` one uint8 tensor [T, N, C, H, W / 8]: the output of this function or
    of pointwise_conv_lif_from_rowbits(packed_out=True)). Returns (spike bits [T, N, C, H, W / 8] uint8, final membrane
    [N, C, H, W] fp32 or None)."""
    packed_in = isinstance(xs, torch.Tensor)
    if packed_in:
        if xs.dtype != torch.uint8 or xs.dim() != 5 or not xs[0].is_contiguous():
            raise RuntimeError("unsupported_layout: row-packed spikes [T, N, C, H, W / 8] uint8 expected")
        xs = list(xs.unbind(0))
    first = xs[0]
    op_dtype = weight.dtype if packed_in else first.dtype
    _check_dtype(op_dtype)
    T = len(xs)
    n, c, h, w = (int(d) for d in first.shape)
    if packed_in:
        w *= 8
    if tuple(weight.shape) != (c, 1, 3, 3) or weight.dtype != op_dtype or bias.dtype != op_dtype:
        raise RuntimeError(f"unsupported_weight: depthwise weight [C, 1, 3, 3] and bias in the activation dtype expected, got {tuple(weight.shape)}")
    if w % 8 != 0:
        raise RuntimeError(f"unsupported_shape: rows of {w} pixels do not pack into whole bytes")
    dev = first.device
    steps = [x if x.is_contiguous() else x.contiguous() for x in xs]
    res = [r if r.is_contiguous() else r.contiguous() for r in residuals] if residuals is not None else None
    vi = None
    if v_init is not None and isinstance(v_init, torch.Tensor) and v_init.dim() != 0:
        if tuple(v_init.shape) != (n, c, h, w) or v_init.dtype != torch.float32 or v_init.device != dev:
            raise RuntimeError("unsupported_membrane_state: v_init must be a float32 [N, C, H, W] tensor on the activations' device")
        vi = v_init if v_init.is_contiguous() else v_init.contiguous()
    bits = torch.empty((T, n, c, h, w // 8), dtype=torch.uint8, device=dev)
    v_out = torch.empty((n, c, h, w), dtype=torch.float32, device=dev) if (want_v or T > _lib.SNNF_MAX_T_PER_LAUNCH) else None
    wc = weight if weight.is_contiguous() else weight.contiguous()
    bc = bias if bias.is_contiguous() else bias.contiguous()
    _lib.check("snnf_dwconv3x3_lif_rowbits", _lib.lib().snnf_dwconv3x3_lif_rowbits(
        _lib.step_pointers(steps), _lib.step_pointers(res) if res is not None else None, T, n, c, h, w, _lib.dtype_code(op_dtype),
        1 if packed_in else 0, wc.data_ptr(), bc.data_ptr(), _lib.ptr(vi), bits.data_ptr(), int(bits.stride(0)), _lib.ptr(v_out),
        float(lif[0]), float(lif[1]), float(lif[2]), _lib.current_stream(dev)))
    return bits, (v_out if want_v else None)


def unpack_rowbits(bits: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Row-packed spikes [..., W / 8] uint8 -> dense 0 / 1 elements [..., W] of `dtype` (bf16 or fp16)."""
    _check_dtype(dtype)
    if bits.dtype != torch.uint8 or not bits.is_contiguous():
        raise RuntimeError("unsupported_layout: contiguous uint8 tensor of row-packed spikes expected")
    dense = torch.empty(tuple(bits.shape[:-1]) + (int(bits.shape[-1]) * 8,), dtype=dtype, device=bits.device)
    _lib.check("snnf_rowbits_unpack", _lib.lib().snnf_rowbits_unpack(bits.data_ptr(), dense.data_ptr(), bits.numel(), _lib.dtype_code(dtype),
                                                                   _lib.current_stream(bits.device)))
    return dense


def pointwise_conv_lif_from_rowbits(bits: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], lif: Sequence[float],
                                    v_init: Optional[torch.Tensor] = None, packed_out: bool = False, want_v: bool = True):
    """Pointwise (1x1, stride 1) convolution + bias + LIF over T steps of row-packed spikes `bits` [T, N, Cin, H, W / 8]
    uint8 (what depthwise_conv_lif_rowbits writes). Returns (spikes [T, N, Cout, H, W] in the weight's dtype, final
    membrane [N, Cout, H, W] fp32): the dense outputs of the operator on the unpacked tensor. `packed_out`: the spikes
    leave row-packed as well ([T, N, Cout, H, W / 8] uint8), and the membrane only when asked for (`want_v`)."""
    _check_dtype(weight.dtype)
    if bits.dtype != torch.uint8 or bits.dim() != 5 or not bits[0].is_contiguous():
        raise RuntimeError("unsupported_layout: row-packed spikes [T, N, Cin, H, W / 8] uint8 expected")
    T, n, cin, h, w8 = (int(d) for d in bits.shape)
    w = w8 * 8
    if weight.dim() != 4 or tuple(weight.shape[1:]) != (cin, 1, 1):
        raise RuntimeError(f"unsupported_weight: pointwise weight [Cout, {cin}, 1, 1] expected, got {tuple(weight.shape)}")
    cout = int(weight.shape[0])
    dev = bits.device
    if bias is None:
        bias = torch.zeros(cout, dtype=weight.dtype, device=weight.device)
    packed = _packed_weight(weight, bias, weight.dtype)
    vi = None
    if v_init is not None and isinstance(v_init, torch.Tensor) and v_init.dim() != 0:
        if tuple(v_init.shape) != (n, cout, h, w) or v_init.dtype != torch.float32 or v_init.device != dev:
            raise RuntimeError("unsupported_membrane_state: v_init must be a float32 [N, Cout, H, W] tensor on the activations' device")
        vi = v_init if v_init.is_contiguous() else v_init.contiguous()
    if packed_out:
        spikes = torch.empty((T, n, cout, h, w8), dtype=torch.uint8, device=dev)
    else:
        spikes = torch.empty((T, n, cout, h, w), dtype=weight.dtype, device=dev)
    need_v = want_v or not packed_out or T > _lib.SNNF_MAX_T_PER_LAUNCH
    v_out = torch.empty((n, cout, h, w), dtype=torch.float32, device=dev) if need_v else None
    _lib.check("snnf_pwconv_lif_rowbits", _lib.lib().snnf_pwconv_lif_rowbits(
        _lib.packed_step_pointers(bits), T, n, cin, h, w, _lib.dtype_code(weight.dtype), packed.data_ptr(), cout, _lib.ptr(vi),
        spikes.data_ptr(), 1 if packed_out else 0, int(spikes.stride(0)), _lib.ptr(v_out),
        float(lif[0]), float(lif[1]), float(lif[2]), _lib.current_stream(dev)))
    return spikes, (v_out if (want_v or not packed_out) else None)


def pack_rowbits(dense: torch.Tensor) -> torch.Tensor:
    """Dense spikes [..., W] (bf16 or fp16, W % 8 == 0) -> row-packed [..., W / 8] uint8, bit j = element 8 x + j != 0."""
    _check_dtype(dense.dtype)
    if int(dense.shape[-1]) % 8 != 0:
        raise RuntimeError(f"unsupported_shape: rows of {int(dense.shape[-1])} pixels do not pack into whole bytes")
    src = dense if dense.is_contiguous() else dense.contiguous()
    bits = torch.empty(tuple(src.shape[:-1]) + (int(src.shape[-1]) // 8,), dtype=torch.uint8, device=src.device)
    _lib.check("snnf_rowbits_pack", _lib.lib().snnf_rowbits_pack(src.data_ptr(), bits.data_ptr(), bits.numel(), _lib.dtype_code(src.dtype),
                                                               _lib.current_stream(src.device)))
    return bits
