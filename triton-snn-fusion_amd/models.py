"""Spiking VGG-11-style and ResNet-18-style networks, as single-step eager modules and as fused temporal executors.

Counterpart of the reference's model harness (benchmarks/validate_chronos_baselines.py:234-244 `SingleStepModeLoopWrapper`,
:286-293 the (v_th 1, v_reset 0, tau 2) neuron, :304-309 state reset, :748-790 the VGG / ResNet constructors; the neuron
contract `CustomStatefulIFNode` as used in benchmarks/benchmark_tensorrt_runtime.py:42-79). The reference builds these
networks from spikingjelly's model zoo and lets its FX compiler group the T unrolled single-step iterations into
temporal operators; here the two networks are defined directly and each has

  * an eager form (`SpikingVGG11`, `SpikingResNet18`): one timestep per call, Conv2d -> BatchNorm2d -> neuron, state kept
    in the neuron modules, driven by `SingleStepModeLoopWrapper` (same analog frame every step, readout = sum / T);
  * a fused form (`FusedSpikingVGG11`, `FusedSpikingResNet18`): layer-major execution of the same network through
    `torch.ops.snn_custom.fused_temporal_*` (BatchNorm folded into the convolution, all T steps of a layer in one
    call, the last neuron + global average pool + classifier in `fused_temporal_lif_avgpool_linear`). This is the
    operator sequence the reference's temporal rewrite produces for such a graph.

What stays on stock PyTorch in the fused form is what the reference leaves as ordinary graph nodes too: the pooling
between stages, the LIF-free 1x1 downsample shortcuts and the last convolution whose neuron belongs to the tail.
"""
from __future__ import annotations

import copy
import math
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .workloads import BN_EPS, LIF_DEFAULT, fold_bn_into_conv_params


# ---------------------------------------------------------------------------------------------------------------
# Neuron and wrappers
# ---------------------------------------------------------------------------------------------------------------
class CustomStatefulIFNode(nn.Module):
    """Single-step LIF neuron that keeps its membrane in `self.v` between calls (forward only).

    forward(x) = `torch.ops.snn_custom.lif_forward_state(x, self.v, v_threshold, v_reset, tau, detach_reset)`; a 0-dim
    (or otherwise mismatching) `self.v` means "start from zeros" (reference runtime/snn_custom_ops.py:378-381)."""

    def __init__(self, v_threshold: float = 1.0, v_reset: float = 0.0, tau: float = 2.0, detach_reset: bool = False,
                 surrogate_function: Optional[Callable] = None, step_mode: str = "s"):
        super().__init__()
        self.v_threshold = float(v_threshold)
        self.v_reset = float(v_reset)
        self.tau = float(tau)
        self.detach_reset = bool(detach_reset)
        self.surrogate_function = surrogate_function     # forward-only: kept for interface compatibility
        self.step_mode = step_mode
        self.v: torch.Tensor = torch.tensor(0.0)

    def reset(self) -> None:
        self.v = torch.tensor(0.0)

    def reset_state_if_needed(self, x: torch.Tensor) -> None:
        v = self.v
        if not isinstance(v, torch.Tensor) or v.shape != x.shape or v.dtype != x.dtype or v.device != x.device:
            self.v = torch.zeros((), dtype=x.dtype, device=x.device)

    @property
    def lif_params(self) -> Tuple[float, float, float]:
        return (self.v_threshold, self.v_reset, self.tau)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        from .runtime import snn_custom_ops  # noqa: F401  (registers torch.ops.snn_custom)
        self.reset_state_if_needed(x)
        spike, self.v = torch.ops.snn_custom.lif_forward_state(x, self.v, self.v_threshold, self.v_reset, self.tau,
                                                               self.detach_reset)
        return spike


def reset_custom_stateful_lif_modules(model: nn.Module) -> None:
    for m in model.modules():
        if isinstance(m, CustomStatefulIFNode):
            m.reset()


reset_lif_modules = reset_custom_stateful_lif_modules


class SingleStepModeLoopWrapper(nn.Module):
    """Feeds the same frame to a single-step network T times and averages its outputs."""

    def __init__(self, layer: nn.Module, T: int):
        super().__init__()
        self.layer = layer
        self.T = int(T)

    def forward(self, x):
        out_spikes_counter = 0
        for _ in range(self.T):
            out_spikes_counter = out_spikes_counter + self.layer(x)
        return out_spikes_counter / self.T


def _neuron() -> CustomStatefulIFNode:
    v_th, v_reset, tau = LIF_DEFAULT
    return CustomStatefulIFNode(v_threshold=v_th, v_reset=v_reset, tau=tau)


# ---------------------------------------------------------------------------------------------------------------
# Eager single-step networks
# ---------------------------------------------------------------------------------------------------------------
class ConvBNNeuron(nn.Module):
    """Conv2d (no bias) -> BatchNorm2d -> neuron; `sn` is None for a LIF-free convolution (shortcut, pre-tail)."""

    def __init__(self, cin: int, cout: int, kernel: int, stride: int, padding: int, neuron: bool = True, groups: int = 1):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, kernel, stride, padding, groups=groups, bias=False)
        self.bn = nn.BatchNorm2d(cout, eps=BN_EPS)
        self.sn = _neuron() if neuron else None

    def forward(self, x):
        y = self.bn(self.conv(x))
        return self.sn(y) if self.sn is not None else y


VGG11_STAGES = ((64,), (128,), (256, 256), (512, 512), (512, 512))


class SpikingVGG11(nn.Module):
    """Conv3x3+BN+LIF stages 64 | 128 | 256-256 | 512-512 | 512-512 with a 2x2 average pool between stages; the last
    convolution's neuron opens the tail LIF -> global average pool -> Linear. `width` scales every channel count."""

    def __init__(self, num_classes: int = 10, in_channels: int = 3, width: int = 64):
        super().__init__()
        layers: List[nn.Module] = []
        cin = in_channels
        convs = [(max(1, c * width // 64), si) for si, stage in enumerate(VGG11_STAGES) for c in stage]
        for i, (cout, si) in enumerate(convs):
            if i > 0 and si != convs[i - 1][1]:
                layers.append(nn.AvgPool2d(2))
            layers.append(ConvBNNeuron(cin, cout, 3, 1, 1, neuron=i + 1 < len(convs)))
            cin = cout
        self.features = nn.Sequential(*layers)
        self.tail_sn = _neuron()
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(cin, num_classes)

    def forward(self, x):
        y = self.tail_sn(self.features(x))
        return self.fc(torch.flatten(self.avgpool(y), 1))


class SpikingBasicBlock(nn.Module):
    """conv3x3-BN-LIF, conv3x3-BN, + identity (1x1/stride conv + BN when the shape changes), LIF."""

    def __init__(self, cin: int, cout: int, stride: int):
        super().__init__()
        self.conv1 = ConvBNNeuron(cin, cout, 3, stride, 1)
        self.conv2 = ConvBNNeuron(cout, cout, 3, 1, 1, neuron=False)
        self.downsample = ConvBNNeuron(cin, cout, 1, stride, 0, neuron=False) if (stride != 1 or cin != cout) else None
        self.sn2: Optional[CustomStatefulIFNode] = _neuron()

    def pre_activation(self, x):
        identity = x if self.downsample is None else self.downsample(x)
        return self.conv2(self.conv1(x)) + identity

    def forward(self, x):
        y = self.pre_activation(x)
        return self.sn2(y) if self.sn2 is not None else y


class SpikingResNet18(nn.Module):
    """Stem 7x7/2 + BN + LIF + 3x3/2 max pool, four stages of two BasicBlocks (64/128/256/512, stride 2 from the
    second stage on, 1x1 downsample shortcuts), tail LIF -> global average pool -> Linear. The last block's output
    neuron is the tail's neuron."""

    def __init__(self, num_classes: int = 1000, in_channels: int = 3, width: int = 64, blocks: Sequence[int] = (2, 2, 2, 2)):
        super().__init__()
        self.stem = ConvBNNeuron(in_channels, width, 7, 2, 3)
        self.maxpool = nn.MaxPool2d(3, 2, 1)
        layers: List[nn.Module] = []
        cin = width
        for si, n in enumerate(blocks):
            cout = width << si
            for bi in range(n):
                layers.append(SpikingBasicBlock(cin, cout, 2 if (si > 0 and bi == 0) else 1))
                cin = cout
        self.blocks = nn.Sequential(*layers)
        self.tail_sn = self.blocks[-1].sn2
        self.blocks[-1].sn2 = None                  # applied as the tail's neuron
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(cin, num_classes)

    def forward(self, x):
        y = self.tail_sn(self.blocks(self.maxpool(self.stem(x))))
        return self.fc(torch.flatten(self.avgpool(y), 1))


# (output channels, stride of the depthwise layer) of the depthwise-separable blocks behind the 3x3/2 stem of 32 channels.
MOBILENET_BLOCKS = ((64, 1), (128, 2), (128, 1), (256, 2))


class SpikingMobileNet(nn.Module):
    """MobileNetV1-style network (counterpart of the reference zoo's MobileNet entries, benchmarks/
    validate_chronos_baselines.py:312-847, in shape only): stem Conv3x3/2 + BN + LIF, then depthwise-separable blocks
    (depthwise Conv3x3 + BN + LIF, pointwise Conv1x1 + BN + LIF), tail LIF -> global average pool -> Linear. The last
    pointwise convolution's neuron is the tail's neuron. `width` scales every channel count (32 = the full network)."""

    def __init__(self, num_classes: int = 10, in_channels: int = 3, width: int = 32, blocks: Sequence[Tuple[int, int]] = MOBILENET_BLOCKS):
        super().__init__()
        scale = lambda c: max(8, c * width // 32 // 8 * 8)      # multiples of 8: whole channel groups for the matrix kernels
        cin = scale(32)
        layers: List[nn.Module] = [ConvBNNeuron(in_channels, cin, 3, 2, 1)]
        for i, (cout, stride) in enumerate(blocks):
            cout = scale(cout)
            layers.append(ConvBNNeuron(cin, cin, 3, stride, 1, groups=cin))
            layers.append(ConvBNNeuron(cin, cout, 1, 1, 0, neuron=i + 1 < len(blocks)))
            cin = cout
        self.features = nn.Sequential(*layers)
        self.tail_sn = _neuron()
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(cin, num_classes)

    def forward(self, x):
        y = self.tail_sn(self.features(x))
        return self.fc(torch.flatten(self.avgpool(y), 1))


def init_synthetic_(model: nn.Module, seed: int = 0, gain: float = 1.0) -> nn.Module:
    """Kaiming-normal convolution and classifier weights (scaled by `gain`), classifier bias N(0, 0.01^2), BatchNorm
    gamma U(0.8, 1.2), beta N(0, 0.1^2), running mean N(0, 0.1^2), running variance U(0.5, 1.5); CPU generator `seed`."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, (nn.Conv2d, nn.Linear)):
                fan_in = m.weight[0].numel()
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * math.sqrt(2.0 / fan_in) * gain)
                if m.bias is not None:
                    m.bias.copy_(torch.randn(m.bias.shape, generator=g) * 0.01)
            elif isinstance(m, nn.BatchNorm2d):
                c = m.num_features
                m.weight.copy_(torch.rand(c, generator=g) * 0.4 + 0.8)
                m.bias.copy_(torch.randn(c, generator=g) * 0.1)
                m.running_mean.copy_(torch.randn(c, generator=g) * 0.1)
                m.running_var.copy_(torch.rand(c, generator=g) + 0.5)
    return model.eval()


def fold_batchnorm(model: nn.Module, round_to: Optional[torch.dtype] = None) -> nn.Module:
    """Copy of `model` with every eval-mode BatchNorm folded into its convolution (which gains a bias) and, when
    `round_to` is given, all convolution / classifier parameters rounded to that dtype (values kept in fp32). The eager
    form of the copy computes with exactly the operands the fused form feeds to the kernels."""
    model = copy.deepcopy(model).eval()

    def rounded(t: torch.Tensor) -> torch.Tensor:
        return t if round_to is None else t.to(round_to).to(torch.float32)

    with torch.no_grad():
        for m in list(model.modules()):
            if isinstance(m, ConvBNNeuron) and isinstance(m.bn, nn.BatchNorm2d):
                w, b = fold_bn_into_conv_params(m.conv.weight.float(), m.conv.bias, m.bn.running_mean.float(),
                                                m.bn.running_var.float(), m.bn.weight.float(), m.bn.bias.float(), m.bn.eps)
                conv = nn.Conv2d(m.conv.in_channels, m.conv.out_channels, m.conv.kernel_size, m.conv.stride, m.conv.padding, groups=m.conv.groups, bias=True)
                conv.weight.copy_(rounded(w))
                conv.bias.copy_(rounded(b))
                m.conv, m.bn = conv.to(w.device), nn.Identity()
            elif isinstance(m, nn.Linear):
                m.weight.copy_(rounded(m.weight.float()))
                if m.bias is not None:
                    m.bias.copy_(rounded(m.bias.float()))
    return model


# ---------------------------------------------------------------------------------------------------------------
# Fused temporal executors
# ---------------------------------------------------------------------------------------------------------------
class _FusedLayer:
    """Folded parameters of one ConvBNNeuron in the activation dtype on the target device."""

    def __init__(self, m: ConvBNNeuron, dtype: torch.dtype, device: torch.device):
        with torch.no_grad():
            if isinstance(m.bn, nn.BatchNorm2d):
                w, b = fold_bn_into_conv_params(m.conv.weight.float(), m.conv.bias, m.bn.running_mean.float(),
                                                m.bn.running_var.float(), m.bn.weight.float(), m.bn.bias.float(), m.bn.eps)
            else:
                w = m.conv.weight.float()
                b = m.conv.bias.float() if m.conv.bias is not None else torch.zeros(w.shape[0])
            self.weight = w.to(device=device, dtype=dtype).contiguous()
            self.bias = b.to(device=device, dtype=dtype).contiguous()
        self.stride = [int(s) for s in m.conv.stride]
        self.padding = [int(p) for p in m.conv.padding]
        self.groups = int(m.conv.groups)
        self.lif = m.sn.lif_params if m.sn is not None else None

    @property
    def geometry(self):
        return (self.stride, self.padding, [1, 1], self.groups)


class _FusedNetwork(nn.Module):
    """Shared plumbing: parameter folding, operator calls, optional recording of every operator call (inputs and
    outputs, for layer-by-layer verification), and whole-forward HIP graph capture."""

    def __init__(self, T: int, dtype: torch.dtype, device, v_dtype: torch.dtype = torch.float32,
                 internal_layouts: bool = False):
        super().__init__()
        from .runtime import snn_custom_ops
        if torch.device(device).type == "cuda":
            # Native kernels only: an operator call they cannot serve raises instead of running the eager ops.
            snn_custom_ops.configure_fused_op("hip", strict_triton=True)
        self.T = int(T)
        self.dtype = dtype
        self.device_ = torch.device(device)
        self.zero_v = torch.zeros((), dtype=v_dtype, device=self.device_)
        self.record: Optional[List[Dict]] = None
        self.native_plain_conv = True        # False: LIF-free convolutions always go to the framework's convolution
        self.native_pool = True              # False: pooling layers always go to the framework's modules
        # True: between the network's own operators spikes travel bit-packed and analog activations channel-blocked
        # (runtime/hip_blocked_backend.py); the dense `snn_custom` operators then only serve the tail. GPU, 16-bit only.
        self.internal_layouts = bool(internal_layouts)
        self.keep_membranes = False          # internal layouts: also write every layer's final membrane (nobody reads it:
                                             # the harness resets all neurons between forwards, like the reference's)
        self._graph = None

    # -- operator calls ------------------------------------------------------------------------------------------
    def _log(self, **entry):
        if self.record is not None:
            self.record.append(entry)

    def conv_lif(self, name: str, xs: List[torch.Tensor], layer: _FusedLayer, residuals: Optional[List[torch.Tensor]] = None):
        S = torch.ops.snn_custom
        if residuals is None:
            # The operator per convolution kind, as the reference's rewrite selects it (compiler/fx_lif_temporal_rewrite.py:1625-1662).
            if layer.groups > 1:
                op = S.fused_temporal_depthwise_conv_lif_state
            elif tuple(layer.weight.shape[2:]) == (1, 1) and layer.stride == [1, 1] and layer.padding == [0, 0]:
                op = S.fused_temporal_pointwise_conv_lif_state
            else:
                op = S.fused_temporal_conv_lif_state
            spikes, v = op(xs, layer.weight, layer.bias, self.zero_v, *layer.geometry, *layer.lif, False)
        else:
            spikes, v = S.fused_temporal_conv_add_lif_state(xs, residuals, layer.weight, layer.bias, self.zero_v,
                                                            *layer.geometry, *layer.lif, False)
        self._log(kind="conv_lif", name=name, xs=xs, residuals=residuals, layer=layer, spikes=spikes, v=v)
        return spikes

    def plain_conv(self, name: str, x_seq: torch.Tensor, layer: _FusedLayer, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """LIF-free convolution (+ residual) of T frames, bias = folded BatchNorm shift: the matrix kernel's neuron-free
        mode where it takes the layer, the framework's convolution otherwise (and on CPU tensors)."""
        y = None
        if x_seq.is_cuda and self.native_plain_conv:
            from .runtime.hip_convlif_backend import run_hip_temporal_conv_bias
            try:
                y = run_hip_temporal_conv_bias(list(x_seq.unbind(0)), layer.weight, layer.bias, layer.stride, layer.padding,
                                               None if residual is None else list(residual.unbind(0)))
                native = True
            except RuntimeError as exc:
                if "unsupported" not in str(exc):
                    raise
        if y is None:
            native = False
            y = F.conv2d(x_seq.flatten(0, 1), layer.weight, layer.bias, layer.stride, layer.padding)
            y = y.view(x_seq.shape[0], x_seq.shape[1], *y.shape[1:])
            if residual is not None:
                y = y + residual
        self._log(kind="plain_conv", name=name, x=x_seq, layer=layer, residual=residual, y=y, native=native)
        return y

    def pooled(self, name: str, x_seq: torch.Tensor, pool: nn.Module) -> torch.Tensor:
        """Pooling of all T*N frames at once: the HIP pooling kernel for the window shapes it has, the module itself
        otherwise (and on CPU tensors)."""
        from .runtime.hip_pool_backend import pool_config, run_hip_pool2d
        config = pool_config(pool) if (x_seq.is_cuda and self.native_pool) else None
        if config is not None:
            y = run_hip_pool2d(x_seq, *config)
        else:
            y = pool(x_seq.flatten(0, 1))
            y = y.view(x_seq.shape[0], x_seq.shape[1], *y.shape[1:])
        self._log(kind="pool", name=name, x=x_seq, pool=pool, y=y, native=config is not None)
        return y

    # -- the same operators on the internal layouts ----------------------------------------------------------------
    def conv_lif_b(self, name: str, x, layer: _FusedLayer, residual=None, out_layout=None):
        """Conv + folded BN (+ residual) + LIF (`layer.lif`), or without a neuron when the layer has none, on Blocked tensors."""
        from .runtime import hip_blocked_backend as B
        if out_layout is None:
            out_layout = B.BITS if layer.lif is not None else B.C8
        # A layer the blocked kernel does not take (large kernels on many channels) runs the dense entry points on
        # unpacked tensors, and its result goes back into the layout the next operator expects.
        out, v = B.conv_lif_blocked_or_dense(x, layer.weight, layer.bias, layer.stride, layer.padding, layer.lif, residual=residual,
                                             out_layout=out_layout, want_v=self.keep_membranes or self.record is not None)
        if self.record is not None:
            T = x.T
            xs = list(B.to_dense(x).unbind(0)) if not x.shared else [B.to_dense(x)[0]] * T
            rs = None if residual is None else list(B.to_dense(residual).unbind(0))
            if layer.lif is not None:
                self._log(kind="conv_lif", name=name, xs=xs, residuals=rs, layer=layer, spikes=B.to_dense(out), v=v, blocked=True)
            else:
                self._log(kind="plain_conv", name=name, x=torch.stack(xs), layer=layer, residual=None if rs is None else torch.stack(rs),
                          y=B.to_dense(out), native=True, blocked=True)
        return out

    def conv_lif_shortcut_b(self, name: str, x, layer: _FusedLayer, shortcut_x, shortcut: _FusedLayer, out_layout=None):
        """The second convolution of a down-sampling block with the block's LIF-free 1x1 shortcut in its accumulators (one
        launch); None when the kernel does not take the pair in this form (the caller then runs the two apart)."""
        from .runtime import hip_blocked_backend as B
        if out_layout is None:
            out_layout = B.BITS if layer.lif is not None else B.C8
        if layer.stride != [1, 1] or shortcut.padding != [0, 0] or tuple(shortcut.weight.shape[2:]) != (1, 1):
            return None
        try:
            out, v = B.conv_lif_blocked_shortcut(x, layer.weight, layer.bias, layer.padding, shortcut_x, shortcut.weight, shortcut.bias,
                                                 shortcut.stride, layer.lif, out_layout=out_layout,
                                                 want_v=self.keep_membranes or self.record is not None)
        except RuntimeError as exc:
            if "unsupported" not in str(exc):
                raise
            return None
        if self.record is not None:
            self._log(kind="conv_lif", name=name, xs=list(B.to_dense(x).unbind(0)), residuals=None, layer=layer, spikes=B.to_dense(out), v=v,
                      blocked=True, shortcut=dict(x=B.to_dense(shortcut_x), layer=shortcut))
        return out

    def conv_lif_pool_b(self, name: str, x, layer: _FusedLayer, pool_name: str, pool: nn.Module):
        """Conv + folded BN + LIF and the 2x2 average pool behind it in one launch (the spikes are never stored); None when
        the pool is another one or the kernel does not take the layer in this form (the caller then runs the two apart)."""
        from .runtime import hip_blocked_backend as B
        from .runtime.hip_pool_backend import pool_config
        if layer.lif is None or pool_config(pool) != (False, 2, 2, 0):
            return None
        try:
            y, v = B.conv_lif_blocked_avgpool(x, layer.weight, layer.bias, layer.stride, layer.padding, layer.lif,
                                              want_v=self.keep_membranes or self.record is not None)
        except RuntimeError as exc:
            if "unsupported" not in str(exc):
                raise
            return None
        if self.record is not None:      # the spikes for the record come from the unpooled launch; the pooled tensor is the fused launch's
            spikes, _ = B.conv_lif_blocked(x, layer.weight, layer.bias, layer.stride, layer.padding, layer.lif)
            xs = list(B.to_dense(x).unbind(0)) if not x.shared else [B.to_dense(x)[0]] * x.T
            self._log(kind="conv_lif", name=name, xs=xs, residuals=None, layer=layer, spikes=B.to_dense(spikes), v=v, blocked=True)
            self._log(kind="pool", name=pool_name, x=B.to_dense(spikes), pool=pool, y=B.to_dense(y), native=True, blocked=True)
        return y

    def last_conv_and_tail_b(self, name: str, x, layer: _FusedLayer, lif, fc_weight, fc_bias, residual=None) -> torch.Tensor:
        """The network's last, neuron-free convolution (+ residual) and the LIF -> average pool -> Linear tail behind it: the
        tail's neuron fires in the convolution's epilogue (bit-packed spikes out), the pool and the classifier run on the
        bits and yield the mean over T. Where a kernel does not take the layer in that form the convolution writes its sums
        dense and the tail operator follows."""
        from .runtime import hip_blocked_backend as B
        with_neuron = copy.copy(layer)
        with_neuron.lif = tuple(lif)
        try:
            spikes = self.conv_lif_b(name, x, with_neuron, residual=residual, out_layout=B.BITS)
            logits = B.spike_pool_linear(spikes, fc_weight, fc_bias, 1.0 / self.T)
        except RuntimeError as exc:
            if "unsupported" not in str(exc):
                raise
            sums = self.conv_lif_b(name, x, layer, residual=residual, out_layout=B.NCHW)
            return self.tail(B.to_dense(sums), lif, fc_weight, fc_bias)
        if self.record is not None:
            self._log(kind="spike_pool_linear", name="tail", x=B.to_dense(spikes), fc_weight=fc_weight, fc_bias=fc_bias, out=logits)
        return logits

    def pooled_b(self, name: str, x, pool: nn.Module):
        from .runtime import hip_blocked_backend as B
        from .runtime.hip_pool_backend import pool_config
        config = pool_config(pool)
        if config is None:
            raise RuntimeError(f"unsupported_kernel: no blocked pooling kernel for {pool}")
        y = B.pool_blocked(x, *config)
        if self.record is not None:
            self._log(kind="pool", name=name, x=B.to_dense(x), pool=pool, y=B.to_dense(y), native=True, blocked=True)
        return y

    def tail(self, x_seq: torch.Tensor, lif, fc_weight, fc_bias) -> torch.Tensor:
        out_sum, v = torch.ops.snn_custom.fused_temporal_lif_avgpool_linear(x_seq, self.zero_v, fc_weight, fc_bias, *lif, False)
        self._log(kind="tail", name="tail", x=x_seq, lif=lif, fc_weight=fc_weight, fc_bias=fc_bias, out_sum=out_sum, v=v)
        return out_sum / self.T

    # -- driver --------------------------------------------------------------------------------------------------
    def _prepare(self, x: torch.Tensor) -> torch.Tensor:
        return x.to(device=self.device_, dtype=self.dtype).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        with torch.no_grad():
            x = self._prepare(x)
            if self.internal_layouts:
                if not x.is_cuda or x.dtype not in (torch.bfloat16, torch.float16):
                    raise RuntimeError("unsupported_dtype: the internal layouts need bfloat16 / float16 tensors on the GPU")
                return self.run_blocked(x)
            return self.run(x)

    def run_blocked(self, x: torch.Tensor) -> torch.Tensor:     # pragma: no cover - implemented by the subclasses
        raise NotImplementedError

    def run(self, x: torch.Tensor) -> torch.Tensor:     # pragma: no cover - implemented by the subclasses
        raise NotImplementedError

    def capture(self, example: torch.Tensor, warmup: int = 3):
        """Captures the whole forward into one HIP graph; returns (replay, static_input, static_output).

        The warm-up forwards run on a side stream first (weight packing, library handles and the caching allocator
        settle outside the capture). Kernels are enqueued by every operator on the current stream without allocating
        or synchronising, so the capture holds kernel nodes only."""
        static_in = self._prepare(example).clone()
        side = torch.cuda.Stream(device=self.device_)
        side.wait_stream(torch.cuda.current_stream(self.device_))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                self.forward(static_in)
        torch.cuda.current_stream(self.device_).wait_stream(side)
        torch.cuda.synchronize(self.device_)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = self.forward(static_in)
        self._graph = graph
        return graph.replay, static_in, static_out


class FusedSpikingVGG11(_FusedNetwork):
    def __init__(self, model: SpikingVGG11, T: int, dtype: torch.dtype = torch.bfloat16, device="cuda:0", internal_layouts: bool = False):
        super().__init__(T, dtype, device, internal_layouts=internal_layouts)
        self.steps: List[Tuple[str, object]] = []
        for i, m in enumerate(model.features):
            if isinstance(m, ConvBNNeuron):
                self.steps.append(("conv" if m.sn is not None else "plain", _FusedLayer(m, dtype, self.device_)))
            else:
                self.steps.append(("pool", copy.deepcopy(m)))
        self.tail_lif = model.tail_sn.lif_params
        self.fc_weight = model.fc.weight.detach().to(device=self.device_, dtype=dtype).contiguous()
        self.fc_bias = model.fc.bias.detach().to(device=self.device_, dtype=dtype).contiguous()

    def run(self, x):
        seq: Optional[torch.Tensor] = None          # [T, N, C, H, W] spikes; None while the input is the analog frame
        for i, (kind, item) in enumerate(self.steps):
            if kind == "conv":
                xs = [x] * self.T if seq is None else list(seq.unbind(0))
                seq = self.conv_lif(f"features.{i}", xs, item)
            elif kind == "pool":
                seq = self.pooled(f"features.{i}", seq, item)
            else:
                seq = self.plain_conv(f"features.{i}", seq, item)
        return self.tail(seq, self.tail_lif, self.fc_weight, self.fc_bias)

    def run_blocked(self, x):
        """The same layer sequence with the frame channel-blocked, every spike tensor bit-packed (a 2x2 average pool runs inside
        the convolution in front of it, which then writes blocked quarters instead of bits); the tail's neuron fires in the
        last convolution, and the pool and the classifier read its bit-packed spikes."""
        from .runtime import hip_blocked_backend as B
        seq = B.input_frame(x, self.T)
        skip = False
        for i, (kind, item) in enumerate(self.steps):
            if skip:            # this pool ran inside the convolution in front of it
                skip = False
                continue
            if kind == "conv":
                if i + 1 < len(self.steps) and self.steps[i + 1][0] == "pool":
                    fused = self.conv_lif_pool_b(f"features.{i}", seq, item, f"features.{i + 1}", self.steps[i + 1][1])
                    if fused is not None:
                        seq, skip = fused, True
                        continue
                seq = self.conv_lif_b(f"features.{i}", seq, item)
            elif kind == "pool":
                seq = self.pooled_b(f"features.{i}", seq, item)
            elif i == len(self.steps) - 1:      # the last convolution: the tail's neuron fires in it
                return self.last_conv_and_tail_b(f"features.{i}", seq, item, self.tail_lif, self.fc_weight, self.fc_bias)
            else:
                seq = self.conv_lif_b(f"features.{i}", seq, item, out_layout=B.C8)
        return self.tail(B.to_dense(seq), self.tail_lif, self.fc_weight, self.fc_bias)


class FusedSpikingResNet18(_FusedNetwork):
    def __init__(self, model: SpikingResNet18, T: int, dtype: torch.dtype = torch.bfloat16, device="cuda:0", internal_layouts: bool = False):
        super().__init__(T, dtype, device, internal_layouts=internal_layouts)
        self.stem = _FusedLayer(model.stem, dtype, self.device_)
        self.maxpool = copy.deepcopy(model.maxpool)
        self.block_layers = []
        for b in model.blocks:
            conv2 = _FusedLayer(b.conv2, dtype, self.device_)
            conv2.lif = b.sn2.lif_params if b.sn2 is not None else None
            down = _FusedLayer(b.downsample, dtype, self.device_) if b.downsample is not None else None
            self.block_layers.append((_FusedLayer(b.conv1, dtype, self.device_), conv2, down))
        self.tail_lif = model.tail_sn.lif_params
        self.fc_weight = model.fc.weight.detach().to(device=self.device_, dtype=dtype).contiguous()
        self.fc_bias = model.fc.bias.detach().to(device=self.device_, dtype=dtype).contiguous()

    def run(self, x):
        seq = self.conv_lif("stem", [x] * self.T, self.stem)
        seq = self.pooled("maxpool", seq, self.maxpool)
        for i, (conv1, conv2, down) in enumerate(self.block_layers):
            identity = seq if down is None else self.plain_conv(f"blocks.{i}.downsample", seq, down)
            hidden = self.conv_lif(f"blocks.{i}.conv1", list(seq.unbind(0)), conv1)
            if conv2.lif is not None:
                seq = self.conv_lif(f"blocks.{i}.conv2", list(hidden.unbind(0)), conv2, residuals=list(identity.unbind(0)))
            else:   # last block: its neuron is the tail's
                seq = self.plain_conv(f"blocks.{i}.conv2", hidden, conv2, residual=identity)
        return self.tail(seq, self.tail_lif, self.fc_weight, self.fc_bias)

    def run_blocked(self, x):
        """Stem on the channel-blocked frame, everything after it on bit-packed spikes; a LIF-free shortcut convolution is
        accumulated inside the block's second convolution (or, where that kernel does not take the pair, produces a blocked
        analog residual); the tail's neuron fires in the last block's second convolution, and the pool and the classifier read
        its bit-packed spikes."""
        from .runtime import hip_blocked_backend as B
        frame = B.input_frame(x, self.T)
        seq = self.conv_lif_b("stem", frame, self.stem)
        seq = self.pooled_b("maxpool", seq, self.maxpool)
        for i, (conv1, conv2, down) in enumerate(self.block_layers):
            hidden = self.conv_lif_b(f"blocks.{i}.conv1", seq, conv1)
            if down is not None and conv2.lif is not None:
                fused = self.conv_lif_shortcut_b(f"blocks.{i}.conv2", hidden, conv2, seq, down)
                if fused is not None:
                    seq = fused
                    continue
            identity = seq if down is None else self.conv_lif_b(f"blocks.{i}.downsample", seq, down)
            if conv2.lif is not None:
                seq = self.conv_lif_b(f"blocks.{i}.conv2", hidden, conv2, residual=identity)
            elif i == len(self.block_layers) - 1:   # last block: its neuron is the tail's and fires in this convolution
                return self.last_conv_and_tail_b(f"blocks.{i}.conv2", hidden, conv2, self.tail_lif, self.fc_weight, self.fc_bias, residual=identity)
            else:
                seq = self.conv_lif_b(f"blocks.{i}.conv2", hidden, conv2, residual=identity, out_layout=B.C8)
        return self.tail(B.to_dense(seq), self.tail_lif, self.fc_weight, self.fc_bias)


class FusedSpikingMobileNet(_FusedNetwork):
    """Layer-major execution of `SpikingMobileNet`. Dense form: the depthwise / pointwise / regular `snn_custom` operators.
    Internal form (`internal_layouts=True`): behind the stem the spikes travel row-packed (one byte = 8 consecutive pixels of
    a channel's row), which is what a depthwise lane holds after a LIF step: `snnf_dwconv3x3_lif_rowbits` ->
    `snnf_pwconv_lif_rowbits` -> ... with no dense spike tensor and no membrane written between them. A layer those entry
    points do not take (a stride-2 depthwise layer, rows that are no multiple of 8 pixels, planes that are no multiple of 64
    pixels) runs the dense operator on unpacked spikes and its output is packed again."""

    def __init__(self, model: SpikingMobileNet, T: int, dtype: torch.dtype = torch.bfloat16, device="cuda:0", internal_layouts: bool = False):
        super().__init__(T, dtype, device, internal_layouts=internal_layouts)
        self.layers = [_FusedLayer(m, dtype, self.device_) for m in model.features]
        self.tail_lif = model.tail_sn.lif_params
        self.fc_weight = model.fc.weight.detach().to(device=self.device_, dtype=dtype).contiguous()
        self.fc_bias = model.fc.bias.detach().to(device=self.device_, dtype=dtype).contiguous()

    def run(self, x):
        seq: Optional[torch.Tensor] = None
        for i, layer in enumerate(self.layers):
            if layer.lif is not None:
                xs = [x] * self.T if seq is None else list(seq.unbind(0))
                seq = self.conv_lif(f"features.{i}", xs, layer)
            else:
                seq = self.plain_conv(f"features.{i}", seq, layer)
        return self.tail(seq, self.tail_lif, self.fc_weight, self.fc_bias)

    def run_blocked(self, x):
        from .runtime import hip_blocked_backend as B
        common = lambda lif: lif is not None and float(lif[1]) == 0.0      # hard reset to zero: what the row-packed variants serve
        dense = self.conv_lif("features.0", [x] * self.T, self.layers[0])    # the analog frame goes through the dense operator
        bits = None                                                           # row-packed spikes [T, N, C, H, W / 8], or None
        for i, layer in enumerate(self.layers[1:], start=1):
            name = f"features.{i}"
            if bits is None and dense.shape[-1] % 8 == 0 and layer.lif is not None:
                bits, dense = B.pack_rowbits(dense), None
            depthwise = layer.groups > 1
            took = False
            if bits is not None and common(layer.lif):
                h, w = int(bits.shape[3]), int(bits.shape[4]) * 8
                try:
                    if depthwise and layer.stride == [1, 1]:
                        out, v = B.depthwise_conv_lif_rowbits(bits, layer.weight, layer.bias, layer.lif, want_v=self.record is not None)
                        took = True
                    elif not depthwise and tuple(layer.weight.shape[2:]) == (1, 1) and layer.stride == [1, 1] and (h * w) % 64 == 0:
                        out, v = B.pointwise_conv_lif_from_rowbits(bits, layer.weight, layer.bias, layer.lif, packed_out=True,
                                                                   want_v=self.record is not None)
                        took = True
                except RuntimeError as exc:
                    if "unsupported" not in str(exc):
                        raise
            if took:
                if self.record is not None:
                    self._log(kind="conv_lif", name=name, xs=list(B.unpack_rowbits(bits, self.dtype).unbind(0)), residuals=None, layer=layer,
                              spikes=B.unpack_rowbits(out, self.dtype), v=v, blocked=True)
                bits = out
                continue
            # Dense operators on unpacked spikes (stride-2 depthwise layers, the LIF-free last convolution, odd shapes).
            if dense is None:
                dense = B.unpack_rowbits(bits, self.dtype)
                bits = None
            if layer.lif is not None:
                dense = self.conv_lif(name, list(dense.unbind(0)), layer)
            elif i == len(self.layers) - 1:
                # The last, neuron-free convolution: on channel-packed bits, with the tail's neuron in its epilogue, and the pool
                # and the classifier on its bits.
                return self.last_conv_and_tail_b(name, B.from_dense(dense, B.BITS), layer, self.tail_lif, self.fc_weight, self.fc_bias)
            else:
                dense = self.plain_conv(name, dense, layer)
        if dense is None:
            dense = B.unpack_rowbits(bits, self.dtype)
        return self.tail(dense, self.tail_lif, self.fc_weight, self.fc_bias)


def build_network(name: str, width: int = 64, num_classes: Optional[int] = None, seed: int = 0, gain: float = 1.0) -> nn.Module:
    """`vgg11` (10 classes), `resnet18` (1000 classes) or `mobilenet` (10 classes; `width` 64 is the full network, as for
    the other two) with the synthetic initialisation."""
    if name == "vgg11":
        model = SpikingVGG11(num_classes=10 if num_classes is None else num_classes, width=width)
    elif name == "mobilenet":
        model = SpikingMobileNet(num_classes=10 if num_classes is None else num_classes, width=width // 2)
    elif name == "resnet18":
        model = SpikingResNet18(num_classes=1000 if num_classes is None else num_classes, width=width)
    else:
        raise ValueError(f"unsupported model: {name}")
    return init_synthetic_(model, seed=seed, gain=gain)


def fuse_network(model: nn.Module, T: int, dtype: torch.dtype = torch.bfloat16, device="cuda:0",
                 internal_layouts: bool = False) -> _FusedNetwork:
    """`internal_layouts`: run the network's own operator-to-operator tensors bit-packed / channel-blocked instead of
    through the dense `snn_custom` operators (same operators, same arithmetic; GPU and 16-bit activations only)."""
    if isinstance(model, SpikingVGG11):
        return FusedSpikingVGG11(model, T, dtype, device, internal_layouts)
    if isinstance(model, SpikingResNet18):
        return FusedSpikingResNet18(model, T, dtype, device, internal_layouts)
    if isinstance(model, SpikingMobileNet):
        return FusedSpikingMobileNet(model, T, dtype, device, internal_layouts)
    raise TypeError(f"no fused executor for {type(model).__name__}")
