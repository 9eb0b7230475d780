"""Seeded synthetic workloads for the fused temporal operators, and eval-mode BatchNorm folding.

Every generator draws from a CPU `torch.Generator` seeded with 0, in fp32, and only then rounds to the storage dtype
and moves to the device, so the CPU oracle and the GPU kernels see bit-identical operands.

Workloads (T = timesteps, B = batch):
  conv3x3_block     one Conv3x3(64->64, stride 1, pad 1, no bias) + BN(eval) + LIF, T=4, B=8, 32x32, Bernoulli(0.2) spikes
  linear_block      Linear(2048->1024, bias N(0, 0.01^2)) + LIF, T=8, B=64, Bernoulli(0.1) spikes
  mobilenet_block   depthwise Conv3x3(128) + BN + LIF, then pointwise Conv1x1(128->256) + BN + LIF, T=4, B=32, 56x56,
                    Bernoulli(0.15) spikes
`gain` (default 1) scales the Kaiming weights: with the plain recipe most layers are nearly silent (spike rates of
1e-2 down to 1e-7), so the parity tests also run gain 3, where 7-15 % of the neurons fire every step.
BatchNorm statistics: gamma ~ U(0.8, 1.2), beta ~ N(0, 0.1^2), running_mean ~ N(0, 0.1^2), running_var ~ U(0.5, 1.5),
eps 1e-5. Conv / linear weights are Kaiming-normal (std = sqrt(2 / fan_in)). LIF: tau 2, v_th 1, hard reset to 0.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

LIF_DEFAULT = (1.0, 0.0, 2.0)  # v_threshold, v_reset, tau
BN_EPS = 1e-5


def fold_bn_into_conv_params(conv_weight, conv_bias, running_mean, running_var, bn_weight, bn_bias, eps: float):
    """Folds an eval-mode BatchNorm2d into the preceding convolution (same result as the reference's
    compiler/fx_lif_rewrite.py:340-353): W' = W * g / sqrt(var + eps), b' = (b - mean) * g / sqrt(var + eps) + beta."""
    if conv_bias is None:
        conv_bias = torch.zeros_like(running_mean)
    if bn_weight is None:
        bn_weight = torch.ones_like(running_mean)
    if bn_bias is None:
        bn_bias = torch.zeros_like(running_mean)
    conv_weight = conv_weight.to(dtype=running_mean.dtype)
    conv_bias = conv_bias.to(dtype=running_mean.dtype)
    scale = bn_weight / torch.sqrt(running_var + float(eps))
    return conv_weight * scale.reshape([-1, 1, 1, 1]), (conv_bias - running_mean) * scale + bn_bias


def _generator(seed: int = 0) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def bernoulli_spikes(shape, p: float, g: torch.Generator) -> torch.Tensor:
    return (torch.rand(shape, generator=g) < p).to(torch.float32)


def kaiming_normal(shape, g: torch.Generator) -> torch.Tensor:
    fan_in = 1
    for d in shape[1:]:
        fan_in *= int(d)
    return torch.randn(shape, generator=g) * math.sqrt(2.0 / fan_in)


def bn_statistics(channels: int, g: torch.Generator) -> Dict[str, torch.Tensor]:
    return {
        "weight": torch.rand(channels, generator=g) * 0.4 + 0.8,
        "bias": torch.randn(channels, generator=g) * 0.1,
        "running_mean": torch.randn(channels, generator=g) * 0.1,
        "running_var": torch.rand(channels, generator=g) + 0.5,
    }


def folded_conv_bn(weight: torch.Tensor, g: torch.Generator) -> Tuple[torch.Tensor, torch.Tensor]:
    bn = bn_statistics(int(weight.shape[0]), g)
    return fold_bn_into_conv_params(weight, None, bn["running_mean"], bn["running_var"], bn["weight"], bn["bias"], BN_EPS)


@dataclass
class ConvLayer:
    """One fused Conv+BN+LIF layer: folded fp32 weight/bias on the CPU plus its convolution geometry."""

    weight: torch.Tensor
    bias: torch.Tensor
    stride: Tuple[int, int] = (1, 1)
    padding: Tuple[int, int] = (1, 1)
    groups: int = 1


@dataclass
class Workload:
    name: str
    T: int
    batch: int
    x_seq: torch.Tensor                       # [T, ...] fp32 on the CPU
    conv_layers: List[ConvLayer] = field(default_factory=list)
    linear_weight: Optional[torch.Tensor] = None
    linear_bias: Optional[torch.Tensor] = None
    lif: Tuple[float, float, float] = LIF_DEFAULT


def conv3x3_block(seed: int = 0, T: int = 4, batch: int = 8, channels: int = 64, size: int = 32,
                  gain: float = 1.0) -> Workload:
    g = _generator(seed)
    x = bernoulli_spikes((T, batch, channels, size, size), 0.2, g)
    w, b = folded_conv_bn(kaiming_normal((channels, channels, 3, 3), g) * gain, g)
    return Workload("conv3x3_block", T, batch, x, [ConvLayer(w, b)])


def linear_block(seed: int = 0, T: int = 8, batch: int = 64, fin: int = 2048, fout: int = 1024,
                 gain: float = 1.0) -> Workload:
    g = _generator(seed)
    x = bernoulli_spikes((T, batch, fin), 0.1, g)
    w = kaiming_normal((fout, fin), g) * gain
    b = torch.randn(fout, generator=g) * 0.01
    return Workload("linear_block", T, batch, x, linear_weight=w, linear_bias=b)


def mobilenet_block(seed: int = 0, T: int = 4, batch: int = 32, cin: int = 128, cout: int = 256, size: int = 56,
                    gain: float = 1.0) -> Workload:
    g = _generator(seed)
    x = bernoulli_spikes((T, batch, cin, size, size), 0.15, g)
    dw_w, dw_b = folded_conv_bn(kaiming_normal((cin, 1, 3, 3), g) * gain, g)
    pw_w, pw_b = folded_conv_bn(kaiming_normal((cout, cin, 1, 1), g) * gain, g)
    return Workload("mobilenet_block", T, batch, x,
                    [ConvLayer(dw_w, dw_b, (1, 1), (1, 1), cin), ConvLayer(pw_w, pw_b, (1, 1), (0, 0), 1)])


def algorithmic_conv_bytes(T: int, n: int, cin: int, h: int, w: int, cout: int, ho: int, wo: int, kh: int, kw: int,
                           groups: int, act_bytes: int, v_bytes: int, shared_input: bool = False) -> int:
    """Compulsory traffic of one fused conv+LIF call: read x once, read W and b once, write dense spikes once in the
    activation dtype, write the final membrane once."""
    x_steps = 1 if shared_input else T
    return (x_steps * n * cin * h * w * act_bytes + cout * (cin // groups) * kh * kw * act_bytes + cout * act_bytes
            + T * n * cout * ho * wo * act_bytes + n * cout * ho * wo * v_bytes)


def conv_flops(T: int, n: int, cin: int, cout: int, ho: int, wo: int, kh: int, kw: int, groups: int) -> int:
    return 2 * T * n * ho * wo * cout * (cin // groups) * kh * kw


# The distinct conv(+residual)+LIF layers of the two network configurations (T = 4; ResNet-18 at batch 16 on 224 x 224
# frames, VGG-11 at batch 64 on 32 x 32 frames), as timed layer by layer and as tuned.
# (name, Cin, Cout, input size, kernel, stride, padding, residual added before the LIF, one analog frame for all T, count)
RESNET18_LAYERS = [
    ("stem 7x7/2 3->64", 3, 64, 224, 7, 2, 3, False, True, 1),
    ("3x3 64->64 @56", 64, 64, 56, 3, 1, 1, False, False, 2), ("3x3 64->64 @56 +res", 64, 64, 56, 3, 1, 1, True, False, 2),
    ("3x3/2 64->128 @56", 64, 128, 56, 3, 2, 1, False, False, 1), ("1x1/2 64->128 @56", 64, 128, 56, 1, 2, 0, False, False, 1),
    ("3x3 128->128 @28", 128, 128, 28, 3, 1, 1, False, False, 1), ("3x3 128->128 @28 +res", 128, 128, 28, 3, 1, 1, True, False, 2),
    ("3x3/2 128->256 @28", 128, 256, 28, 3, 2, 1, False, False, 1), ("1x1/2 128->256 @28", 128, 256, 28, 1, 2, 0, False, False, 1),
    ("3x3 256->256 @14", 256, 256, 14, 3, 1, 1, False, False, 1), ("3x3 256->256 @14 +res", 256, 256, 14, 3, 1, 1, True, False, 2),
    ("3x3/2 256->512 @14", 256, 512, 14, 3, 2, 1, False, False, 1), ("1x1/2 256->512 @14", 256, 512, 14, 1, 2, 0, False, False, 1),
    ("3x3 512->512 @7", 512, 512, 7, 3, 1, 1, False, False, 1), ("3x3 512->512 @7 +res", 512, 512, 7, 3, 1, 1, True, False, 2),
]
# The down-sampling blocks of the ResNet-18 configuration as the internal-layout executor runs them: the block's second
# convolution with the 1x1 stride-2 shortcut accumulated in the same launch, in place of one "+res" layer and the shortcut layer.
# (name, the "+res" layer it stands for, the shortcut layer it absorbs, channels, plane size, shortcut channels, shortcut plane size)
RESNET18_SHORTCUT_BLOCKS = [
    ("3x3 128->128 @28 + 1x1/2 64->128 @56", "3x3 128->128 @28 +res", "1x1/2 64->128 @56", 128, 28, 64, 56),
    ("3x3 256->256 @14 + 1x1/2 128->256 @28", "3x3 256->256 @14 +res", "1x1/2 128->256 @28", 256, 14, 128, 28),
    ("3x3 512->512 @7 + 1x1/2 256->512 @14", "3x3 512->512 @7 +res", "1x1/2 256->512 @14", 512, 7, 256, 14),
]
VGG11_LAYERS = [
    ("3x3 3->64 @32", 3, 64, 32, 3, 1, 1, False, True, 1), ("3x3 64->128 @16", 64, 128, 16, 3, 1, 1, False, False, 1),
    ("3x3 128->256 @8", 128, 256, 8, 3, 1, 1, False, False, 1), ("3x3 256->256 @8", 256, 256, 8, 3, 1, 1, False, False, 1),
    ("3x3 256->512 @4", 256, 512, 4, 3, 1, 1, False, False, 1), ("3x3 512->512 @4", 512, 512, 4, 3, 1, 1, False, False, 1),
    ("3x3 512->512 @2", 512, 512, 2, 3, 1, 1, False, False, 2),
]
RESNET18_BATCH = 16
VGG11_BATCH = 64
