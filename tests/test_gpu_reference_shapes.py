"""GPU parity at the sizes the reference itself runs: every fused convolution layer of the spiking ResNet-18 (T=4, B=16,
224x224) and VGG-11 (T=4, B=64, 32x32) configurations at full size, teacher forced (each layer gets its own seeded
spikes, so a near-threshold flip in one layer cannot cascade), and the shapes of the reference's operator
micro-benchmarks (benchmarks/benchmark_temporal_linear_lif_kernel.py:58-63,214; benchmark_temporal_lif_kernel.py:21-26;
benchmark_depthwise_convlif_kernel.py:66-72). Each convolution case also pins the kernel family the planner selects for
that shape, so that a planner change cannot silently move a layer onto a variant no test has seen.
"""
import pytest
import torch

from helpers import DEV, LIF, check, dev, gen, q, spikes, zero_v
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16
S = torch.ops.snn_custom

# name, Cin, Cout, input size, kernel, stride, padding, residual, one analog frame for all T, expected kernel family
RESNET18_LAYERS = [
    ("stem", 3, 64, 224, 7, 2, 3, False, True, "matrix"),
    ("l1", 64, 64, 56, 3, 1, 1, False, False, "matrix"), ("l1res", 64, 64, 56, 3, 1, 1, True, False, "matrix"),
    ("l2down", 64, 128, 56, 3, 2, 1, False, False, "matrix"),
    ("l2", 128, 128, 28, 3, 1, 1, False, False, "matrix"), ("l2res", 128, 128, 28, 3, 1, 1, True, False, "matrix"),
    ("l3down", 128, 256, 28, 3, 2, 1, False, False, "matrix"),
    ("l3", 256, 256, 14, 3, 1, 1, False, False, "matrix"), ("l3res", 256, 256, 14, 3, 1, 1, True, False, "matrix"),
    ("l4down", 256, 512, 14, 3, 2, 1, False, False, "matrix"),
    ("l4", 512, 512, 7, 3, 1, 1, False, False, "matrix"), ("l4res", 512, 512, 7, 3, 1, 1, True, False, "matrix"),
]
VGG11_LAYERS = [
    ("c1", 3, 64, 32, 3, 1, 1, False, True, "matrix"), ("c2", 64, 128, 16, 3, 1, 1, False, False, "matrix"),
    ("c3", 128, 256, 8, 3, 1, 1, False, False, "matrix"), ("c4", 256, 256, 8, 3, 1, 1, False, False, "matrix"),
    ("c5", 256, 512, 4, 3, 1, 1, False, False, "matrix"), ("c6", 512, 512, 4, 3, 1, 1, False, False, "matrix"),
    ("c7", 512, 512, 2, 3, 1, 1, False, False, "matrix"),
]


def _layer_case(seed, T, N, Cin, Cout, size, k, stride, pad, residual, analog, dtype=BF16):
    g = gen(seed)
    if analog:
        frame = q(torch.randn(N, Cin, size, size, generator=g), dtype)
        xs = [frame] * T
    else:
        xs = [spikes((N, Cin, size, size), 0.15, g) for _ in range(T)]
    w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * 2.0, dtype)
    b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    out = (size + 2 * pad - k) // stride + 1
    rs = [spikes((N, Cout, out, out), 0.15, g) for _ in range(T)] if residual else None
    return xs, w, b, rs


def _run_layer(hip_ops, what, xs, w, b, rs, stride, pad, family, dtype=BF16):
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    T = len(xs)
    ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (stride, stride), (pad, pad), (1, 1), 1, *LIF, residuals=rs)
    if xs[0] is xs[-1] and T > 1:
        frame = dev(xs[0], dtype)
        dx = [frame] * T
    else:
        dx = [dev(x, dtype) for x in xs]
    geo = ([stride, stride], [pad, pad], [1, 1], 1)
    if rs is not None:
        sp, v = S.fused_temporal_conv_add_lif_state(dx, [dev(r, dtype) for r in rs], dev(w, dtype), dev(b, dtype), zero_v(), *geo, *LIF, False)
    else:
        sp, v = S.fused_temporal_conv_lif_state(dx, dev(w, dtype), dev(b, dtype), zero_v(), *geo, *LIF, False)
    torch.cuda.synchronize()
    plan = last_conv_plan()
    assert plan["kernel"] == family, plan
    rep = check(sp, v, ref, what=what)
    assert rep["neurons_with_matching_history"] >= 0.999 * rep["neurons"], rep
    rate = float(ref[0].mean())
    assert 0.001 < rate < 0.9, f"{what}: degenerate spike rate {rate}"      # the spiking branch is exercised
    stats = hip_ops.get_fused_op_call_stats()
    assert stats["fallback"] == 0, stats["fallback_reasons"]


@pytest.mark.parametrize("name,Cin,Cout,size,k,stride,pad,residual,analog,family", RESNET18_LAYERS, ids=[l[0] for l in RESNET18_LAYERS])
def test_resnet18_layer_shapes_at_full_size(hip_ops, name, Cin, Cout, size, k, stride, pad, residual, analog, family):
    xs, w, b, rs = _layer_case(2000 + Cin + Cout + size + k, 4, 16, Cin, Cout, size, k, stride, pad, residual, analog)
    _run_layer(hip_ops, f"resnet18 {name}", xs, w, b, rs, stride, pad, family)


@pytest.mark.parametrize("name,Cin,Cout,size,k,stride,pad,residual,analog,family", VGG11_LAYERS, ids=[l[0] for l in VGG11_LAYERS])
def test_vgg11_layer_shapes_at_full_size(hip_ops, name, Cin, Cout, size, k, stride, pad, residual, analog, family):
    xs, w, b, rs = _layer_case(2100 + Cin + Cout + size + k, 4, 64, Cin, Cout, size, k, stride, pad, residual, analog)
    _run_layer(hip_ops, f"vgg11 {name}", xs, w, b, rs, stride, pad, family)


@pytest.mark.parametrize("Cin,Cout,size", [(64, 128, 56), (128, 256, 28), (256, 512, 14)])
def test_resnet18_downsample_shortcuts_at_full_size(hip_ops, Cin, Cout, size):
    """The LIF-free 1x1/2 Conv+BN shortcuts (neuron-free mode of the matrix kernel) against F.conv2d."""
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan, run_hip_temporal_conv_bias
    xs, w, b, _ = _layer_case(2200 + Cin, 4, 16, Cin, Cout, size, 1, 2, 0, False, False)
    want = torch.stack([torch.nn.functional.conv2d(x, w, b, 2, 0) for x in xs])
    got = run_hip_temporal_conv_bias([dev(x, BF16) for x in xs], dev(w, BF16), dev(b, BF16), [2, 2], [0, 0])
    assert last_conv_plan()["kernel"] == "matrix"
    assert torch.allclose(got.float().cpu(), want, rtol=2 ** -8, atol=1e-3), (got.float().cpu() - want).abs().max()


# ---------------------------------------------------------------------------------------------------------------
# The reference's operator micro-benchmarks
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [1, 4, 16])
@pytest.mark.parametrize("Fin,Fout", [(512, 512), (1024, 512), (4096, 4096), (4096, 1000), (25088, 4096)])
def test_linear_lif_at_the_reference_benchmark_shapes(hip_ops, Fin, Fout, batch):
    """benchmarks/benchmark_temporal_linear_lif_kernel.py:58-63,214: analog inputs N(0, 0.04^2), weights N(0, 0.02^2) (scaled
    up here so that neurons fire), bias N(0, 0.01^2), a full-shape zero v_init, T = 4; list and packed forms."""
    T = 4
    g = gen(2026 + T + batch + Fin + Fout)
    x = q(torch.randn(T, batch, Fin, generator=g) * 0.04, BF16)
    w = q(torch.randn(Fout, Fin, generator=g) * 0.02 * (60.0 * (512.0 / Fin) ** 0.5), BF16)
    b = q(torch.randn(Fout, generator=g) * 0.01, BF16)
    v0 = torch.zeros(batch, Fout)
    ref = O.temporal_linear_lif(x, w, b, v0, *LIF)
    dx, dw, db, dv = dev(x, BF16), dev(w, BF16), dev(b, BF16), dev(v0, F32)
    s, v = S.fused_temporal_linear_lif_state_packed(dx, dw, db, dv, *LIF, False)
    check(s, v, ref, what=f"linear {Fin}->{Fout} batch {batch}")
    assert 0.001 < float(ref[0].mean()) < 0.9
    s_l, v_l = S.fused_temporal_linear_lif_state([dx[t] for t in range(T)], dw, db, dv, *LIF, False)
    assert torch.equal(s_l, s) and torch.equal(v_l, v)
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0


@pytest.mark.parametrize("T", [1, 4, 16])
@pytest.mark.parametrize("shape", [(16, 64, 56, 56), (16, 128, 28, 28), (16, 256, 14, 14), (16, 512, 7, 7)])
def test_temporal_lif_and_tail_at_the_reference_benchmark_shapes(hip_ops, shape, T):
    """benchmarks/benchmark_temporal_lif_kernel.py:21-26 (RESNET_LIKE_SHAPES), fp16 as there: the scan is bit exact, the
    tail's logits within the fp16 tier of the reference's tolerances (2e-3)."""
    g = gen(2300 + shape[1] + T)
    x = q(torch.randn((T,) + shape, generator=g) * 0.75 + 0.15, F16)
    ref = O.temporal_lif(x, torch.tensor(0.0), *LIF)
    s, v = S.fused_temporal_lif_state(dev(x, F16), zero_v(F16), *LIF, False)
    assert torch.equal(s.float().cpu(), ref[0])
    check(s, v, ref, v_dtype=F16, what=f"lif scan {shape} T={T}")
    K = 1000
    w = q(torch.randn(K, shape[1], generator=g) * 0.05, F16)
    b = q(torch.randn(K, generator=g) * 0.05, F16)
    ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(x, torch.tensor(0.0), w, b, *LIF)
    out, vt = S.fused_temporal_lif_avgpool_linear(dev(x, F16), zero_v(F32), dev(w, F16), dev(b, F16), *LIF, False)
    assert torch.equal(vt.cpu(), ref_v)
    assert torch.allclose(out.float().cpu(), ref_out, rtol=2e-3, atol=2e-3 * max(1.0, T / 4)), (out.float().cpu() - ref_out).abs().max()
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0


@pytest.mark.parametrize("dtype", [F16, F32])
@pytest.mark.parametrize("stride", [1, 2])
def test_depthwise_at_the_reference_benchmark_shape(hip_ops, stride, dtype):
    """benchmarks/benchmark_depthwise_convlif_kernel.py:66-72: T=4, N=2, C=64, 64x64, a 0-dim tensor as v_init; operands
    scaled up from the benchmark's N(0, 0.03^2) so that neurons fire."""
    T, N, C, H = 4, 2, 64, 64
    g = gen(2026 + stride + T + C)
    x = q(torch.randn(T, N, C, H, H, generator=g) * 0.9, dtype)
    w = q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, dtype)
    b = q(torch.randn(C, generator=g) * 0.03, dtype)
    ref = O.temporal_conv_lif([x[t] for t in range(T)], w, b, torch.tensor(0.0), (stride, stride), (1, 1), (1, 1), C, *LIF)
    dx = dev(x, dtype)
    s, v = S.fused_temporal_depthwise_conv_lif_state([dx[t] for t in range(T)], dev(w, dtype), dev(b, dtype),
                                                     torch.tensor(0.0, device=DEV, dtype=dtype), [stride, stride], [1, 1], [1, 1], C, *LIF, False)
    assert s.dtype == dtype and v.dtype == dtype
    check(s, v, ref, v_dtype=dtype, what=f"depthwise benchmark shape s{stride}")
    assert 0.001 < float(ref[0].mean()) < 0.9
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0
