"""GPU parity of the internal-layout convolution + LIF kernel (`snnf_conv_lif_blocked`) at the sizes the network executors
run it: every conv layer of the spiking ResNet-18 (T=4, B=16, 224x224) and VGG-11 (T=4, B=64, 32x32) configurations at
full size, in the layouts the executors pass (models.py `run_blocked`): the first layer on one channel-blocked analog
frame shared by all timesteps, bit-packed spikes between layers, 2x2 average pools handing over channel-blocked quarters,
bit-packed and channel-blocked residuals, the LIF-free shortcut and pre-tail convolutions. Teacher forced: each layer gets
its own seeded operands, so a near-threshold flip in one layer cannot cascade. Gate: tests/helpers.py:check against the
oracle's dense operator (reference runtime/snn_custom_ops.py:430-453, 491-518). Each case also pins what the planner
selects (kernel family, straight-line epilogue, a single launch window), so that a planner change cannot silently move a
benchmarked layer onto a variant no test has seen.
"""
import pytest
import torch
import torch.nn.functional as F

from helpers import LIF, check, dev, gen, q, spikes
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


@pytest.fixture()
def B(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime import hip_blocked_backend
    from triton_snn_fusion_amd.runtime import hip_convlif_backend
    hip_convlif_backend.clear_packed_weight_cache()
    return hip_blocked_backend


# name, Cin, Cout, input size, kernel, stride, padding, input ("frame": one analog C8 frame for all T, "bits", "quarters":
# C8 averages of 2x2 spikes), residual layout, neuron, output layout
RESNET18 = [
    ("stem", 3, 64, 224, 7, 2, 3, "frame", None, True, "bits"),
    ("l1", 64, 64, 56, 3, 1, 1, "bits", None, True, "bits"), ("l1+res", 64, 64, 56, 3, 1, 1, "bits", "bits", True, "bits"),
    ("l2down", 64, 128, 56, 3, 2, 1, "bits", None, True, "bits"), ("l2short", 64, 128, 56, 1, 2, 0, "bits", None, False, "c8"),
    ("l2+short", 128, 128, 28, 3, 1, 1, "bits", "c8", True, "bits"),
    ("l2", 128, 128, 28, 3, 1, 1, "bits", None, True, "bits"), ("l2+res", 128, 128, 28, 3, 1, 1, "bits", "bits", True, "bits"),
    ("l3down", 128, 256, 28, 3, 2, 1, "bits", None, True, "bits"), ("l3short", 128, 256, 28, 1, 2, 0, "bits", None, False, "c8"),
    ("l3+short", 256, 256, 14, 3, 1, 1, "bits", "c8", True, "bits"),
    ("l3", 256, 256, 14, 3, 1, 1, "bits", None, True, "bits"), ("l3+res", 256, 256, 14, 3, 1, 1, "bits", "bits", True, "bits"),
    ("l4down", 256, 512, 14, 3, 2, 1, "bits", None, True, "bits"), ("l4short", 256, 512, 14, 1, 2, 0, "bits", None, False, "c8"),
    ("l4+short", 512, 512, 7, 3, 1, 1, "bits", "c8", True, "bits"),
    ("l4", 512, 512, 7, 3, 1, 1, "bits", None, True, "bits"),
    ("l4pretail", 512, 512, 7, 3, 1, 1, "bits", "bits", False, "nchw"),
]
VGG11 = [
    ("c1", 3, 64, 32, 3, 1, 1, "frame", None, True, "bits"), ("c2", 64, 128, 16, 3, 1, 1, "quarters", None, True, "bits"),
    ("c3", 128, 256, 8, 3, 1, 1, "quarters", None, True, "bits"), ("c4", 256, 256, 8, 3, 1, 1, "bits", None, True, "bits"),
    ("c5", 256, 512, 4, 3, 1, 1, "quarters", None, True, "bits"), ("c6", 512, 512, 4, 3, 1, 1, "bits", None, True, "bits"),
    ("c7", 512, 512, 2, 3, 1, 1, "quarters", None, True, "bits"), ("c8pretail", 512, 512, 2, 3, 1, 1, "bits", None, False, "nchw"),
    ("c8+tail-neuron", 512, 512, 2, 3, 1, 1, "bits", None, True, "bits"),
]


def _run(B, what, seed, T, N, Cin, Cout, size, k, stride, pad, source, resl, neuron, outl):
    g = gen(seed)
    if source == "frame":
        frame = q(torch.randn(N, Cin, size, size, generator=g), BF16)
        xs = [frame] * T
        x = B.from_dense(dev(frame, BF16), B.C8, shared=True)
        x.T = T
    elif source == "quarters":
        seq = F.avg_pool2d(spikes((T * N, Cin, 2 * size, 2 * size), 0.3, g), 2).reshape(T, N, Cin, size, size)
        xs = [seq[t] for t in range(T)]
        x = B.from_dense(dev(seq, BF16), B.C8)
    else:
        seq = spikes((T, N, Cin, size, size), 0.15, g)
        xs = [seq[t] for t in range(T)]
        x = B.from_dense(dev(seq, BF16), B.BITS)
    gain = 2.0 if source != "quarters" else 3.0
    w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * gain, BF16)
    b = q(torch.randn(Cout, generator=g) * 0.1, BF16)
    out_size = (size + 2 * pad - k) // stride + 1
    rs = res = None
    if resl == "bits":
        rs = spikes((T, N, Cout, out_size, out_size), 0.15, g)
        res = B.from_dense(dev(rs, BF16), B.BITS)
    elif resl == "c8":
        rs = q(torch.randn(T, N, Cout, out_size, out_size, generator=g) * 0.3, BF16)
        res = B.from_dense(dev(rs, BF16), B.C8)
    layouts = {"bits": B.BITS, "c8": B.C8, "nchw": B.NCHW}
    print(f"blocked {what}: {Cin}->{Cout} @{size} k{k} s{stride} N={N} {source}/{resl}/{outl} neuron={neuron}", flush=True)
    out, v = B.conv_lif_blocked(x, dev(w, BF16), dev(b, BF16), [stride, stride], [pad, pad], LIF if neuron else None, residual=res,
                                out_layout=layouts[outl], want_v=neuron)
    torch.cuda.synchronize()
    plan = B.last_conv_plan()
    assert plan["kernel"] == "blocked" and plan["launches"] == 1, plan
    assert plan["window"] == T, plan                                   # all four steps side by side (stems: one frame, T LIF steps)
    assert out.layout == layouts[outl] and out.shape == (T, N, Cout, out_size, out_size)
    if neuron:
        # the straight-line epilogue serves bit-packed outputs with no or a bit-packed residual
        assert (plan["variant"] >= 60) == (resl in (None, "bits")), plan
        ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (stride, stride), (pad, pad), (1, 1), 1, *LIF,
                                  residuals=None if rs is None else [rs[t] for t in range(T)])
        rep = check(B.to_dense(out), v, ref, what=what)
        assert rep["neurons_with_matching_history"] >= 0.999 * rep["neurons"], rep
        rate = float(ref[0].mean())
        assert 0.001 < rate < 0.9, f"{what}: degenerate spike rate {rate}"
        # the same launch without a membrane output (what the executors run) writes the same spikes
        out2, none = B.conv_lif_blocked(x, dev(w, BF16), dev(b, BF16), [stride, stride], [pad, pad], LIF, residual=res,
                                        out_layout=layouts[outl], want_v=False)
        assert none is None
        if size * size <= B.PLANE_MATRIX_MAX_PIXELS and stride == 1 and res is None and outl == "bits":
            # a plane of a few pixels without a membrane output goes through the Linear + LIF kernel as one matrix product per
            # frame: other sums in another order, so it is checked against the oracle and not against the other launch
            plan2 = B.last_conv_plan()
            assert plan2["kernel"] == "plane_matrix" and plan2["x"] == ("bits" if source == "bits" else "c8"), plan2
            assert (plan2["features_in"], plan2["features_out"]) == (Cin * size * size, Cout * size * size), plan2
            rep2 = check(B.to_dense(out2), ref[1], ref, what=what + " as a matrix product")      # spikes only: the oracle's membrane stands in
            assert rep2["neurons_with_matching_history"] >= 0.999 * rep2["neurons"], rep2
        else:
            assert torch.equal(out2.data, out.data)
    else:
        assert v is None
        want = torch.stack([F.conv2d(xs[t], w, b, stride, pad) for t in range(T)])
        if rs is not None:
            want = want + rs
        got = B.to_dense(out).float().cpu()
        assert torch.allclose(got, want, rtol=2 ** -8, atol=1e-3), (got - want).abs().max()      # one rounding to bf16 at the store
    return plan


@pytest.mark.parametrize("name,Cin,Cout,size,k,stride,pad,source,resl,neuron,outl", RESNET18, ids=[c[0] for c in RESNET18])
def test_resnet18_layers_on_the_internal_layouts_at_full_size(B, name, Cin, Cout, size, k, stride, pad, source, resl, neuron, outl):
    plan = _run(B, f"resnet18 {name}", 5000 + Cin + Cout + size + k + len(name), 4, 16, Cin, Cout, size, k, stride, pad, source, resl, neuron, outl)
    tuned = B.get_autotune_best_config(4, 16, Cin, size, size, (Cout, Cin, k, k), [stride, stride], [pad, pad], source == "frame")
    assert (plan["tuned"] != 0) == bool(tuned), (plan, tuned)          # a layer of the measured table runs its entry


@pytest.mark.parametrize("name,Cin,Cout,size,k,stride,pad,source,resl,neuron,outl", VGG11, ids=[c[0] for c in VGG11])
def test_vgg11_layers_on_the_internal_layouts_at_full_size(B, name, Cin, Cout, size, k, stride, pad, source, resl, neuron, outl):
    _run(B, f"vgg11 {name}", 5100 + Cin + Cout + size + k + len(name), 4, 64, Cin, Cout, size, k, stride, pad, source, resl, neuron, outl)
