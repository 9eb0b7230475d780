"""Spiking VGG-11 / ResNet-18 harness: eager single-step form (CPU) and fused temporal form (GPU).

CPU tests pin the eager form: wrapper semantics (T identical frames, sum / T, state reset), BatchNorm folding, and one
Conv+BN+neuron module stepped T times against the oracle's temporal operator. GPU tests check the fused form operator by
operator against the oracle on the operator's own inputs (so a near-threshold flip in one layer does not cascade into
false alarms downstream), against the eager form end to end, and under HIP graph replay.
"""
import pytest
import torch
import torch.nn.functional as F

from helpers import DEV, check, gen, q
from oracle import snn_oracle as O
from triton_snn_fusion_amd import models as M

BF16, F32 = torch.bfloat16, torch.float32
SMALL = {"vgg11": dict(width=16, size=32, batch=3), "resnet18": dict(width=16, size=64, batch=2)}


def _frame(name, seed=5):
    cfg = SMALL[name]
    return q(torch.randn(cfg["batch"], 3, cfg["size"], cfg["size"], generator=gen(seed)), BF16)


# ---------------------------------------------------------------------------------------------------------------
# Eager form (CPU)
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_single_step_loop_wrapper_and_state_reset(name):
    model = M.build_network(name, width=8, gain=5.0)
    x = torch.randn(2, 3, 32, 32, generator=gen(1))
    T = 4
    with torch.no_grad():
        M.reset_lif_modules(model)
        per_step = [model(x) for _ in range(T)]                 # the state lives in the neuron modules
        M.reset_lif_modules(model)
        y = M.SingleStepModeLoopWrapper(model, T)(x)
        y_stale = M.SingleStepModeLoopWrapper(model, T)(x)      # no reset: continues from the last membrane
        M.reset_lif_modules(model)
        y_again = M.SingleStepModeLoopWrapper(model, T)(x)
    assert torch.allclose(y, sum(per_step) / T, rtol=0, atol=1e-6)
    assert not torch.equal(per_step[0], per_step[1])
    assert torch.equal(y, y_again) and not torch.equal(y, y_stale)
    neurons = [m for m in model.modules() if isinstance(m, M.CustomStatefulIFNode)]
    assert len(neurons) == (8 if name == "vgg11" else 17)
    assert all(n.v.dim() == 4 for n in neurons)
    M.reset_lif_modules(model)
    assert all(n.v.dim() == 0 for n in neurons)


@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_batchnorm_folding_keeps_the_network_function(name):
    model = M.build_network(name, width=8, gain=5.0)
    folded = M.fold_batchnorm(model)
    assert not any(isinstance(m, torch.nn.BatchNorm2d) for m in folded.modules())
    x = torch.randn(2, 3, 32, 32, generator=gen(2))
    with torch.no_grad():
        block, fblock = (model.features[0], folded.features[0]) if name == "vgg11" else (model.stem, folded.stem)
        pre = block.bn(block.conv(x))
        assert torch.allclose(fblock.conv(x), pre, rtol=1e-5, atol=1e-5)
        M.reset_lif_modules(model)
        y = M.SingleStepModeLoopWrapper(model, 3)(x)
        y_f = M.SingleStepModeLoopWrapper(folded, 3)(x)
    assert torch.allclose(y, y_f, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fused_operator_sequence_is_the_eager_network_exactly_on_cpu(name):
    """Wiring: on CPU tensors the snn_custom operators evaluate the eager formulas, so the layer-major fused form and the
    time-major single-step form run the same fp32 arithmetic in a different order of calls and must agree exactly."""
    T = 4
    model = M.fold_batchnorm(M.build_network(name, width=16, gain=5.0))
    x = torch.randn(2, 3, 64 if name == "resnet18" else 32, 64 if name == "resnet18" else 32, generator=gen(3))
    with torch.no_grad():
        want = M.SingleStepModeLoopWrapper(model, T)(x)
    fused = M.fuse_network(model, T, F32, "cpu")
    fused.record = []
    got = fused(x)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6), float((got - want).abs().max())
    kinds = [e["kind"] for e in fused.record]
    if name == "vgg11":
        assert kinds == ["conv_lif", "pool", "conv_lif", "pool", "conv_lif", "conv_lif", "pool", "conv_lif", "conv_lif", "pool",
                         "conv_lif", "plain_conv", "tail"]
    else:
        assert kinds.count("conv_lif") == 16 and kinds.count("plain_conv") == 4 and kinds[-2:] == ["plain_conv", "tail"]
        assert sum(e["kind"] == "conv_lif" and e["residuals"] is not None for e in fused.record) == 7


def test_conv_bn_neuron_module_stepped_T_times_is_the_temporal_operator():
    m = M.init_synthetic_(M.ConvBNNeuron(6, 10, 3, 2, 1), seed=3, gain=5.0)
    xs = [torch.randn(2, 6, 9, 9, generator=gen(10 + t)) for t in range(5)]
    with torch.no_grad():
        got = torch.stack([m(x) for x in xs])
    w, b = O.fold_bn(m.conv.weight, None, m.bn.running_mean, m.bn.running_var, m.bn.weight, m.bn.bias, m.bn.eps)
    ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (2, 2), (1, 1), (1, 1), 1, *m.sn.lif_params)
    rep = O.parity_report(got, m.sn.v, ref[0], ref[1], ref[2], 1.0, rtol=1e-3, atol=1e-4)
    O.assert_parity(rep, what="ConvBNNeuron")


def test_network_shapes_follow_the_benchmark_configurations():
    vgg = M.build_network("vgg11")
    convs = [m for m in vgg.features if isinstance(m, M.ConvBNNeuron)]
    assert [c.conv.out_channels for c in convs] == [64, 128, 256, 256, 512, 512, 512, 512]
    assert sum(isinstance(m, torch.nn.AvgPool2d) for m in vgg.features) == 4 and vgg.fc.weight.shape == (10, 512)
    res = M.build_network("resnet18")
    assert res.stem.conv.kernel_size == (7, 7) and res.stem.conv.stride == (2, 2) and len(res.blocks) == 8
    assert [b.conv1.conv.out_channels for b in res.blocks] == [64, 64, 128, 128, 256, 256, 512, 512]
    assert [b.downsample is not None for b in res.blocks] == [False, False, True, False, True, False, True, False]
    assert res.fc.weight.shape == (1000, 512) and res.blocks[-1].sn2 is None


# ---------------------------------------------------------------------------------------------------------------
# Fused form (GPU)
# ---------------------------------------------------------------------------------------------------------------
def _fused(name, T=4, gain=5.0):
    model = M.build_network(name, width=SMALL[name]["width"], gain=gain)
    return model, M.fuse_network(model, T, BF16, DEV)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fused_network_operator_by_operator_against_the_oracle(hip_ops, name):
    T = 4
    model, fused = _fused(name, T)
    fused.record = []
    out = fused(_frame(name))
    torch.cuda.synchronize()
    kinds = [e["kind"] for e in fused.record]
    assert kinds.count("conv_lif") == (7 if name == "vgg11" else 16) and kinds.count("tail") == 1
    active = 0
    for e in fused.record:
        if e["kind"] == "conv_lif":
            L = e["layer"]
            xs = [x.float().cpu() for x in e["xs"]]
            rs = None if e["residuals"] is None else [r.float().cpu() for r in e["residuals"]]
            ref = O.temporal_conv_lif(xs, L.weight.float().cpu(), L.bias.float().cpu(), torch.tensor(0.0), tuple(L.stride),
                                      tuple(L.padding), (1, 1), 1, *L.lif, residuals=rs)
            check(e["spikes"], e["v"], ref, what=f"{name} {e['name']}")
            active += int(ref[0].mean() > 0.01)
        elif e["kind"] == "plain_conv":
            L = e["layer"]
            ref = F.conv2d(e["x"].float().cpu().flatten(0, 1), L.weight.float().cpu(), L.bias.float().cpu(), L.stride, L.padding)
            if e["residual"] is not None:
                ref = ref + e["residual"].float().cpu().flatten(0, 1)
            assert e["native"], e["name"]
            # fp32 accumulation, one rounding to bf16 on the way out
            assert torch.allclose(e["y"].float().cpu().flatten(0, 1), ref, rtol=2 ** -8, atol=1e-3), e["name"]
        elif e["kind"] == "pool":
            ref = e["pool"](e["x"].float().cpu().flatten(0, 1))
            assert torch.equal(e["y"].float().cpu().flatten(0, 1), ref), e["name"]      # spikes: exact in bf16
        elif e["kind"] == "tail":
            ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(e["x"].float().cpu(), torch.tensor(0.0), e["fc_weight"].float().cpu(),
                                                                 e["fc_bias"].float().cpu(), *e["lif"])
            assert torch.equal(e["v"].cpu(), ref_v)
            assert torch.allclose(e["out_sum"].float().cpu(), ref_out, rtol=8e-3, atol=8e-3)
            assert torch.allclose(out.float().cpu(), ref_out / T, rtol=8e-3, atol=8e-3)
    assert active >= 5, "the test network is nearly silent"
    stats = hip_ops.get_fused_op_call_stats()
    assert stats["fallback"] == 0 and stats["triton"] == kinds.count("conv_lif") + 1, stats


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fused_network_tracks_the_eager_network(hip_ops, name):
    """End to end on the GPU. Summation order differs between the two forms, so a few neurons within rounding distance
    of the threshold flip, and with random weights every flipped spike flips more downstream: exact agreement holds
    for the first layer and decays with depth (the wiring itself is pinned exactly by the CPU test above, every
    operator by the oracle test). The logits must still point the same way."""
    T = 4
    model, fused = _fused(name, T)
    x = _frame(name)
    eager = M.fold_batchnorm(model, round_to=BF16)
    first = eager.features[0] if name == "vgg11" else eager.stem
    first_spikes = []
    first.register_forward_hook(lambda _m, _i, o: first_spikes.append(o.clone()))
    M.reset_lif_modules(eager)
    with torch.no_grad():
        want = M.SingleStepModeLoopWrapper(eager, T)(x)
    fused.record = []
    got = fused(x).float().cpu()
    mismatch = (fused.record[0]["spikes"].float().cpu() != torch.stack(first_spikes)).float().mean()
    assert float(mismatch) <= 1e-4, float(mismatch)
    cos = float(F.cosine_similarity(got.flatten(), want.flatten(), dim=0))
    print(f"{name}: cosine similarity of the logits {cos:.4f}")
    assert cos > 0.8, cos


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fused_network_graph_replay_matches_eager_launches(hip_ops, name):
    T = 4
    _, fused = _fused(name, T)
    frames = [_frame(name, seed=20 + i) for i in range(3)]
    replay, static_in, static_out = fused.capture(frames[0])
    for f in frames + [frames[0]]:
        want = fused(f).clone()                 # eager launches between the replays
        torch.cuda.synchronize()
        static_in.copy_(f.to(DEV, BF16))
        replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, want)
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0
