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
from triton_snn_fusion_amd import fx_temporal_rewrite as R
from triton_snn_fusion_amd import models as M

BF16, F32 = torch.bfloat16, torch.float32
SMALL = {"vgg11": dict(width=16, size=32, batch=3), "resnet18": dict(width=16, size=64, batch=2), "mobilenet": dict(width=32, size=64, batch=2)}
NEURONS = {"vgg11": 8, "resnet18": 17, "mobilenet": 9}          # neuron modules = fused layers incl. the tail


def _frame(name, seed=5):
    cfg = SMALL[name]
    return q(torch.randn(cfg["batch"], 3, cfg["size"], cfg["size"], generator=gen(seed)), BF16)


# ---------------------------------------------------------------------------------------------------------------
# Eager form (CPU)
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
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
    assert len(neurons) == NEURONS[name]
    assert all(n.v.dim() == 4 for n in neurons)
    M.reset_lif_modules(model)
    assert all(n.v.dim() == 0 for n in neurons)


@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
def test_batchnorm_folding_keeps_the_network_function(name):
    model = M.build_network(name, width=8, gain=5.0)
    folded = M.fold_batchnorm(model)
    assert not any(isinstance(m, torch.nn.BatchNorm2d) for m in folded.modules())
    x = torch.randn(2, 3, 32, 32, generator=gen(2))
    with torch.no_grad():
        block, fblock = (model.stem, folded.stem) if name == "resnet18" else (model.features[0], folded.features[0])
        pre = block.bn(block.conv(x))
        assert torch.allclose(fblock.conv(x), pre, rtol=1e-5, atol=1e-5)
        M.reset_lif_modules(model)
        y = M.SingleStepModeLoopWrapper(model, 3)(x)
        y_f = M.SingleStepModeLoopWrapper(folded, 3)(x)
    assert torch.allclose(y, y_f, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
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
    elif name == "mobilenet":
        assert kinds == ["conv_lif"] * 8 + ["plain_conv", "tail"]
        assert [e["layer"].groups > 1 for e in fused.record[:8]] == [False, True, False, True, False, True, False, True]
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
# FX temporal rewrite (CPU: the snn_custom operators evaluate the eager formulas there)
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("tail_first", [False, True])
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_rewrite_graph_invariants_and_numerical_equality(name, tail_first):
    T = 4
    model = M.build_network(name, width=16, gain=5.0)
    wrapper = M.SingleStepModeLoopWrapper(model, T)
    x = torch.randn(2, 3, 64 if name == "resnet18" else 32, 64 if name == "resnet18" else 32, generator=gen(4))
    with torch.no_grad():
        want = wrapper(x)
    traced = R.trace_single_step_loop(wrapper)
    lifs = [n for n in traced.graph.nodes if R.is_custom_lif_state_node(n)]
    assert len(lifs) == T * (8 if name == "vgg11" else 17)
    assert all(n.v.dim() == 0 for n in model.modules() if isinstance(n, M.CustomStatefulIFNode))     # tracing left no proxies behind
    gm, stats = R.compile_temporal(wrapper, tail_first=tail_first, batch_time=False)
    S = torch.ops.snn_custom
    targets = [n.target for n in gm.graph.nodes if n.op == "call_function"]
    n_conv = sum(t in (S.fused_temporal_conv_lif_state, S.fused_temporal_pointwise_conv_lif_state) for t in targets)
    n_res = targets.count(S.fused_temporal_conv_add_lif_state)
    n_tail = targets.count(S.fused_temporal_lif_avgpool_linear)
    assert not any(R.is_custom_lif_state_node(n) for n in gm.graph.nodes), "every neuron call is inside a fused operator"
    if name == "vgg11":
        assert (n_conv, n_res, n_tail) == ((7, 0, 1) if tail_first else (8, 0, 0))
    else:
        assert (n_conv, n_res, n_tail) == ((9, 7, 1) if tail_first else (9, 8, 0))
    assert stats.replaced_patterns == T * (8 if name == "vgg11" else 17) and not stats.skipped
    # fused layers have no per-timestep Conv2d / BatchNorm2d calls left; LIF-free ones are called once per timestep
    convs = [n for n in gm.graph.nodes if n.op == "call_module" and isinstance(gm.get_submodule(n.target), torch.nn.Conv2d)]
    assert len(convs) == T * ({"vgg11": 0, "resnet18": 3}[name] + (1 if tail_first else 0))
    # every fused operator takes its T inputs as a list of T nodes and starts from the scalar-zero membrane
    for n in gm.graph.nodes:
        if n.op == "call_function" and n.target in (S.fused_temporal_conv_lif_state, S.fused_temporal_conv_add_lif_state):
            assert isinstance(n.args[0], (list, tuple)) and len(n.args[0]) == T
            v0 = n.args[4] if n.target is S.fused_temporal_conv_add_lif_state else n.args[3]
            assert v0.op == "get_attr" and getattr(gm, v0.target).dim() == 0
    with torch.no_grad():
        got = gm(x)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5), float((got - want).abs().max())
    # Stateless layers batched over time: one call each instead of T, same result.
    removed = R.batch_timestep_calls(gm)
    modules = [n for n in gm.graph.nodes if n.op == "call_module"]
    assert len(modules) == len({n.target for n in modules}), "every remaining layer is called once"
    assert removed > 0 and removed % T == 0
    functions = [n.target for n in gm.graph.nodes if n.op == "call_function"]
    assert functions.count(R.pooled_frames) == (4 if name == "vgg11" else 1)                       # one call per pooling layer
    assert functions.count(R.conv_bias_frames) == (3 if name == "resnet18" else 0) + (1 if tail_first else 0)   # LIF-free Conv+BN, folded
    assert not any(isinstance(gm.get_submodule(n.target), (torch.nn.Conv2d, torch.nn.BatchNorm2d)) for n in modules)
    assert not any(n.op == "call_function" and n.target is torch.stack for n in gm.graph.nodes)
    with torch.no_grad():
        again = gm(x)
    assert torch.allclose(again, want, rtol=1e-4, atol=1e-5), float((again - want).abs().max())


def test_fx_rewrite_leaves_a_layer_alone_when_its_state_chain_is_broken():
    """A neuron whose membrane is read between the steps (here: exported by the module) must not be fused."""
    class Leaky(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.block = M.init_synthetic_(M.ConvBNNeuron(4, 8, 3, 1, 1), gain=5.0)

        def forward(self, x):
            a = self.block(x)
            peek = self.block.sn.v          # the intermediate membrane escapes
            b = self.block(x)
            return a + b + peek.mean()

    module = Leaky()
    gm, stats = R.compile_temporal(module)
    assert stats.replaced_patterns == 0 and len(stats.skipped) == 1 and "other users" in stats.skipped[0]
    x = torch.randn(1, 4, 6, 6, generator=gen(8))
    M.reset_lif_modules(module)
    with torch.no_grad():
        want = module(x)
        M.reset_lif_modules(module)
        assert torch.allclose(gm(x), want)


class _EncoderMlp(torch.nn.Module):
    """A neuron on the analog frame (no layer in front), one Conv+BN+neuron, then two Linear+neuron layers and a Linear
    readout: the Linear -> LIF and standalone LIF pattern families next to the convolution one."""

    def __init__(self):
        super().__init__()
        self.enc = M.CustomStatefulIFNode(v_threshold=0.5)
        self.conv = M.ConvBNNeuron(3, 8, 3, 2, 1)
        self.fc1, self.sn1 = torch.nn.Linear(8 * 4 * 4, 32), M.CustomStatefulIFNode()
        self.fc2, self.sn2 = torch.nn.Linear(32, 16, bias=False), M.CustomStatefulIFNode(v_reset=-1.0)
        self.head = torch.nn.Linear(16, 5)

    def forward(self, x):
        y = torch.flatten(self.conv(self.enc(x)), 1)
        return self.head(self.sn2(self.fc2(self.sn1(self.fc1(y)))))


@pytest.mark.parametrize("window", [None, 2])
def test_fx_rewrite_linear_lif_and_standalone_lif_pattern_families(window):
    T = 4
    net = M.init_synthetic_(_EncoderMlp(), gain=4.0)
    wrapper = M.SingleStepModeLoopWrapper(net, T)
    x = torch.randn(3, 3, 8, 8, generator=gen(11))
    with torch.no_grad():
        want = wrapper(x)
    gm, stats = R.compile_temporal(wrapper, window=window)
    S = torch.ops.snn_custom
    targets = [n.target for n in gm.graph.nodes if n.op == "call_function"]
    per_layer = 1 if window is None else T // window
    assert targets.count(S.fused_temporal_lif_state) == per_layer and stats.temporal_lif_groups == 1
    assert targets.count(S.fused_temporal_linear_lif_state) == 2 * per_layer and stats.temporal_linear_lif_groups == 2
    assert targets.count(S.fused_temporal_conv_lif_state) == per_layer and stats.temporal_conv_bn_lif_groups == 1
    assert stats.temporal_windows == 4 * per_layer and stats.replaced_patterns == 4 * T and not stats.skipped
    assert not any(R.is_custom_lif_state_node(n) for n in gm.graph.nodes)
    # the encoder reads one frame T times: its stack is built from the placeholder; the Linear layers take lists of T nodes
    for n in gm.graph.nodes:
        if n.op == "call_function" and n.target is S.fused_temporal_linear_lif_state:
            assert isinstance(n.args[0], (list, tuple)) and len(n.args[0]) == (T if window is None else window)
            assert n.args[2] is None or n.args[2].op == "get_attr"                   # the bias-free layer passes None
    # windows chain through the final membrane: every window after a layer's first starts from the previous one's second output
    fused = [n for n in gm.graph.nodes if n.op == "call_function" and n.target in
             (S.fused_temporal_lif_state, S.fused_temporal_linear_lif_state, S.fused_temporal_conv_lif_state)]
    from_zero = [n for n in fused if any(isinstance(a, torch.fx.Node) and a.op == "get_attr" and "zero_membrane" in a.target for a in n.args)]
    assert len(from_zero) == 4 and len(fused) - len(from_zero) == 4 * (per_layer - 1)
    with torch.no_grad():
        got = gm(x)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5), float((got - want).abs().max())
    assert float(want.abs().max()) > 0.01


@pytest.mark.parametrize("T,window,allow_tail,fused_per_layer,single_steps", [(4, 2, True, 2, 0), (5, 3, True, 2, 0), (5, 3, False, 1, 2),
                                                                           (5, 2, True, 2, 1), (4, 4, True, 1, 0)])
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_rewrite_temporal_windows_shorter_than_T(name, T, window, allow_tail, fused_per_layer, single_steps):
    """Windows of `window` steps: every window is one fused node, the next window (or a step that stayed a single-step
    neuron call) continues from its final membrane; the result equals the eager T-step loop."""
    model = M.build_network(name, width=8, gain=5.0)
    wrapper = M.SingleStepModeLoopWrapper(model, T)
    size = 32
    x = torch.randn(2, 3, size, size, generator=gen(12))
    with torch.no_grad():
        want = wrapper(x)
    gm, stats = R.compile_temporal(wrapper, tail_first=True, window=window, allow_tail=allow_tail)
    S = torch.ops.snn_custom
    targets = [n.target for n in gm.graph.nodes if n.op == "call_function"]
    layers = 8 if name == "vgg11" else 17
    n_fused = sum(t in (S.fused_temporal_conv_lif_state, S.fused_temporal_conv_add_lif_state, S.fused_temporal_lif_avgpool_linear) for t in targets)
    assert n_fused == layers * fused_per_layer == stats.temporal_windows and not stats.skipped
    left = sum(R.is_custom_lif_state_node(n) for n in gm.graph.nodes)
    assert left == layers * single_steps
    with torch.no_grad():
        got = gm(x)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5), float((got - want).abs().max())


@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_layout_propagation_graph_invariants(name):
    """compile_temporal(internal_layouts=True): every fused convolution, LIF-free convolution and pool of the rewritten graph
    calls an internal-layout entry point on `Blocked` values; dense tensors exist at the input (one conversion of the
    shared frame) and in front of the tail operator (one conversion, of a tensor the last convolution wrote dense)."""
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B
    T = 4
    model = M.build_network(name, width=16, gain=5.0)
    gm, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, internal_layouts=True)
    S = torch.ops.snn_custom
    calls = [n for n in gm.graph.nodes if n.op == "call_function"]
    targets = [n.target for n in calls]
    n_conv, n_pool = (7, 4) if name == "vgg11" else (19, 1)      # without the last convolution, which is part of the tail's node
    n_shortcut = 0 if name == "vgg11" else 3      # 1x1 shortcut convolutions folded into the convolution they are added to
    n_pooled = 4 if name == "vgg11" else 0        # 2x2 average pools folded into the convolution in front of them
    assert targets.count(R.blocked_conv_lif) == n_conv - 2 * n_shortcut - n_pooled and targets.count(R.blocked_conv_lif_shortcut) == n_shortcut
    assert targets.count(R.blocked_pool) == n_pool - n_pooled and targets.count(R.blocked_conv_lif_avgpool) == n_pooled
    assert stats.internal_layout_nodes == n_conv + 1 - n_shortcut + n_pool - n_pooled and not stats.skipped
    # the last convolution, the tail's neuron, the pool, the classifier and the mean over T are one node: nothing leaves the layouts
    assert targets.count(R.blocked_input) == 1 and targets.count(R.blocked_to_dense) == 0 and targets.count(R.blocked_residual) == 0
    assert targets.count(S.fused_temporal_lif_avgpool_linear) == 0 and targets.count(R.blocked_conv_lif_pool_linear) == 1
    assert next(n for n in gm.graph.nodes if n.op == "output").args[0].target is R.blocked_conv_lif_pool_linear
    dense_ops = (S.fused_temporal_conv_lif_state, S.fused_temporal_conv_add_lif_state, R.pooled_frames, R.conv_bias_frames)
    assert not any(t in dense_ops for t in targets) and not any(n.op == "call_module" for n in gm.graph.nodes)
    first = next(n for n in calls if n.target is R.blocked_input)
    assert first.args[0].op == "placeholder" and first.args[1:] == (T, True)          # one shared analog frame
    convs = [n for n in calls if n.target is R.blocked_conv_lif]
    # layouts: every spike tensor leaves bit-packed; no LIF-free convolution is left
    assert all(n.args[5] is not None and n.args[7] == B.BITS for n in convs)
    tail = next(n for n in calls if n.target is R.blocked_conv_lif_pool_linear)
    assert tail.args[5] == (1.0, 0.0, 2.0) and tail.args[9] == 1.0 / T
    produced = (R.blocked_conv_lif, R.blocked_conv_lif_shortcut, R.blocked_conv_lif_avgpool, R.blocked_pool)
    if name == "resnet18":
        # residuals: the block input itself (bits) for plain blocks; a down-sampling block's shortcut convolution is part of
        # the node of its second convolution, which reads the block input (the shortcut's operand) and the first convolution's spikes
        with_res = [n for n in convs if n.args[6] is not None]
        assert len(with_res) == 4 and all(n.args[6].target in produced for n in with_res)
        assert tail.args[6] is not None and tail.args[6].target in produced              # the pre-tail sum is the convolution's residual
        for n in (c for c in calls if c.target is R.blocked_conv_lif_shortcut):
            first_conv = n.args[0]
            assert first_conv.target is R.blocked_conv_lif and first_conv.args[0] is n.args[5] and n.args[9] == B.BITS
            assert list(n.args[8]) == [2, 2] and list(first_conv.args[3]) == [2, 2]
    # every operand of a converted node is another converted node (or the input conversion): no dense hop in between
    for n in convs + [c for c in calls if c.target in (R.blocked_pool, R.blocked_conv_lif_shortcut, R.blocked_conv_lif_avgpool, R.blocked_conv_lif_pool_linear)]:
        assert n.args[0].target in produced + (R.blocked_input,)


def test_fx_layout_propagation_keeps_dense_tensors_around_nodes_it_does_not_know():
    """A stateless layer the pass has no kernel for (here a Hardtanh between two fused layers) reads a dense tensor and hands
    one on: the graph converts once on either side of it."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = M.ConvBNNeuron(3, 16, 3, 1, 1)
            self.clip = torch.nn.Hardtanh(0.0, 0.5)
            self.b = M.ConvBNNeuron(16, 16, 3, 1, 1)
            self.c = M.ConvBNNeuron(16, 16, 3, 1, 1)

        def forward(self, x):
            return self.c(self.b(self.clip(self.a(x)))).mean((2, 3))

    net = M.init_synthetic_(Net(), gain=5.0)
    gm, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(net, 4), internal_layouts=True)
    targets = [n.target for n in gm.graph.nodes if n.op == "call_function"]
    assert targets.count(R.blocked_conv_lif) == 3 and stats.internal_layout_nodes == 3
    assert targets.count(R.blocked_input) == 2 and targets.count(R.blocked_to_dense) == 2
    convs = [n for n in gm.graph.nodes if n.op == "call_function" and n.target is R.blocked_conv_lif]
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B
    assert [n.args[7] for n in convs] == [B.NCHW, B.BITS, B.NCHW]       # only the b -> c hand-over stays inside the layouts
    assert convs[2].args[0] is convs[1]


# ---------------------------------------------------------------------------------------------------------------
# Fused form (GPU)
# ---------------------------------------------------------------------------------------------------------------
def _fused(name, T=4, gain=5.0, internal=False):
    model = M.build_network(name, width=SMALL[name]["width"], gain=gain)
    return model, M.fuse_network(model, T, BF16, DEV, internal_layouts=internal)


def _check_recorded_operators(hip_ops, name, fused, out, T, internal):
    """Every recorded operator call of one forward against the oracle on that call's own operands (teacher forcing)."""
    kinds = [e["kind"] for e in fused.record]
    if internal:     # the tail's neuron fires in the last convolution; pool and classifier read its bits
        assert kinds.count("conv_lif") == NEURONS[name] and kinds.count("spike_pool_linear") == 1 and kinds.count("tail") == 0
    else:
        assert kinds.count("conv_lif") == NEURONS[name] - 1 and kinds.count("tail") == 1
    active = 0
    for e in fused.record:
        if e["kind"] == "conv_lif":
            L = e["layer"]
            xs = [x.float().cpu() for x in e["xs"]]
            rs = None if e["residuals"] is None else [r.float().cpu() for r in e["residuals"]]
            if e.get("shortcut") is not None:     # a projection shortcut accumulated in the same launch: its sums, unrounded
                D = e["shortcut"]["layer"]
                rs = [F.conv2d(x.float().cpu(), D.weight.float().cpu(), D.bias.float().cpu(), D.stride, D.padding) for x in e["shortcut"]["x"]]
            ref = O.temporal_conv_lif(xs, L.weight.float().cpu(), L.bias.float().cpu(), torch.tensor(0.0), tuple(L.stride),
                                      tuple(L.padding), (1, 1), L.groups, *L.lif, residuals=rs)
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
        elif e["kind"] == "spike_pool_linear":
            x = e["x"].double().cpu()
            want = (x.sum((0, 3, 4)) @ e["fc_weight"].double().cpu().t() / (x.shape[3] * x.shape[4]) + T * e["fc_bias"].double().cpu()) / T
            assert torch.allclose(e["out"].double().cpu(), want, rtol=8e-3, atol=1e-3)
            assert torch.equal(out, e["out"])
        elif e["kind"] == "tail":
            ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(e["x"].float().cpu(), torch.tensor(0.0), e["fc_weight"].float().cpu(),
                                                                 e["fc_bias"].float().cpu(), *e["lif"])
            assert torch.equal(e["v"].cpu(), ref_v)
            assert torch.allclose(e["out_sum"].float().cpu(), ref_out, rtol=8e-3, atol=8e-3)
            assert torch.allclose(out.float().cpu(), ref_out / T, rtol=8e-3, atol=8e-3)
    assert active >= 5, "the test network is nearly silent"
    stats = hip_ops.get_fused_op_call_stats()
    if internal and name == "mobilenet":
        # row-packed spikes between the stride-1 depthwise and the pointwise layers; the stem (analog frame) and the two stride-2
        # depthwise layers go through the dense operator layer; the last convolution (with the tail's neuron) runs on
        # channel-packed bits
        packed = [e["name"] for e in fused.record if e.get("blocked")]
        assert packed == ["features.1", "features.2", "features.4", "features.5", "features.6", "features.8"], packed
        assert stats["fallback"] == 0 and stats["triton"] == 3, stats
    elif internal:      # nothing goes through the dense operator layer
        assert all(e.get("blocked") for e in fused.record if e["kind"] != "spike_pool_linear")
        assert stats["fallback"] == 0 and stats["triton"] == 0, stats
    else:
        assert stats["fallback"] == 0 and stats["triton"] == kinds.count("conv_lif") + 1, stats


@pytest.mark.gpu
@pytest.mark.parametrize("internal", [False, True], ids=["dense", "internal_layouts"])
@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
def test_fused_network_operator_by_operator_against_the_oracle(hip_ops, name, internal):
    """`internal`: spikes bit-packed and analog activations channel-blocked between the network's own operators; the
    executor records every operator's operands and results converted back to dense tensors."""
    T = 4
    model, fused = _fused(name, T, internal=internal)
    fused.record = []
    out = fused(_frame(name))
    torch.cuda.synchronize()
    _check_recorded_operators(hip_ops, name, fused, out, T, internal)


FULL = {"vgg11": dict(size=32, batch=64), "resnet18": dict(size=224, batch=16), "mobilenet": dict(size=64, batch=32)}


@pytest.mark.gpu
@pytest.mark.parametrize("internal", [False, True], ids=["dense", "internal_layouts"])
@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
def test_full_width_network_operator_by_operator_against_the_oracle(hip_ops, name, internal):
    """The benchmark configurations at their real size (width 64; VGG-11 T=4 B=64 32x32, ResNet-18 T=4 B=16 224x224, and the
    MobileNet-style network T=4 B=32 64x64):
    every operator call of one forward, with the launch plans those sizes select, against the oracle on its own operands."""
    T = 4
    cfg = FULL[name]
    model = M.build_network(name, width=64, gain=5.0)
    fused = M.fuse_network(model, T, BF16, DEV, internal_layouts=internal)
    x = q(torch.randn(cfg["batch"], 3, cfg["size"], cfg["size"], generator=gen(7)), BF16)
    fused.record = []
    print(f"full-width {name} internal={internal}", flush=True)
    out = fused(x)
    torch.cuda.synchronize()
    _check_recorded_operators(hip_ops, name, fused, out, T, internal)


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
@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
def test_internal_layouts_track_the_dense_executor(hip_ops, name):
    """Same network, same operands: the two executors differ in summation order only, so the first layer agrees up to
    near-threshold flips and the logits point the same way."""
    T = 4
    _, dense = _fused(name, T)
    _, internal = _fused(name, T, internal=True)
    x = _frame(name)
    dense.record, internal.record = [], []
    want, got = dense(x).float().cpu(), internal(x).float().cpu()
    mismatch = (dense.record[0]["spikes"].float().cpu() != internal.record[0]["spikes"].float().cpu()).float().mean()
    assert float(mismatch) <= 1e-4, float(mismatch)
    cos = float(F.cosine_similarity(got.flatten(), want.flatten(), dim=0))
    print(f"{name}: internal layouts vs dense executor, cosine similarity of the logits {cos:.5f}")
    assert cos > 0.8, cos
    if name == "mobilenet":
        # The row-packed entry points are the dense kernels with another fetch / store: every spike tensor up to the last
        # convolution is the same, bit for bit (the last convolution and the tail differ: its sums meet the tail's neuron
        # unrounded on the internal layouts).
        same = [(d["name"], torch.equal(d["spikes"], i["spikes"])) for d, i in zip(dense.record, internal.record)
                if d["kind"] == "conv_lif" and i["kind"] == "conv_lif" and d["name"] == i["name"] and d["name"] != "features.8"]
        assert len(same) == 8 and all(ok for _, ok in same), same
        assert cos > 0.9999, cos


@pytest.mark.gpu
@pytest.mark.parametrize("internal", [False, True], ids=["dense", "internal_layouts"])
@pytest.mark.parametrize("name", ["vgg11", "resnet18", "mobilenet"])
def test_fused_network_graph_replay_matches_eager_launches(hip_ops, name, internal):
    T = 4
    _, fused = _fused(name, T, internal=internal)
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

@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_rewritten_graph_runs_on_the_hip_kernels(hip_ops, name):
    """compile on the CPU in fp32, move to the GPU in bf16: the rewritten graph calls the same fused operators with the
    same operands as the hand-lowered executor (tail_first = the executor's lowering), so the logits agree closely (the
    LIF-free convolutions differ: per-timestep framework calls here, one batched matrix-kernel call there)."""
    T = 4
    model, fused = _fused(name, T)
    x = _frame(name)
    gm, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, device=DEV, dtype=BF16)
    assert not stats.skipped
    hip_ops.reset_fused_op_call_stats()
    with torch.no_grad():
        got = gm(x.to(DEV, BF16)).float().cpu()
    stats_ops = hip_ops.get_fused_op_call_stats()
    assert stats_ops["fallback"] == 0 and stats_ops["triton"] == (8 if name == "vgg11" else 17), stats_ops
    want = fused(x).float().cpu()
    cos = float(F.cosine_similarity(got.flatten(), want.flatten(), dim=0))
    print(f"{name}: FX graph vs executor, cosine similarity of the logits {cos:.5f}")
    assert cos > 0.8, cos


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_graph_on_the_internal_layouts_equals_the_hand_lowered_executor(hip_ops, name):
    """The layout-propagated graph launches the same kernels on the same operands as `fuse_network(internal_layouts=True)`:
    bit-identical logits, eagerly and under HIP graph replay, with nothing going through the dense operator layer."""
    T = 4
    model, internal = _fused(name, T, internal=True)
    gm, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, device=DEV, dtype=BF16, internal_layouts=True)
    # VGG-11: 12 less the four pools that run inside a convolution; ResNet-18: 21 less the three folded shortcuts
    assert not stats.skipped and stats.internal_layout_nodes == (8 if name == "vgg11" else 18)
    frames = [_frame(name, seed=30 + i).to(DEV, BF16) for i in range(3)]
    hip_ops.reset_fused_op_call_stats()
    with torch.no_grad():
        got = gm(frames[0])
    stats_ops = hip_ops.get_fused_op_call_stats()
    assert stats_ops["fallback"] == 0 and stats_ops["triton"] == 0, stats_ops
    assert torch.equal(got, internal(frames[0]))
    # whole-graph capture and replay, eager work in between
    static_in = frames[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        gm(static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        static_out = gm(static_in)
    for f in frames + [frames[0]]:
        want = internal(f).clone()
        torch.cuda.synchronize()
        static_in.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, want)


@pytest.mark.gpu
@pytest.mark.parametrize("T", [3, 6])
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_internal_layouts_with_other_step_counts_take_the_unfused_forms_where_needed(hip_ops, name, T):
    """Three timesteps (one short window) and six (two windows): the convolution + average pool launch only takes four, so the
    graph's nodes run convolution and pool apart; the shortcut and the bit-packed tail take both. Graph == hand-lowered
    executor bit for bit, every recorded operator against the oracle, no eager fallback."""
    model, internal = _fused(name, T, internal=True)
    gm, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, device=DEV, dtype=BF16, internal_layouts=True)
    assert not stats.skipped
    x = _frame(name, seed=40 + T)
    hip_ops.reset_fused_op_call_stats()
    with torch.no_grad():
        got = gm(x.to(DEV, BF16))
    internal.record = []
    want = internal(x)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0
    kinds = [e["kind"] for e in internal.record]
    assert kinds.count("conv_lif") == NEURONS[name] and kinds.count("spike_pool_linear") == 1
    if name == "vgg11":
        assert kinds.count("pool") == 4          # as launches of their own (recorded by the pooling call, not by a fused launch)
    for e in internal.record:
        if e["kind"] != "conv_lif":
            continue
        L = e["layer"]
        rs = None if e["residuals"] is None else [r.float().cpu() for r in e["residuals"]]
        if e.get("shortcut") is not None:
            D = e["shortcut"]["layer"]
            rs = [F.conv2d(f.float().cpu(), D.weight.float().cpu(), D.bias.float().cpu(), D.stride, D.padding) for f in e["shortcut"]["x"]]
        ref = O.temporal_conv_lif([f.float().cpu() for f in e["xs"]], L.weight.float().cpu(), L.bias.float().cpu(), torch.tensor(0.0),
                                  tuple(L.stride), tuple(L.padding), (1, 1), L.groups, *L.lif, residuals=rs)
        check(e["spikes"], e["v"], ref, what=f"{name} T={T} {e['name']}")


@pytest.mark.gpu
def test_fx_graph_with_an_unknown_layer_between_fused_layers_on_the_gpu(hip_ops):
    """Dense hand-overs around a node the layout pass does not know: same logits as the dense rewritten graph up to
    near-threshold flips (both graphs run the same arithmetic on different kernels)."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = M.ConvBNNeuron(3, 16, 3, 1, 1)
            self.clip = torch.nn.Hardtanh(0.0, 0.5)
            self.b = M.ConvBNNeuron(16, 32, 3, 1, 1)
            self.c = M.ConvBNNeuron(32, 16, 3, 1, 1)

        def forward(self, x):
            return self.c(self.b(self.clip(self.a(x)))).mean((2, 3))

    net = M.init_synthetic_(Net(), gain=5.0)
    x = q(torch.randn(2, 3, 16, 16, generator=gen(41)), BF16).to(DEV, BF16)
    dense, _ = R.compile_temporal(M.SingleStepModeLoopWrapper(net, 4), device=DEV, dtype=BF16)
    blocked, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(net, 4), device=DEV, dtype=BF16, internal_layouts=True)
    assert stats.internal_layout_nodes == 3
    with torch.no_grad():
        want, got = dense(x).float(), blocked(x).float()
    assert float((want - got).abs().max()) <= 0.05 and float(want.abs().max()) > 0.05, (want, got)
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0


@pytest.mark.gpu
@pytest.mark.parametrize("window", [None, 2])
def test_fx_graph_reaches_the_linear_and_scan_kernels(hip_ops, window):
    """Linear -> LIF and standalone LIF layers of a compiled graph run on `snnf_linear_lif` / `snnf_lif_scan` (no eager
    fallback), window by window when asked; the logits follow the eager CPU loop on the same bf16-rounded parameters."""
    T = 4
    net = M.init_synthetic_(_EncoderMlp(), gain=4.0)
    with torch.no_grad():
        for prm in net.parameters():
            prm.copy_(q(prm, BF16))
    x = q(torch.randn(3, 3, 8, 8, generator=gen(13)), BF16)
    wrapper = M.SingleStepModeLoopWrapper(net, T)
    with torch.no_grad():
        M.reset_lif_modules(net)
        want = wrapper(x)
    gm, stats = R.compile_temporal(wrapper, device=DEV, dtype=BF16, window=window)
    assert not stats.skipped and stats.temporal_linear_lif_groups == 2 and stats.temporal_lif_groups == 1
    hip_ops.reset_fused_op_call_stats()
    with torch.no_grad():
        got = gm(x.to(DEV, BF16)).float().cpu()
    s = hip_ops.get_fused_op_call_stats()
    per_layer = 1 if window is None else T // window
    assert s["fallback"] == 0 and s["triton"] == 4 * per_layer, s
    by_kind = s.get("by_op_kind", {})
    print("native calls by operator:", by_kind)
    assert float((got - want).abs().max()) <= 0.08 * max(1.0, float(want.abs().max())), (got, want)
    assert float(want.abs().max()) > 0.01


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["vgg11", "resnet18"])
def test_fx_graph_with_windows_of_two_steps_on_the_gpu(hip_ops, name):
    """T = 4 as two chained windows of 2: twice the fused nodes, every later window continuing from a float32 membrane;
    the logits stay those of the one-window graph up to near-threshold flips."""
    T = 4
    model, _ = _fused(name, T)
    x = _frame(name).to(DEV, BF16)
    whole, _ = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, device=DEV, dtype=BF16)
    halves, stats = R.compile_temporal(M.SingleStepModeLoopWrapper(model, T), tail_first=True, device=DEV, dtype=BF16, window=2)
    layers = 8 if name == "vgg11" else 17
    assert stats.temporal_windows == 2 * layers and not stats.skipped
    hip_ops.reset_fused_op_call_stats()
    with torch.no_grad():
        got = halves(x).float().cpu()
    s = hip_ops.get_fused_op_call_stats()
    assert s["fallback"] == 0 and s["triton"] == 2 * layers, s
    with torch.no_grad():
        want = whole(x).float().cpu()
    cos = float(F.cosine_similarity(got.flatten(), want.flatten(), dim=0))
    print(f"{name}: windows of 2 vs one window, cosine similarity of the logits {cos:.5f}")
    assert cos > 0.8, cos      # same bar as the other executor comparisons: flips near the threshold cascade with random weights


@pytest.mark.gpu
def test_internal_layouts_fall_back_to_the_dense_operator_for_a_refused_layer(hip_ops, monkeypatch):
    """A layer the blocked kernel refuses (large kernels on many channels: `unsupported_*`) runs the dense operator on
    unpacked tensors and re-enters the internal layout; the network's output stays that of the other executors."""
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B
    T = 4
    _, dense = _fused("resnet18", T)
    _, internal = _fused("resnet18", T, internal=True)
    x = _frame("resnet18")
    want = dense(x).float().cpu()
    real = B.conv_lif_blocked
    calls = {"n": 0, "refused": 0}

    def picky(xb, weight, *args, **kwargs):
        calls["n"] += 1
        if calls["n"] in (2, 5, 7):          # three layers along the network (with and without a residual)
            calls["refused"] += 1
            raise RuntimeError("unsupported_shape: refused for the test")
        return real(xb, weight, *args, **kwargs)

    monkeypatch.setattr(B, "conv_lif_blocked", picky)
    got = internal(x).float().cpu()
    assert calls["refused"] == 3
    cos = float(F.cosine_similarity(got.flatten(), want.flatten(), dim=0))
    assert cos > 0.8, cos
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0
