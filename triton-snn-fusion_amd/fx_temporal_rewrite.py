"""Minimal temporal FX rewriter: T unrolled single-step iterations -> fused temporal operators.

Counterpart of the reference's rewrite pipeline for the patterns the fused operators serve
(compiler/fx_lif_temporal_rewrite.py: `collect_conv_bn_lif_state_patterns` :337, `collect_conv_bn_add_lif_state_patterns`
:423, `collect_standalone_lif_state_patterns` :534, `collect_temporal_linear_lif_state_patterns` :694,
`collect_temporal_lif_avgpool_linear_patterns` :791, `group_temporal_patterns` :884, `check_temporal_state_chain` :929,
`make_temporal_windows` :955-1094, `rewrite_temporal_conv_bn_lif_state_to_fused` :2037, residual :2214, standalone LIF
:2408, Linear + LIF :2548, tail :2745; BatchNorm folding compiler/fx_lif_rewrite.py:340-353). The reference obtains its graph from torch.compile and works on function-level
nodes; this one traces a `SingleStepModeLoopWrapper`-style module with `torch.fx.symbolic_trace`, so convolutions,
BatchNorms, pools and the classifier are `call_module` nodes and each neuron call is a
`torch.ops.snn_custom.lif_forward_state` node whose membrane operand is the previous call's second output.

Pipeline (`compile_temporal`):
  1. `trace_single_step_loop`  - unrolls the T iterations; a neuron's first membrane is the scalar-zero constant.
  2. collect                   - Conv2d -> BatchNorm2d -> LIF, Conv2d -> BatchNorm2d -> add(residual) -> LIF, Linear -> LIF, the
                                 tail LIF -> AdaptiveAvgPool2d(1) -> flatten -> Linear -> running sum, and LIF calls on their
                                 own; one pattern per timestep.
  3. group + check             - patterns of one layer (same conv and BN module, same Linear, same neuron) ordered by
                                 timestep; the state chain must be v_getitem[t-1] -> v_prev[t] with a scalar-zero start,
                                 otherwise the layer is left alone.
  4. windows                   - a layer's T patterns are cut into windows of `window` consecutive timesteps (all T by
                                 default); the final membrane of one window is the initial membrane of the next.
  5. rewrite                   - one fused operator node per window over the list of its inputs (operator chosen by
                                 convolution kind: regular / pointwise / depthwise, as compiler/fx_lif_temporal_rewrite.py
                                 :1625-1662), folded weights as graph attributes, per-timestep spikes as `spike_stack[t]`.
The graph is then re-emitted in dependency order, which turns the time-major trace into layer-major execution.
"""
from __future__ import annotations

import operator
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.fx as fx
import torch.nn as nn
import torch.nn.functional as F

from .runtime.hip_pool_backend import pool_config
from .workloads import fold_bn_into_conv_params


def _lif_targets():
    from .runtime import snn_custom_ops  # noqa: F401  (registers torch.ops.snn_custom)
    return (torch.ops.snn_custom.lif_forward_state, torch.ops.snn_custom.lif_forward_state.default)


def is_custom_lif_state_node(node: fx.Node) -> bool:
    return node.op == "call_function" and node.target in _lif_targets()


def _is_add_node(node: fx.Node) -> bool:
    return node.op == "call_function" and node.target in (operator.add, operator.iadd, torch.add)


def _module_of(gm: fx.GraphModule, node: fx.Node, kind) -> Optional[nn.Module]:
    if node.op != "call_module":
        return None
    mod = gm.get_submodule(node.target)
    return mod if isinstance(mod, kind) else None


def find_tuple_getitems(node: fx.Node) -> Dict[int, fx.Node]:
    out: Dict[int, fx.Node] = {}
    for user in node.users:
        if user.op == "call_function" and user.target is operator.getitem and isinstance(user.args[1], int):
            out[user.args[1]] = user
    return out


def _is_scalar_zero(gm: fx.GraphModule, arg) -> bool:
    """The membrane a neuron starts from: a 0-dim zero tensor held by the traced module."""
    if isinstance(arg, fx.Node) and arg.op == "get_attr":
        value = gm
        for part in arg.target.split("."):
            value = getattr(value, part)
        return isinstance(value, torch.Tensor) and value.dim() == 0 and float(value) == 0.0
    return False


# ---------------------------------------------------------------------------------------------------------------
# Tracing
# ---------------------------------------------------------------------------------------------------------------
def trace_single_step_loop(wrapper: nn.Module) -> fx.GraphModule:
    """symbolic_trace of a module that calls a single-step network T times (the loop unrolls). Neuron modules are traced
    through a forward that skips the shape check of the state (a 0-dim membrane means zeros to the operator anyway): the
    first call of a neuron takes one shared scalar-zero constant, later calls the previous call's second output. The
    modules are reset afterwards."""
    from .models import CustomStatefulIFNode, reset_custom_stateful_lif_modules
    from .runtime import snn_custom_ops  # noqa: F401  (registers torch.ops.snn_custom)

    zero = torch.zeros(())

    def traced_forward(self, x):
        v_prev = self.v if isinstance(self.v, fx.Proxy) else zero
        spike, self.v = torch.ops.snn_custom.lif_forward_state(x, v_prev, self.v_threshold, self.v_reset, self.tau, self.detach_reset)
        return spike

    reset_custom_stateful_lif_modules(wrapper)
    original = CustomStatefulIFNode.forward
    CustomStatefulIFNode.forward = traced_forward
    try:
        gm = fx.symbolic_trace(wrapper)
    finally:
        CustomStatefulIFNode.forward = original
        reset_custom_stateful_lif_modules(wrapper)
    return gm


# ---------------------------------------------------------------------------------------------------------------
# Patterns
# ---------------------------------------------------------------------------------------------------------------
@dataclass
class TemporalPattern:
    layer_id: str
    timestep_index: int
    conv_node: fx.Node
    bn_node: fx.Node
    lif_node: fx.Node
    spike_getitem: Optional[fx.Node]
    v_getitem: Optional[fx.Node]
    conv_input: fx.Node
    v_prev_node: object
    lif_params: Tuple
    add_node: Optional[fx.Node] = None          # residual form: lif(add(bn(conv(x)), residual))
    residual_node: Optional[fx.Node] = None


@dataclass
class TemporalLifAvgPoolLinearPattern:
    layer_id: str
    timestep_index: int
    lif_node: fx.Node
    input_node: fx.Node
    v_prev_node: object
    spike_getitem: fx.Node
    v_getitem: Optional[fx.Node]
    pool_node: fx.Node
    flatten_node: fx.Node
    linear_node: fx.Node
    acc_node: fx.Node
    acc_prev: object
    lif_params: Tuple


@dataclass
class TemporalGroup:
    layer_id: str
    patterns: List = field(default_factory=list)


def _conv_bn_of(gm: fx.GraphModule, node) -> Optional[Tuple[fx.Node, fx.Node]]:
    """(conv_node, bn_node) when `node` is BatchNorm2d(Conv2d(x)) with the convolution feeding only the BatchNorm."""
    if not isinstance(node, fx.Node) or _module_of(gm, node, nn.BatchNorm2d) is None:
        return None
    conv = node.args[0]
    if not isinstance(conv, fx.Node) or _module_of(gm, conv, nn.Conv2d) is None or len(conv.users) != 1:
        return None
    if gm.get_submodule(node.target).training:
        return None
    return conv, node


def _lif_state_is_usable(node: fx.Node) -> Tuple[bool, str]:
    if len(node.args) < 6 or node.kwargs:
        return False, "unsupported lif args"
    if not all(isinstance(a, (int, float, bool)) for a in node.args[2:6]):
        return False, "lif parameters are not constants"
    extra = [u for u in node.users if not (u.op == "call_function" and u.target is operator.getitem)]
    return (not extra), ("lif output used as a tuple" if extra else "")


def _collect(gm: fx.GraphModule, residual: bool) -> List[TemporalPattern]:
    counts: Dict[str, int] = {}
    patterns: List[TemporalPattern] = []
    for node in gm.graph.nodes:
        if not is_custom_lif_state_node(node) or not _lif_state_is_usable(node)[0]:
            continue
        source = node.args[0]
        add_node = residual_node = None
        if residual:
            if not isinstance(source, fx.Node) or not _is_add_node(source) or len(source.users) != 1:
                continue
            a, b = source.args[0], source.args[1]
            pair = _conv_bn_of(gm, a)
            other = b
            if pair is None:
                pair, other = _conv_bn_of(gm, b), a
            if pair is None or not isinstance(other, fx.Node) or len(pair[1].users) != 1:
                continue
            add_node, residual_node = source, other
        else:
            pair = _conv_bn_of(gm, source)
            if pair is None or len(pair[1].users) != 1:
                continue
        conv_node, bn_node = pair
        layer_id = f"conv={conv_node.target}|bn={bn_node.target}|params={tuple(node.args[2:6])!r}"
        getitems = find_tuple_getitems(node)
        t = counts.get(layer_id, 0)
        counts[layer_id] = t + 1
        patterns.append(TemporalPattern(layer_id, t, conv_node, bn_node, node, getitems.get(0), getitems.get(1),
                                        conv_node.args[0], node.args[1], tuple(node.args[2:6]), add_node, residual_node))
    return patterns


def collect_conv_bn_lif_state_patterns(gm: fx.GraphModule) -> List[TemporalPattern]:
    return _collect(gm, residual=False)


def collect_conv_bn_add_lif_state_patterns(gm: fx.GraphModule) -> List[TemporalPattern]:
    return _collect(gm, residual=True)


def _single_user(node: Optional[fx.Node]) -> Optional[fx.Node]:
    if node is None or len(node.users) != 1:
        return None
    return next(iter(node.users))


def collect_temporal_lif_avgpool_linear_patterns(gm: fx.GraphModule, excluded_lif_nodes=None) -> List[TemporalLifAvgPoolLinearPattern]:
    excluded = set(excluded_lif_nodes or [])
    counts: Dict[str, int] = {}
    patterns: List[TemporalLifAvgPoolLinearPattern] = []
    for node in gm.graph.nodes:
        if node in excluded or not is_custom_lif_state_node(node) or not _lif_state_is_usable(node)[0]:
            continue
        getitems = find_tuple_getitems(node)
        pool = _single_user(getitems.get(0))
        pool_mod = _module_of(gm, pool, nn.AdaptiveAvgPool2d) if pool is not None else None
        if pool_mod is None or tuple(pool_mod.output_size if isinstance(pool_mod.output_size, (tuple, list)) else (pool_mod.output_size,) * 2) != (1, 1):
            continue
        flatten = _single_user(pool)
        if flatten is None or not (flatten.op == "call_function" and flatten.target is torch.flatten and tuple(flatten.args[1:]) in ((1,), (1, -1))):
            continue
        linear = _single_user(flatten)
        if linear is None or _module_of(gm, linear, nn.Linear) is None:
            continue
        acc = _single_user(linear)
        if acc is None or not _is_add_node(acc):
            continue
        acc_prev = acc.args[1] if acc.args[0] is linear else acc.args[0]
        layer_id = f"lif_avgpool_linear|fc={linear.target}|params={tuple(node.args[2:6])!r}"
        t = counts.get(layer_id, 0)
        counts[layer_id] = t + 1
        patterns.append(TemporalLifAvgPoolLinearPattern(layer_id, t, node, node.args[0], node.args[1], getitems[0], getitems.get(1),
                                                        pool, flatten, linear, acc, acc_prev, tuple(node.args[2:6])))
    return patterns


@dataclass
class TemporalLinearLifPattern:
    layer_id: str
    timestep_index: int
    linear_node: fx.Node
    linear_input: fx.Node
    lif_node: fx.Node
    spike_getitem: Optional[fx.Node]
    v_getitem: Optional[fx.Node]
    v_prev_node: object
    lif_params: Tuple


@dataclass
class TemporalLifPattern:
    layer_id: str
    timestep_index: int
    lif_node: fx.Node
    input_node: fx.Node
    spike_getitem: Optional[fx.Node]
    v_getitem: Optional[fx.Node]
    v_prev_node: object
    lif_params: Tuple


def collect_temporal_linear_lif_state_patterns(gm: fx.GraphModule, excluded_lif_nodes=None) -> List[TemporalLinearLifPattern]:
    """LIF(Linear(x)) with the Linear feeding only its neuron (compiler/fx_lif_temporal_rewrite.py:694-770)."""
    excluded = set(excluded_lif_nodes or [])
    counts: Dict[str, int] = {}
    patterns: List[TemporalLinearLifPattern] = []
    for node in gm.graph.nodes:
        if node in excluded or not is_custom_lif_state_node(node) or not _lif_state_is_usable(node)[0]:
            continue
        linear = node.args[0]
        if not isinstance(linear, fx.Node) or _module_of(gm, linear, nn.Linear) is None or len(linear.users) != 1:
            continue
        if not isinstance(linear.args[0], fx.Node):
            continue
        layer_id = f"linear_lif|fc={linear.target}|params={tuple(node.args[2:6])!r}"
        getitems = find_tuple_getitems(node)
        t = counts.get(layer_id, 0)
        counts[layer_id] = t + 1
        patterns.append(TemporalLinearLifPattern(layer_id, t, linear, linear.args[0], node, getitems.get(0), getitems.get(1),
                                                 node.args[1], tuple(node.args[2:6])))
    return patterns


def _produces_rank_two(gm: fx.GraphModule, node) -> bool:
    """Linear outputs and flattened tensors are [N, F]; the temporal LIF operator takes [T, N, C, H, W] only
    (runtime/snn_custom_ops.py:529; the same exclusion as compiler/fx_lif_temporal_rewrite.py:563-568)."""
    if not isinstance(node, fx.Node):
        return True
    if _module_of(gm, node, (nn.Linear, nn.Flatten)) is not None:
        return True
    if node.op == "call_function" and node.target is torch.flatten:
        return True
    if node.op == "call_method" and node.target in ("flatten", "view", "reshape"):
        return True
    rank = node.meta.get("chronos_rank")
    return rank is not None and rank != 4


def collect_standalone_lif_state_patterns(gm: fx.GraphModule, excluded_lif_nodes=None) -> List[TemporalLifPattern]:
    """LIF calls that no other pattern has claimed, on [N, C, H, W] inputs (compiler/fx_lif_temporal_rewrite.py:534-598).
    The reference keys a layer by the call's occurrence inside a timestep and its shape; here a layer is one neuron's state
    chain: it starts at a call on the scalar-zero membrane and continues through v_getitem -> v_prev."""
    excluded = set(excluded_lif_nodes or [])
    patterns: List[TemporalLifPattern] = []
    chain_of: Dict[fx.Node, Tuple[str, int]] = {}
    chains = 0
    for node in gm.graph.nodes:
        if not is_custom_lif_state_node(node):
            continue
        v_prev = node.args[1]
        if isinstance(v_prev, fx.Node) and v_prev.op == "call_function" and v_prev.target is operator.getitem and v_prev.args[0] in chain_of:
            layer_id, t = chain_of[v_prev.args[0]]
            chain_of[node] = (layer_id, t + 1)
        else:
            chain_of[node] = (f"standalone_lif|chain={chains}|params={tuple(node.args[2:6])!r}", 0)
            chains += 1
        if node in excluded or not _lif_state_is_usable(node)[0] or _produces_rank_two(gm, node.args[0]):
            continue
        layer_id, t = chain_of[node]
        getitems = find_tuple_getitems(node)
        patterns.append(TemporalLifPattern(layer_id, t, node, node.args[0], getitems.get(0), getitems.get(1), node.args[1],
                                           tuple(node.args[2:6])))
    return patterns


def make_temporal_windows(groups: List["TemporalGroup"], window_size: Optional[int], allow_tail: bool = True) -> List["TemporalGroup"]:
    """Cuts every group's timestep-ordered patterns into windows of `window_size` consecutive timesteps (None: one window of
    all of them). A shorter last window is kept when `allow_tail`; windows of a single timestep are left to the single-step
    nodes already in the graph (compiler/fx_lif_temporal_rewrite.py:955-974). Patterns of a window must be consecutive."""
    windows: List[TemporalGroup] = []
    for group in groups:
        steps = [p.timestep_index for p in group.patterns]
        if steps != list(range(steps[0], steps[0] + len(steps))):
            continue        # a claimed or unusable call interrupts the layer: leave it alone
        size = len(group.patterns) if window_size is None else int(window_size)
        if size < 1:
            continue
        for start in range(0, len(group.patterns), size):
            chunk = group.patterns[start:start + size]
            if len(chunk) < size and not allow_tail:
                continue
            if len(chunk) <= 1 and window_size is not None:
                continue
            windows.append(TemporalGroup(group.layer_id, chunk))
    return windows


def group_temporal_patterns(patterns) -> List[TemporalGroup]:
    grouped: Dict[str, List] = {}
    for p in patterns:
        grouped.setdefault(p.layer_id, []).append(p)
    return [TemporalGroup(k, sorted(v, key=lambda p: p.timestep_index)) for k, v in grouped.items()]


def check_temporal_state_chain(gm: fx.GraphModule, patterns) -> Tuple[bool, str]:
    """The membrane of step t must be exactly the second output of step t-1, the first one the scalar zero, and nothing
    else may read the intermediate membranes."""
    if patterns[0].timestep_index == 0 and not _is_scalar_zero(gm, patterns[0].v_prev_node):
        return False, f"{patterns[0].lif_node.name} does not start from the scalar-zero membrane"
    for prev, nxt in zip(patterns, patterns[1:]):
        if prev.v_getitem is None or nxt.v_prev_node is not prev.v_getitem:
            return False, f"{prev.lif_node.name} membrane does not feed {nxt.lif_node.name} v_prev"
        if len(prev.v_getitem.users) != 1:
            return False, f"{prev.v_getitem.name} has other users"
    last = patterns[-1].v_getitem
    if last is not None and len(last.users) != 0:
        return False, f"{last.name} (final membrane) is read by the graph"
    return True, ""


def check_temporal_lif_avgpool_linear_state_and_acc_chain(gm: fx.GraphModule, patterns) -> Tuple[bool, str]:
    ok, reason = check_temporal_state_chain(gm, patterns)
    if not ok:
        return ok, reason
    if not (isinstance(patterns[0].acc_prev, (int, float)) and patterns[0].acc_prev == 0):
        return False, "the running sum does not start from 0"
    for prev, nxt in zip(patterns, patterns[1:]):
        if nxt.acc_prev is not prev.acc_node:
            return False, f"{prev.acc_node.name} does not feed {nxt.acc_node.name}"
        if len(prev.acc_node.users) != 1:
            return False, f"{prev.acc_node.name} has other users"
    return True, ""


# ---------------------------------------------------------------------------------------------------------------
# Rewrite
# ---------------------------------------------------------------------------------------------------------------
@dataclass
class RewriteStats:
    temporal_conv_bn_lif_groups: int = 0
    temporal_conv_bn_add_lif_groups: int = 0
    temporal_lif_avgpool_linear_groups: int = 0
    temporal_linear_lif_groups: int = 0
    temporal_lif_groups: int = 0
    temporal_windows: int = 0
    replaced_patterns: int = 0
    batched_timestep_calls: int = 0
    internal_layout_nodes: int = 0
    skipped: List[str] = field(default_factory=list)


def classify_conv_kind(conv: nn.Conv2d) -> str:
    if conv.groups == conv.in_channels == conv.out_channels and conv.groups > 1:
        return "depthwise"
    if conv.groups == 1 and tuple(conv.kernel_size) == (1, 1) and tuple(conv.stride) == (1, 1) and tuple(conv.padding) == (0, 0):
        return "pointwise"
    return "regular"


def _register(gm: fx.GraphModule, name: str, value: torch.Tensor) -> str:
    base, i = name, 0
    while hasattr(gm, name):
        i += 1
        name = f"{base}_{i}"
    gm.register_buffer(name, value, persistent=False)
    return name


def _folded_params(gm: fx.GraphModule, group: TemporalGroup, index: int) -> Tuple[str, str, nn.Conv2d]:
    conv = gm.get_submodule(group.patterns[0].conv_node.target)
    bn = gm.get_submodule(group.patterns[0].bn_node.target)
    with torch.no_grad():
        w, b = fold_bn_into_conv_params(conv.weight.float(), conv.bias, bn.running_mean.float(), bn.running_var.float(),
                                        None if bn.weight is None else bn.weight.float(), None if bn.bias is None else bn.bias.float(), bn.eps)
        w = w.to(conv.weight.dtype).contiguous()
        b = b.to(conv.weight.dtype).contiguous()
    return _register(gm, f"fused_weight_{index}", w), _register(gm, f"fused_bias_{index}", b), conv


def rewrite_temporal_to_fused(gm: fx.GraphModule, stats: Optional[RewriteStats] = None, tail_first: bool = False,
                              window_size: Optional[int] = None, allow_tail: bool = True) -> RewriteStats:
    """Replaces every layer whose patterns pass the state-chain check by fused temporal operator nodes: one per window of
    `window_size` consecutive timesteps (None: one node over all T). The final membrane of a window is the initial membrane
    of the layer's next step, fused or not (compiler/fx_lif_temporal_rewrite.py:955-974, 2085, 2144-2145)."""
    stats = stats or RewriteStats()
    S = torch.ops.snn_custom
    graph = gm.graph
    output_node = next(n for n in graph.nodes if n.op == "output")
    device = next((p.device for p in gm.parameters()), torch.device("cpu"))
    zero_name = _register(gm, "chronos_zero_membrane", torch.zeros((), dtype=torch.float32, device=device))
    index = 0
    claimed = set()
    in_a_family = set()      # neuron calls behind a convolution, a Linear or in front of the classifier: never "standalone"

    def windows_of(group: TemporalGroup, check) -> List[TemporalGroup]:
        ok, reason = check(gm, group.patterns)
        if not ok:
            stats.skipped.append(f"{group.layer_id}: {reason}")
            return []
        return make_temporal_windows([group], window_size, allow_tail)

    def initial_membrane(first) -> fx.Node:
        """Scalar zero for a layer's first step; otherwise whatever feeds that step now: the previous window's final
        membrane, or the second output of a single step that was left alone."""
        if first.timestep_index == 0:
            return graph.get_attr(zero_name)
        return first.lif_node.args[1]

    def finish_window(window: TemporalGroup, fused: fx.Node) -> None:
        """Per-timestep spikes become `spike_stack[i]`; a later step that continues from the window reads `fused[1]`."""
        spike_stack = graph.call_function(operator.getitem, (fused, 0))
        for i, p in enumerate(window.patterns):
            if p.spike_getitem is not None:
                p.spike_getitem.replace_all_uses_with(graph.call_function(operator.getitem, (spike_stack, i)))
            claimed.add(p.lif_node)
        last = window.patterns[-1].v_getitem
        if last is not None and len(last.users) > 0:
            last.replace_all_uses_with(graph.call_function(operator.getitem, (fused, 1)))
        stats.replaced_patterns += len(window.patterns)
        stats.temporal_windows += 1

    tail_groups = []
    if tail_first:
        # The neuron in front of the classifier belongs to the tail operator; its convolution stays a plain layer.
        tail_groups = group_temporal_patterns(collect_temporal_lif_avgpool_linear_patterns(gm))
        for group in tail_groups:
            if check_temporal_lif_avgpool_linear_state_and_acc_chain(gm, group.patterns)[0]:
                claimed.update(p.lif_node for p in group.patterns)

    conv_groups = [(g, False) for g in group_temporal_patterns(collect_conv_bn_lif_state_patterns(gm))]
    conv_groups += [(g, True) for g in group_temporal_patterns(collect_conv_bn_add_lif_state_patterns(gm))]
    for group, residual in conv_groups:
        in_a_family.update(p.lif_node for p in group.patterns)
        if any(p.lif_node in claimed for p in group.patterns):
            continue
        windows = windows_of(group, check_temporal_state_chain)
        if not windows:
            continue
        w_name, b_name, conv = _folded_params(gm, group, index)
        index += 1
        kind = classify_conv_kind(conv)
        geometry = (list(conv.stride), list(conv.padding), list(conv.dilation), int(conv.groups))
        lif = tuple(group.patterns[0].lif_params)
        for window in windows:
            # Operands are read from the nodes now: an earlier rewrite may have redirected them to its spike_stack[t].
            xs = [p.conv_node.args[0] for p in window.patterns]
            residuals = [next(a for a in p.add_node.args if a is not p.bn_node) for p in window.patterns] if residual else None
            # New nodes go in front of the output; the graph is re-emitted in dependency order at the end.
            with graph.inserting_before(output_node):
                w_node = graph.get_attr(w_name)
                b_node = graph.get_attr(b_name)
                v0 = initial_membrane(window.patterns[0])
                if residual:
                    op = S.fused_temporal_conv_add_lif_state_depthwise if kind == "depthwise" else S.fused_temporal_conv_add_lif_state
                    args = (xs, residuals, w_node, b_node, v0, *geometry, *lif)
                else:
                    op = {"regular": S.fused_temporal_conv_lif_state, "pointwise": S.fused_temporal_pointwise_conv_lif_state,
                          "depthwise": S.fused_temporal_depthwise_conv_lif_state}[kind]
                    args = (xs, w_node, b_node, v0, *geometry, *lif)
                finish_window(window, graph.call_function(op, args))
        if residual:
            stats.temporal_conv_bn_add_lif_groups += 1
        else:
            stats.temporal_conv_bn_lif_groups += 1

    # Linear -> LIF: the list form of the operator reads the T inputs where they are (no stack).
    for group in group_temporal_patterns(collect_temporal_linear_lif_state_patterns(gm, excluded_lif_nodes=claimed)):
        in_a_family.update(p.lif_node for p in group.patterns)
        windows = windows_of(group, check_temporal_state_chain)
        if not windows:
            continue
        fc = gm.get_submodule(group.patterns[0].linear_node.target)
        w_name = _register(gm, f"fused_linear_weight_{index}", fc.weight.detach().contiguous())
        b_name = None if fc.bias is None else _register(gm, f"fused_linear_bias_{index}", fc.bias.detach().contiguous())
        index += 1
        for window in windows:
            xs = [p.linear_node.args[0] for p in window.patterns]
            with graph.inserting_before(output_node):
                w_node = graph.get_attr(w_name)
                b_node = None if b_name is None else graph.get_attr(b_name)
                v0 = initial_membrane(window.patterns[0])
                finish_window(window, graph.call_function(S.fused_temporal_linear_lif_state, (xs, w_node, b_node, v0, *group.patterns[0].lif_params)))
        stats.temporal_linear_lif_groups += 1

    if not tail_first:
        tail_groups = group_temporal_patterns(collect_temporal_lif_avgpool_linear_patterns(gm, excluded_lif_nodes=claimed))
    for group in tail_groups:
        in_a_family.update(p.lif_node for p in group.patterns)
        windows = windows_of(group, check_temporal_lif_avgpool_linear_state_and_acc_chain)
        if not windows:
            continue
        fc = gm.get_submodule(group.patterns[0].linear_node.target)
        w_name = _register(gm, "fused_fc_weight", fc.weight.detach().contiguous())
        b_name = _register(gm, "fused_fc_bias", fc.bias.detach().contiguous() if fc.bias is not None else torch.empty(0, dtype=fc.weight.dtype, device=fc.weight.device))
        for window in windows:
            xs = [p.lif_node.args[0] for p in window.patterns]
            first, last = window.patterns[0], window.patterns[-1]
            # The running sum in front of the window, as the graph holds it now (0 for the first step).
            acc_before = next(a for a in first.acc_node.args if a is not first.linear_node)
            with graph.inserting_before(output_node):
                x_seq = graph.call_function(torch.stack, (xs,))
                w_node = graph.get_attr(w_name)
                b_node = graph.get_attr(b_name)
                v0 = initial_membrane(first)
                fused = graph.call_function(S.fused_temporal_lif_avgpool_linear, (x_seq, v0, w_node, b_node, *first.lif_params))
                out_sum = graph.call_function(operator.getitem, (fused, 0))
                if isinstance(acc_before, fx.Node) or acc_before != 0:
                    out_sum = graph.call_function(operator.add, (acc_before, out_sum))
                if last.v_getitem is not None and len(last.v_getitem.users) > 0:
                    last.v_getitem.replace_all_uses_with(graph.call_function(operator.getitem, (fused, 1)))
            last.acc_node.replace_all_uses_with(out_sum)
            claimed.update(p.lif_node for p in window.patterns)
            stats.replaced_patterns += len(window.patterns)
            stats.temporal_windows += 1
        stats.temporal_lif_avgpool_linear_groups += 1

    # Neurons on their own (no convolution or Linear in front that a pattern above has taken): one scan over the stacked inputs.
    for group in group_temporal_patterns(collect_standalone_lif_state_patterns(gm, excluded_lif_nodes=claimed | in_a_family)):
        if any(p.lif_node in claimed for p in group.patterns):
            continue
        windows = windows_of(group, check_temporal_state_chain)
        if not windows:
            continue
        for window in windows:
            xs = [p.lif_node.args[0] for p in window.patterns]
            with graph.inserting_before(output_node):
                x_seq = graph.call_function(torch.stack, (xs,))
                v0 = initial_membrane(window.patterns[0])
                finish_window(window, graph.call_function(S.fused_temporal_lif_state, (x_seq, v0, *group.patterns[0].lif_params)))
        stats.temporal_lif_groups += 1

    _emit_in_dependency_order(gm)
    gm.graph.lint()
    gm.recompile()
    return stats


def pooled_frames(x_seq: torch.Tensor, is_max: bool, kernel: int, stride: int, padding: int) -> torch.Tensor:
    """Pooling of a [T, N, C, H, W] sequence: the HIP pooling kernel on the GPU, the framework's pooling on CPU tensors."""
    if x_seq.is_cuda:
        from .runtime.hip_pool_backend import run_hip_pool2d
        return run_hip_pool2d(x_seq, is_max, kernel, stride, padding)
    flat = x_seq.flatten(0, 1)
    y = F.max_pool2d(flat, kernel, stride, padding) if is_max else F.avg_pool2d(flat, kernel, stride, padding)
    return y.unflatten(0, (x_seq.shape[0], -1))


def conv_bias_frames(x_seq: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, stride, padding) -> torch.Tensor:
    """LIF-free convolution + folded BatchNorm of a [T, N, C, H, W] sequence: the matrix kernel's neuron-free mode where
    it takes the layer, the framework's convolution otherwise."""
    if x_seq.is_cuda:
        from .runtime.hip_convlif_backend import run_hip_temporal_conv_bias
        try:
            return run_hip_temporal_conv_bias(list(x_seq.unbind(0)), weight, bias, stride, padding)
        except RuntimeError as exc:
            if "unsupported" not in str(exc):
                raise
    y = F.conv2d(x_seq.flatten(0, 1), weight, bias, stride, padding)
    return y.unflatten(0, (x_seq.shape[0], -1))


_TIME_BATCHABLE = (nn.Conv2d, nn.BatchNorm2d, nn.MaxPool2d, nn.AvgPool2d, nn.AdaptiveAvgPool2d, nn.Identity, nn.Linear)


def _following_batchnorm(gm: fx.GraphModule, conv_members: Dict[int, fx.Node]) -> Optional[Dict[int, fx.Node]]:
    """The eval-mode BatchNorm2d nodes (one module) that are the only users of the T convolution nodes, else None."""
    out: Dict[int, fx.Node] = {}
    target = None
    for t, conv in conv_members.items():
        user = _single_user(conv)
        mod = _module_of(gm, user, nn.BatchNorm2d) if user is not None else None
        if mod is None or mod.training or (target is not None and user.target != target):
            return None
        target = user.target
        out[t] = user
    return out


def batch_timestep_calls(gm: fx.GraphModule) -> int:
    """Stateless layers that the trace applies once per timestep to `stack[t]`, t = 0..T-1, of one [T, N, ...] tensor
    (pools, LIF-free convolutions and their BatchNorm, residual adds, flatten, the classifier) are applied once to the T*N frames
    instead (the role of the reference's `_batched_tn` operator variants). Repeats until nothing changes, so chains such
    as Conv2d -> BatchNorm2d batch link by link. Returns the number of per-timestep calls removed."""
    removed = 0
    changed = True
    while changed:
        changed = False
        graph = gm.graph            # re-emission below replaces the graph object
        groups: Dict[Tuple, Dict[int, fx.Node]] = {}
        for node in graph.nodes:
            key = None
            if node.op == "call_module" and len(node.args) == 1 and not node.kwargs:
                mod = gm.get_submodule(node.target)
                if isinstance(mod, _TIME_BATCHABLE) and not (isinstance(mod, nn.BatchNorm2d) and mod.training):
                    key = ("module", node.target)
            elif node.op == "call_function" and node.target is torch.flatten and tuple(node.args[1:]) == (1,) and not node.kwargs:
                key = ("flatten",)
            elif _is_add_node(node) and len(node.args) == 2 and not node.kwargs:
                key = ("add",)
            if key is None:
                continue
            sources = node.args[:2] if key[0] == "add" else node.args[:1]
            if not all(isinstance(src, fx.Node) and src.op == "call_function" and src.target is operator.getitem
                       and isinstance(src.args[1], int) and isinstance(src.args[0], fx.Node) for src in sources):
                continue
            if len({src.args[1] for src in sources}) != 1:
                continue    # operands of different timesteps
            groups.setdefault(key + tuple(src.args[0] for src in sources), {})[sources[0].args[1]] = node
        for key, members in groups.items():
            stacks = key[2:] if key[0] == "module" else key[1:]
            stack = stacks[0]
            T = len(members)
            complete = T >= 2 and sorted(members) == list(range(T))
            for st in stacks:
                steps = {u.args[1] for u in st.users if u.op == "call_function" and u.target is operator.getitem}
                complete = complete and steps == set(range(T))
            if not complete:
                continue    # not every timestep of the stack goes through this layer
            first = min(members.values(), key=lambda n: list(graph.nodes).index(n)) if key[0] == "add" else members[0]
            targets = members
            with graph.inserting_before(first):
                if key[0] == "module":
                    mod = gm.get_submodule(key[1])
                    pool = pool_config(mod)
                    bn_members = _following_batchnorm(gm, members) if isinstance(mod, nn.Conv2d) else None
                    if pool is not None:
                        y_seq = graph.call_function(pooled_frames, (stack, *pool))
                    elif bn_members is not None and mod.groups == 1 and tuple(mod.dilation) == (1, 1):
                        # Conv2d -> BatchNorm2d(eval) with no neuron behind it: one folded convolution over all frames.
                        bn = gm.get_submodule(bn_members[0].target)
                        with torch.no_grad():
                            w, b = fold_bn_into_conv_params(mod.weight.float(), mod.bias, bn.running_mean.float(), bn.running_var.float(),
                                                            None if bn.weight is None else bn.weight.float(),
                                                            None if bn.bias is None else bn.bias.float(), bn.eps)
                        index = sum(1 for name, _ in gm.named_buffers() if name.startswith("folded_weight_"))
                        w_name = _register(gm, f"folded_weight_{index}", w.to(mod.weight.dtype).contiguous())
                        b_name = _register(gm, f"folded_bias_{index}", b.to(mod.weight.dtype).contiguous())
                        y_seq = graph.call_function(conv_bias_frames, (stack, graph.get_attr(w_name), graph.get_attr(b_name),
                                                                       list(mod.stride), list(mod.padding)))
                        targets = bn_members
                        removed += T
                    else:
                        flat = graph.call_method("flatten", (stack, 0, 1))
                        y = graph.call_module(key[1], (flat,))
                        y_seq = graph.call_method("unflatten", (y, 0, (T, -1)))
                elif key[0] == "add":
                    y_seq = graph.call_function(operator.add, (stacks[0], stacks[1]))
                else:
                    y_seq = graph.call_function(torch.flatten, (stack, 2))
            for t, node in targets.items():
                with graph.inserting_after(y_seq):
                    step = graph.call_function(operator.getitem, (y_seq, t))
                node.replace_all_uses_with(step)
            removed += T
            changed = True
        if changed:
            _emit_in_dependency_order(gm)
    # stack([y[0], ..., y[T-1]]) of one [T, ...] tensor is that tensor
    for node in list(gm.graph.nodes):
        if node.op == "call_function" and node.target is torch.stack and len(node.args) == 1 and not node.kwargs:
            parts = node.args[0]
            if (isinstance(parts, (list, tuple)) and parts and all(isinstance(p, fx.Node) and p.op == "call_function" and p.target is operator.getitem for p in parts)
                    and len({p.args[0] for p in parts}) == 1 and [p.args[1] for p in parts] == list(range(len(parts)))):
                whole = parts[0].args[0]
                steps = {u.args[1] for u in whole.users if u.op == "call_function" and u.target is operator.getitem}
                if steps == set(range(len(parts))):
                    node.replace_all_uses_with(whole)
    _emit_in_dependency_order(gm)
    gm.graph.lint()
    gm.recompile()
    return removed


# ---------------------------------------------------------------------------------------------------------------
# Internal layouts between the fused operators of one graph
# ---------------------------------------------------------------------------------------------------------------
# The reference's executor recognises fused convolution nodes of the rewritten graph and runs them on a faster entry point
# of the same backend, with pooled caller-owned buffers (runtime/fx_standalone_executor.py:900-952), and its rewrite is what
# hands it those nodes (compiler/fx_lif_temporal_rewrite.py:2037-2113, 2214-2333). The counterpart here is a pass over the
# rewritten graph: wherever a fused operator's [T, N, C, H, W] output is consumed by other operators the internal-layout
# kernels serve (fused convolutions, LIF-free convolutions, pools), the tensor between them travels bit-packed (spikes) or
# channel-blocked (analog values) as a `Blocked` value and the nodes call the internal-layout entry points
# (runtime/hip_blocked_backend.py); dense tensors remain at the graph's inputs and outputs and in front of every node the
# pass does not know. The graph functions below are the targets of the new nodes.
def blocked_input(frames, T: int, shared: bool, spikes: bool = False):
    """Graph input side: one analog frame [N, C, H, W] shared by all T steps (read as it is when it has at most 8 channels),
    or a dense [T, N, C, H, W] tensor (or the list of its T steps), into the channel-blocked layout; `spikes`: the tensor is
    the spike output of a fused operator (zeros and ones) and goes into the bit-packed layout."""
    from .runtime import hip_blocked_backend as B
    if shared:
        return B.input_frame(frames, T)
    if isinstance(frames, (list, tuple)):
        frames = torch.stack(list(frames))
    return B.from_dense(frames, B.BITS if spikes else B.C8)


def blocked_residual(frames):
    """A dense [T, N, C, H, W] tensor (or the list of its steps) as a residual operand: no conversion, the kernel reads
    dense residuals as they are."""
    from .runtime import hip_blocked_backend as B
    if isinstance(frames, (list, tuple)):
        frames = torch.stack(list(frames))
    return B.from_dense(frames, B.NCHW)


def blocked_conv_lif(x, weight, bias, stride, padding, lif, residual, out_layout: int):
    """Conv + folded BN (+ residual) + LIF over the T steps of a `Blocked` value, or without a neuron when `lif` is None."""
    from .runtime import hip_blocked_backend as B
    out, _ = B.conv_lif_blocked_or_dense(x, weight, bias, stride, padding, lif, residual=residual, out_layout=out_layout)
    return out


def blocked_conv_lif_shortcut(x, weight, bias, padding, lif, shortcut_x, shortcut_weight, shortcut_bias, shortcut_stride, out_layout: int):
    """The second convolution of a residual block with the block's 1x1 projection shortcut accumulated in the same launch
    (LIF(conv(x) + conv1x1(shortcut_x))); the two convolutions one after the other where the kernel does not take the pair."""
    from .runtime import hip_blocked_backend as B
    try:
        out, _ = B.conv_lif_blocked_shortcut(x, weight, bias, padding, shortcut_x, shortcut_weight, shortcut_bias, shortcut_stride, lif,
                                             out_layout=out_layout)
        return out
    except RuntimeError as exc:
        if "unsupported" not in str(exc):
            raise
    shortcut, _ = B.conv_lif_blocked_or_dense(shortcut_x, shortcut_weight, shortcut_bias, shortcut_stride, [0, 0], None, out_layout=B.C8)
    out, _ = B.conv_lif_blocked_or_dense(x, weight, bias, [1, 1], padding, lif, residual=shortcut, out_layout=out_layout)
    return out


def blocked_conv_lif_avgpool(x, weight, bias, stride, padding, lif):
    """Conv + folded BN + LIF and the 2x2 / 2 average pool of its spikes in one launch; the two one after the other where the
    kernel does not take the layer in that form."""
    from .runtime import hip_blocked_backend as B
    try:
        out, _ = B.conv_lif_blocked_avgpool(x, weight, bias, stride, padding, lif)
        return out
    except RuntimeError as exc:
        if "unsupported" not in str(exc):
            raise
    return blocked_pool(blocked_conv_lif(x, weight, bias, stride, padding, lif, None, B.BITS), False, 2, 2, 0)


def blocked_conv_lif_pool_linear(x, weight, bias, stride, padding, lif, residual, fc_weight, fc_bias, scale: float):
    """The network's last convolution with the tail's neuron in its epilogue (bit-packed spikes out), then average pool and
    classifier on those spikes, summed over T and scaled (1 / T: the mean over the timesteps): [N, K]. Where a kernel does
    not take the layer in this form, the convolution writes its sums dense and the LIF -> pool -> Linear operator follows."""
    from .runtime import hip_blocked_backend as B
    try:
        spikes, _ = B.conv_lif_blocked(x, weight, bias, stride, padding, lif, residual=residual, out_layout=B.BITS)
        return B.spike_pool_linear(spikes, fc_weight, fc_bias, scale)
    except RuntimeError as exc:
        if "unsupported" not in str(exc):
            raise
    sums, _ = B.conv_lif_blocked_or_dense(x, weight, bias, stride, padding, None, residual=residual, out_layout=B.NCHW)
    zero = torch.zeros((), dtype=torch.float32, device=sums.data.device)
    out_sum, _ = torch.ops.snn_custom.fused_temporal_lif_avgpool_linear(B.to_dense(sums), zero, fc_weight, fc_bias, *lif, False)
    return out_sum * scale


def blocked_pool(x, is_max: bool, kernel: int, stride: int, padding: int):
    from .runtime import hip_blocked_backend as B
    try:
        return B.pool_blocked(x, is_max, kernel, stride, padding)
    except RuntimeError as exc:
        if "unsupported" not in str(exc):
            raise
    y = pooled_frames(B.to_dense(x), is_max, kernel, stride, padding)
    return B.from_dense(y.contiguous(), x.layout if is_max else B.C8)


def blocked_to_dense(x):
    from .runtime import hip_blocked_backend as B
    return B.to_dense(x)


def _scalar_zero_node(gm: fx.GraphModule, node) -> bool:
    return _is_scalar_zero(gm, node)


def _sequence_source(arg, T_hint: Optional[int] = None):
    """What a list of per-timestep operands is made of: ("shared", frame node, T) for one node repeated, ("stack", node, T)
    for stack[0], ..., stack[T-1] in order, ("list", [nodes], T) otherwise; a single node stands for a whole stack."""
    if isinstance(arg, fx.Node):
        return ("stack", arg, T_hint)
    parts = list(arg)
    T = len(parts)
    if T > 1 and all(p is parts[0] for p in parts):
        return ("shared", parts[0], T)
    if (all(isinstance(p, fx.Node) and p.op == "call_function" and p.target is operator.getitem for p in parts)
            and len({p.args[0] for p in parts}) == 1 and [p.args[1] for p in parts] == list(range(T))):
        return ("stack", parts[0].args[0], T)
    return ("list", parts, T)


def propagate_internal_layouts(gm: fx.GraphModule) -> int:
    """Moves every chain fused operator -> (pool | LIF-free convolution) -> fused operator of a rewritten graph onto the
    internal layouts. Returns the number of nodes that now call an internal-layout entry point. A node is converted when
    it is a fused (residual) convolution from the scalar-zero membrane with nobody reading its final membrane, a
    `conv_bias_frames` / `pooled_frames` call, or the sum of a LIF-free convolution and a stack (folded into that
    convolution as its residual); everything else keeps reading dense tensors, converted once where needed."""
    from .runtime import hip_blocked_backend as B
    S = torch.ops.snn_custom
    conv_ops = {S.fused_temporal_conv_lif_state: False, S.fused_temporal_conv_lif_state.default: False,
                S.fused_temporal_conv_add_lif_state: True, S.fused_temporal_conv_add_lif_state.default: True}
    graph = gm.graph

    def fused_conv(node: fx.Node):
        """(has_residual, spike stack node) of a convertible fused convolution node, else None."""
        if node.op != "call_function" or node.target not in conv_ops or node.kwargs:
            return None
        res = conv_ops[node.target]
        a = node.args
        base = 2 if res else 1
        if len(a) != base + 11:
            return None
        w, b, v0, stride, padding, dilation, groups = a[base:base + 7]
        if not _scalar_zero_node(gm, v0) or list(dilation) != [1, 1] or int(groups) != 1:
            return None
        items = find_tuple_getitems(node)
        if len(node.users) != 1 or 0 not in items:
            return None                       # somebody reads the final membrane (or the tuple itself)
        return res, items[0]

    def pool_ok(node: fx.Node) -> bool:
        if node.op != "call_function" or node.target is not pooled_frames or node.kwargs or len(node.args) != 5:
            return False
        _, is_max, k, s, p = node.args
        return (bool(is_max) and k in (2, 3) and s == 2) or (not is_max and k == 2 and s == 2 and p == 0)

    def plain_conv_ok(node: fx.Node) -> bool:
        return node.op == "call_function" and node.target is conv_bias_frames and not node.kwargs and len(node.args) == 5

    def pretail_sum(node: fx.Node):
        """(conv_bias_frames node, other operand) when `node` adds a LIF-free convolution that nobody else reads to a stack."""
        if not _is_add_node(node) or len(node.args) != 2 or node.kwargs:
            return None
        for conv, other in ((node.args[0], node.args[1]), (node.args[1], node.args[0])):
            if isinstance(conv, fx.Node) and plain_conv_ok(conv) and len(conv.users) == 1 and isinstance(other, fx.Node):
                return conv, other
        return None

    # Phase 1: which nodes will read their operands as Blocked values (a node's own output layout depends on them).
    convertible = set()
    absorbed = set()        # LIF-free convolutions folded into the sum that follows them
    for node in graph.nodes:
        pair = pretail_sum(node)
        if pair is not None:
            convertible.add(node)
            absorbed.add(pair[0])
        elif fused_conv(node) is not None or pool_ok(node) or plain_conv_ok(node):
            convertible.add(node)
    convertible -= absorbed

    def reads_blocked(stack: fx.Node) -> Tuple[bool, bool]:
        """(some user reads the stack as a Blocked value, some user needs it dense)."""
        blocked = dense = False
        for user in stack.users:
            if user in absorbed:
                user = next(iter(user.users))
            if user.op == "call_function" and user.target is operator.getitem and isinstance(user.args[1], int):
                for leaf in user.users:
                    if leaf in convertible and fused_conv(leaf) is not None:
                        blocked = True
                    else:
                        dense = True
            elif user in convertible:
                blocked = True
            else:
                dense = True
        return blocked, dense

    blocked_of: Dict[fx.Node, fx.Node] = {}      # stack-level node -> node holding its Blocked value
    layout_of: Dict[fx.Node, int] = {}
    inputs: Dict[Tuple, fx.Node] = {}
    converted = 0

    def is_spike_stack(node) -> bool:
        """The stack is element 0 of a fused temporal operator that returns (spikes, membrane): zeros and ones."""
        if not (isinstance(node, fx.Node) and node.op == "call_function" and node.target is operator.getitem and node.args[1] == 0):
            return False
        producer = node.args[0]
        name = getattr(getattr(producer, "target", None), "__name__", "") or str(getattr(producer, "target", ""))
        return isinstance(producer, fx.Node) and producer.op == "call_function" and "fused_temporal" in name and "lif_state" in name

    def as_blocked(arg, residual: bool, T_hint=None) -> fx.Node:
        kind, src, T = _sequence_source(arg, T_hint)
        if kind == "stack" and src in blocked_of:
            return blocked_of[src]
        key = (kind, src if kind != "list" else tuple(src), residual)
        if key not in inputs:
            if residual:
                inputs[key] = graph.call_function(blocked_residual, (src if kind != "list" else list(src),))
            elif kind == "stack" and is_spike_stack(src):
                inputs[key] = graph.call_function(blocked_input, (src, T, False, True))
            else:
                inputs[key] = graph.call_function(blocked_input, (src if kind != "list" else list(src), T, kind == "shared"))
        return inputs[key]

    for node in list(graph.nodes):
        if node not in convertible:
            continue
        with graph.inserting_before(node):
            conv = fused_conv(node)
            pair = pretail_sum(node)
            if conv is not None:
                res, stack = conv
                base = 2 if res else 1
                w, b, _, stride, padding = node.args[base:base + 5]
                lif = tuple(node.args[base + 7:base + 10])
                wants_blocked, wants_dense = reads_blocked(stack)
                out_layout = B.BITS if wants_blocked or not wants_dense else B.NCHW
                xb = as_blocked(node.args[0], residual=False)
                rb = as_blocked(node.args[1], residual=True) if res else None
                new = graph.call_function(blocked_conv_lif, (xb, w, b, list(stride), list(padding), lif, rb, out_layout))
            elif pair is not None:
                stack = node
                plain, other = pair
                x_arg, w, b, stride, padding = plain.args
                wants_blocked, wants_dense = reads_blocked(stack)
                out_layout = B.C8 if wants_blocked else B.NCHW
                xb = as_blocked(x_arg, residual=False)
                rb = as_blocked(other, residual=True)
                new = graph.call_function(blocked_conv_lif, (xb, w, b, list(stride), list(padding), None, rb, out_layout))
            elif plain_conv_ok(node):
                stack = node
                x_arg, w, b, stride, padding = node.args
                wants_blocked, wants_dense = reads_blocked(stack)
                out_layout = B.C8 if wants_blocked or not wants_dense else B.NCHW
                new = graph.call_function(blocked_conv_lif, (as_blocked(x_arg, residual=False), w, b, list(stride), list(padding), None, None, out_layout))
            else:
                stack = node
                if node.args[0] not in blocked_of:
                    continue                      # a pool of a dense tensor stays on the dense pooling kernel
                new = graph.call_function(blocked_pool, (blocked_of[node.args[0]], *node.args[1:]))
            blocked_of[stack] = new
            converted += 1
    # Projection shortcuts: a LIF-free 1x1 convolution whose only reader is the residual operand of a plane-keeping fused
    # convolution becomes further K steps of that convolution (one launch, the shortcut's sums never stored).
    def weight_shape(arg):
        if isinstance(arg, fx.Node) and arg.op == "get_attr":
            value = gm
            for part in arg.target.split("."):
                value = getattr(value, part)
            return tuple(value.shape)
        return None

    for stack, node in list(blocked_of.items()):
        if node.target is not blocked_conv_lif or node.args[5] is None:
            continue
        x_main, w, b, stride, padding, lif, shortcut, out_layout = node.args
        if not (isinstance(shortcut, fx.Node) and shortcut.target is blocked_conv_lif and shortcut.args[5] is None and shortcut.args[6] is None):
            continue
        sc_stack = next((s for s, n in blocked_of.items() if n is shortcut), None)
        shape, sc_shape = weight_shape(w), weight_shape(shortcut.args[1])
        if (sc_stack is None or shape is None or sc_shape is None or len(shortcut.users) != 1 or reads_blocked(sc_stack)[1]
                or sc_shape[2:] != (1, 1) or list(shortcut.args[4]) != [0, 0] or list(stride) != [1, 1]
                or [2 * p + 1 for p in padding] != list(shape[2:]) or shape[1] % 16 or sc_shape[1] % 16):
            continue
        with graph.inserting_before(node):
            fused = graph.call_function(blocked_conv_lif_shortcut, (x_main, w, b, list(padding), lif, shortcut.args[0], shortcut.args[1],
                                                                    shortcut.args[2], list(shortcut.args[3]), out_layout))
        node.replace_all_uses_with(fused)
        blocked_of[stack] = fused
        del blocked_of[sc_stack]
        graph.erase_node(node)
        graph.erase_node(shortcut)
        converted -= 1
    # A 2x2 average pool that is the only reader of a fused convolution's spikes runs inside that convolution's launch.
    for stack, node in list(blocked_of.items()):
        if node.target is not blocked_pool or tuple(node.args[1:]) != (False, 2, 2, 0):
            continue
        conv = node.args[0]
        conv_stack = next((s for s, n in blocked_of.items() if n is conv), None)
        if (not isinstance(conv, fx.Node) or conv.target is not blocked_conv_lif or conv.args[5] is None or conv.args[6] is not None
                or conv.args[7] != B.BITS or len(conv.users) != 1 or conv_stack is None or reads_blocked(conv_stack)[1]):
            continue
        with graph.inserting_before(node):
            fused = graph.call_function(blocked_conv_lif_avgpool, tuple(conv.args[:6]))
        node.replace_all_uses_with(fused)
        blocked_of[stack] = fused
        del blocked_of[conv_stack]
        graph.erase_node(node)
        graph.erase_node(conv)
        converted -= 1
    # The tail: a LIF -> average pool -> Linear operator from the zero membrane whose only operand is a LIF-free convolution
    # that nobody else reads, and whose membrane nobody reads: the neuron fires in that convolution's epilogue and the pool
    # and the classifier run on the bit-packed spikes; a division of the logits by a constant (the mean over T) is folded in.
    tail_ops = (S.fused_temporal_lif_avgpool_linear, S.fused_temporal_lif_avgpool_linear.default)
    for tail in [n for n in graph.nodes if n.op == "call_function" and n.target in tail_ops]:
        if tail.kwargs or len(tail.args) != 8:
            continue
        stack, v0, fc_w, fc_b, v_th, v_reset, tau, detach = tail.args
        conv = blocked_of.get(stack) if isinstance(stack, fx.Node) else None
        items = find_tuple_getitems(tail)
        if (conv is None or conv.target is not blocked_conv_lif or conv.args[5] is not None or conv.args[7] != B.NCHW
                or not _scalar_zero_node(gm, v0) or len(stack.users) != 1 or len(tail.users) != 1 or 0 not in items):
            continue
        logits = items[0]
        scale, last = 1.0, logits
        if len(logits.users) == 1:
            user = next(iter(logits.users))
            if (user.op == "call_function" and user.target in (operator.truediv, torch.div) and user.args[0] is logits
                    and isinstance(user.args[1], (int, float)) and not user.kwargs and user.args[1] != 0):
                scale, last = 1.0 / float(user.args[1]), user
        with graph.inserting_before(tail):
            fused = graph.call_function(blocked_conv_lif_pool_linear, (*conv.args[:5], (v_th, v_reset, tau), conv.args[6], fc_w, fc_b, scale))
        last.replace_all_uses_with(fused)
        del blocked_of[stack]
        for dead in ([last] if last is not logits else []) + [logits, tail, conv]:
            graph.erase_node(dead)
    # Phase 2: whoever still reads a converted stack as a tensor gets it converted back (a no-op for dense outputs).
    for stack, new in blocked_of.items():
        with graph.inserting_after(new):
            dense = graph.call_function(blocked_to_dense, (new,))
        stack.replace_all_uses_with(dense)
    _emit_in_dependency_order(gm)
    gm.graph.lint()
    gm.recompile()
    return converted


def _emit_in_dependency_order(gm: fx.GraphModule) -> None:
    """Rebuilds the graph from its output backwards: dead nodes (the replaced per-timestep chains) disappear and every
    node lands after its operands, whatever position it was inserted at."""
    old = gm.graph
    new = fx.Graph()
    env: Dict[fx.Node, fx.Node] = {}
    for node in old.nodes:
        if node.op == "placeholder":
            env[node] = new.node_copy(node, lambda n: env[n])

    def emit(node: fx.Node) -> fx.Node:
        stack = [node]
        while stack:
            top = stack[-1]
            if top in env:
                stack.pop()
                continue
            pending = [a for a in top.all_input_nodes if a not in env]
            if pending:
                stack.extend(pending)
                continue
            env[top] = new.node_copy(top, lambda n: env[n])
            stack.pop()
        return env[node]

    output = next(n for n in old.nodes if n.op == "output")
    for dep in output.all_input_nodes:
        emit(dep)
    new.output(fx.node.map_arg(output.args[0], lambda n: env[n]))
    gm.graph = new


def compile_temporal(wrapper: nn.Module, tail_first: bool = False, device=None, dtype: Optional[torch.dtype] = None,
                     batch_time: bool = True, internal_layouts: bool = False, window: Optional[int] = None,
                     allow_tail: bool = True) -> Tuple[fx.GraphModule, RewriteStats]:
    """Traces `wrapper` (a module that runs a single-step spiking network T times on the same input and averages) and
    rewrites it to fused temporal operators. BatchNorm is folded with the parameters as they are at call time (fold in
    fp32, before any cast); `device` / `dtype` then move and cast the rewritten module (weights and activations in
    `dtype`, the membranes stay fp32). `tail_first`: give the neuron in front of the classifier to the
    LIF -> AvgPool -> Linear operator (its convolution then stays a plain layer); by default the convolution patterns
    claim it, as in the reference, whose tail rewrite only sees the neurons the convolution rewrites left over.
    `window` / `allow_tail`: fuse windows of that many consecutive timesteps instead of all T (the reference's
    `--temporal-fuse-window`); a window hands its final membrane to the layer's next step.
    `batch_time`: also merge the per-timestep calls of stateless layers into one call over T*N frames.
    `internal_layouts` (needs `batch_time`; the compiled module then runs on the GPU with bfloat16 / float16 tensors only):
    tensors between the graph's own fused operators, pools and LIF-free convolutions travel bit-packed / channel-blocked
    and those nodes call the internal-layout kernels (`propagate_internal_layouts`)."""
    gm = trace_single_step_loop(wrapper)
    stats = rewrite_temporal_to_fused(gm, tail_first=tail_first, window_size=window, allow_tail=allow_tail)
    if batch_time:
        stats.batched_timestep_calls = batch_timestep_calls(gm)
    if internal_layouts:
        if not batch_time:
            raise ValueError("internal_layouts needs batch_time: the pass works on whole [T, N, C, H, W] stacks")
        stats.internal_layout_nodes = propagate_internal_layouts(gm)
    if device is not None or dtype is not None:
        gm.to(device=device, dtype=dtype)
        for name, buf in list(gm.named_buffers()):
            if name.startswith("chronos_zero_membrane") or (buf.dim() == 0 and name.startswith("_tensor_constant")):
                setattr(gm, name, torch.zeros((), dtype=torch.float32, device=buf.device))
    return gm, stats
