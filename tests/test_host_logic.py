"""CPU-only tests: the C ABI library loads and exports what include/snnf.h declares, argument validation that returns
before any GPU work, the support predicates / kernel-key classification, and the operator layer's CPU, Meta and
statistics behaviour (counterparts of the reference's runtime/snn_custom_ops.py and runtime/triton_*_backend.py)."""
import ctypes
import os
import re

import pytest
import torch

from oracle import snn_oracle as O
from triton_snn_fusion_amd import _lib, workloads as W
from triton_snn_fusion_amd.runtime import hip_convlif_backend as CB
from triton_snn_fusion_amd.runtime import hip_temporal_lif_avgpool_linear_backend as TB
from triton_snn_fusion_amd.runtime import hip_temporal_lif_backend as LB
from triton_snn_fusion_amd.runtime import hip_temporal_linear_lif_backend as NB
from triton_snn_fusion_amd.runtime import snn_custom_ops as ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIF = (1.0, 0.0, 2.0)


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "snnf.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(snnf_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(snnf_lib):
    declared = _declared_symbols()
    assert len(declared) >= 11
    for name in declared:
        assert hasattr(snnf_lib, name), f"{name} declared in include/snnf.h but not exported by libsnnf.so"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes signature table and header disagree"
    assert snnf_lib.snnf_abi_version() == 1
    assert snnf_lib.snnf_status_string(0) == b"ok"
    assert snnf_lib.snnf_status_string(-2) == b"unsupported configuration"


def test_argument_validation_happens_before_any_gpu_work(snnf_lib):
    none = ctypes.POINTER(ctypes.c_void_p)()
    assert snnf_lib.snnf_lif_scan(none, 4, 128, 0, None, 0, None, 128, None, 1.0, 0.0, 2.0, None) == -1
    assert b"non-null" in snnf_lib.snnf_last_error()
    one = (ctypes.c_void_p * 1)(16)
    assert snnf_lib.snnf_lif_scan(one, 0, 128, 0, None, 0, 16, 128, 16, 1.0, 0.0, 2.0, None) == -1       # T = 0
    assert snnf_lib.snnf_lif_scan(one, 1, 128, 7, None, 0, 16, 128, 16, 1.0, 0.0, 2.0, None) == -1       # dtype code
    assert snnf_lib.snnf_lif_scan(one, 1, 128, 0, None, 0, 16, 128, 16, 1.0, 0.0, 0.0, None) == -2       # tau = 0
    assert snnf_lib.snnf_lif_scan(one, 1, 0, 0, None, 0, 16, 0, 16, 1.0, 0.0, 2.0, None) == 0            # empty input
    assert snnf_lib.snnf_dwconv3x3_lif(one, None, 1, 1, 8, 8, 8, 3, 0, 16, 16, 0, None, 0, 16, 512, 16, 1.0, 0.0, 2.0, None) == -2
    assert b"unsupported_stride" in snnf_lib.snnf_last_error()
    assert snnf_lib.snnf_conv_lif(one, None, 1, 1, 8, 8, 8, 0, 16, 8, 3, 3, 1, 1, 2, 2, None, 0, 16, 512, 16, 1.0, 0.0, 2.0, None) == -2
    assert b"unsupported_padding" in snnf_lib.snnf_last_error()
    assert snnf_lib.snnf_lif_pool_linear(one, 1, 2, 8, 7, 7, 0, None, 0, 16, None, 10, 0, 16, 16, None, 0, 1.0, 0.0, 2.0, None) == -4
    assert snnf_lib.snnf_linear_lif(one, 1, 4, 0, 0, 0, 16, None, 8, 0, None, 0, 16, 32, 16, 1.0, 0.0, 2.0, None) == -1


def test_packed_weight_size_is_whole_fragments(snnf_lib):
    # [ceil(Cout/32)][ceil(Cin/CK)][ceil(taps * CK/8 / 2)] fragments of 1 KiB + the fp32 bias, padded with zeros to whole
    # 64-channel tiles plus one tile (the kernels load a tile's bias without a bounds check)
    def bias_bytes(cout):
        nocf = (cout + 31) // 32
        return (((nocf + 1) // 2) * 64 + 64) * 4
    assert snnf_lib.snnf_conv_packed_weight_bytes(64, 64, 3, 3, 1) == 2 * 2 * 18 * 1024 + bias_bytes(64)
    # fp32 tensors: 16-channel chunks, and three parts of the channel axis (w_hi, w_lo, w_hi: two bf16 terms per operand)
    assert snnf_lib.snnf_conv_packed_weight_bytes(64, 64, 3, 3, 0) == 3 * 2 * 4 * 9 * 1024 + bias_bytes(64)
    assert snnf_lib.snnf_conv_packed_weight_bytes(64, 3, 7, 7, 1) == 2 * 1 * 25 * 1024 + bias_bytes(64)
    assert snnf_lib.snnf_conv_packed_weight_bytes(70, 40, 1, 1, 2) == 3 * 1 * 4 * 1024 + bias_bytes(70)     # pointwise: one 64-channel chunk
    assert snnf_lib.snnf_lif_pool_linear_workspace_bytes(16, 512) == 16 * 512 * 4
    assert snnf_lib.snnf_conv_packed_weight_bytes(0, 3, 3, 3, 1) == 0


def test_which_tails_run_as_one_launch(snnf_lib):
    """The tail runs as one launch (a workgroup per sample and class range) when a sample is small, its channels come in whole
    vectors of 8 and fit the workgroup's counters; otherwise as the pooling launch followed by the classifier launch."""
    f = snnf_lib.snnf_lif_pool_linear_launches
    assert f(4, 64, 512, 1, 1, 10) == 1            # VGG-11's tail
    assert f(4, 4, 512, 2, 2, 1000) == 1
    assert f(16, 5, 64, 4, 4, 100) == 1
    assert f(4, 16, 512, 7, 7, 1000) == 2          # ResNet-18's tail: 100 k neuron steps per sample
    assert f(4, 64, 512, 28, 28, 1000) == 2
    assert f(4, 3, 30, 7, 7, 10) == 2              # channels no multiple of 8
    assert f(4, 3, 8, 3, 3, 10) == 1 and f(4, 3, 8, 3, 5, 10) == 1 and f(4, 3, 24, 3, 3, 10) == 1
    assert f(2, 2, 4096, 1, 1, 10) == 2            # more channels than counters
    assert f(0, 1, 8, 1, 1, 1) == 0 and f(4, 1, 8, 1, 1, 0) == 0


@pytest.mark.parametrize("shape,stride,padding,groups,key", [
    ((8, 4, 1, 1), (1, 1), (0, 0), 1, "k1_s1_p0"),
    ((8, 4, 3, 3), (1, 1), (1, 1), 1, "k3_s1_p1"),
    ((8, 4, 3, 3), (2, 2), (1, 1), 1, "k3_s2_p1"),
    ((8, 4, 5, 5), (1, 1), (2, 2), 1, "k5_s1_p2"),
    ((8, 3, 7, 7), (2, 2), (3, 3), 1, "k7_s2_p3"),
    ((8, 3, 11, 11), (4, 4), (2, 2), 1, "k11_s4_p2"),
    ((8, 1, 3, 3), (1, 1), (1, 1), 8, "depthwise_k3_s1_p1"),
    ((8, 1, 3, 3), (2, 2), (1, 1), 8, "depthwise_k3_s2_p1"),
    ((8, 1, 5, 5), (1, 1), (2, 2), 8, "unsupported"),
    ((8, 2, 3, 3), (1, 1), (1, 1), 2, "unsupported"),
    ((8, 4, 3, 3), (1, 1), (0, 0), 1, "k3x3_s1x1_p0x0"),
    ((8, 4, 3, 3), (1, 1), (2, 2), 1, "unsupported"),
])
def test_classify_conv_lif_config(shape, stride, padding, groups, key):
    w = torch.empty(shape, device="meta")
    assert CB.classify_conv_lif_config(w, stride, padding, (1, 1), groups) == key
    assert CB.classify_conv_lif_config(w, stride, padding, (2, 2), groups) == "unsupported"
    kind = CB.classify_conv_lif_runtime_kind(w, stride, padding, (1, 1), groups)
    assert kind == ("depthwise" if key.startswith("depthwise") else "pointwise" if key == "k1_s1_p0"
                    else "unsupported" if key == "unsupported" else "regular")


def test_conv_support_reasons_use_the_reference_prefixes():
    x = torch.empty(2, 4, 8, 8)
    w, b, v = torch.empty(8, 4, 3, 3), torch.empty(8), torch.tensor(0.0)
    r = CB.check_triton_support(x, w, b, v, (1, 1), (1, 1), (1, 1), 1, *LIF, False)
    assert r == ["unsupported_device: x is not CUDA"]
    xm, wm, bm, vm = (t.to("meta") for t in (x, w, b, v))

    def reasons(**kw):
        args = dict(x=xm, weight=wm, bias=bm, v_prev=vm, stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1)
        args.update(kw)
        out = CB.check_triton_support(args["x"], args["weight"], args["bias"], args["v_prev"], args["stride"],
                                      args["padding"], args["dilation"], args["groups"], *LIF, False)
        return [t.split(":")[0] for t in out if not t.startswith("unsupported_device")]

    assert reasons() == []
    assert reasons(dilation=(2, 2)) == ["unsupported_dilation"]
    assert reasons(groups=2) == ["unsupported_groups"]
    assert reasons(bias=None) == ["missing_or_unsupported_bias"]
    assert reasons(weight=wm.to(torch.float16)) == ["unsupported_dtype"]
    assert reasons(x=xm.to(torch.float64), weight=wm.to(torch.float64), bias=bm.to(torch.float64)) == ["unsupported_dtype"]
    assert reasons(padding=(2, 2)) == ["unsupported_padding"]
    assert reasons(v_prev=torch.empty(2, 8, 4, 4, device="meta")) == ["v_prev shape (2, 8, 4, 4) does not match conv output shape (2, 8, 8, 8)"]
    assert reasons(x=xm.to(torch.bfloat16), weight=wm.to(torch.bfloat16), bias=bm.to(torch.bfloat16)) == []   # fp32 membrane next to bf16
    dw = torch.empty(4, 1, 3, 3, device="meta")
    assert reasons(weight=dw, bias=torch.empty(4, device="meta"), groups=4, stride=(3, 3)) == ["unsupported_stride"]


def test_other_support_predicates():
    x = torch.empty(4, 2, 3, 5, 5, device="meta")
    v = torch.tensor(0.0, device="meta")
    assert [r.split(":")[0] for r in LB.check_temporal_lif_support(x, v, *LIF, False)] == ["unsupported_device"]
    assert "unsupported_rank" in " ".join(LB.check_temporal_lif_support(x[0], v, *LIF, False))
    assert "unsupported_tau" in " ".join(LB.check_temporal_lif_support(x, v, 1.0, 0.0, 0.0, False))
    assert "unsupported_membrane_state" in " ".join(LB.check_temporal_lif_support(x, torch.empty(2, 3, 5, 4, device="meta"), *LIF, False))
    fw, fb = torch.empty(10, 3, device="meta"), torch.empty(10, device="meta")
    assert [r.split(":")[0] for r in TB.check_temporal_lif_avgpool_linear_support(x, v, fw, fb, 2.0)] == ["unsupported_device"]
    assert "unsupported_linear" in " ".join(TB.check_temporal_lif_avgpool_linear_support(x, v, torch.empty(10, 4, device="meta"), fb, 2.0))
    xl = torch.empty(4, 6, 32, device="meta")
    lw = torch.empty(16, 32, device="meta")
    assert [r.split(":")[0] for r in NB.check_temporal_linear_lif_support(xl, lw, None, v, *LIF, False)] == ["unsupported_device"]
    assert "unsupported_shape" in " ".join(NB.check_temporal_linear_lif_support(xl, torch.empty(16, 31, device="meta"), None, v, *LIF, False))
    assert "unsupported_bias" in " ".join(NB.check_temporal_linear_lif_support(xl, lw, torch.empty(15, device="meta"), v, *LIF, False))
    assert TB.run_triton_fused_temporal_lif_tail is TB.run_triton_fused_temporal_lif_avgpool_linear


def test_backends_accept_use_autotune_and_raise_reason_strings_on_cpu_tensors():
    x = torch.rand(2, 1, 3, 4, 4)
    with pytest.raises(RuntimeError, match="unsupported_device"):
        LB.run_triton_fused_temporal_lif_state(x, torch.tensor(0.0), *LIF, False, strict=False, verbose=False, use_autotune=True)
    with pytest.raises(RuntimeError, match=r"\[HIP\]\[STRICT\]"):
        TB.run_triton_fused_temporal_lif_avgpool_linear(x, torch.tensor(0.0), torch.rand(5, 3), torch.rand(5), *LIF, False, strict=True, use_autotune=False)
    with pytest.raises(RuntimeError, match="xs must be a non-empty"):
        CB.run_triton_fused_temporal_conv_lif_state([], torch.rand(4, 3, 3, 3), torch.rand(4), torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *LIF, False)
    with pytest.raises(RuntimeError, match="compute_dtype"):
        CB._check_compute_dtype("float16", torch.float32)


def test_configure_and_stats_vocabulary():
    with pytest.raises(ValueError):
        ops.configure_fused_op("cuda")
    for name in ("torch", "triton", "hip"):
        ops.configure_fused_op(name)
    ops.configure_fused_op("torch")
    ops.reset_fused_op_call_stats()
    stats = ops.get_fused_op_call_stats()
    for key in ("total", "triton", "fallback", "temporal_k3_s1_p1", "temporal_lif_tail_total", "kernel_temporal_configs",
                "temporal_conv_lif_runtime_by_signature", "fallback_reasons"):
        assert key in stats
    assert ops._reason_key(["3x3 only"]) == "unsupported_kernel_size"
    assert ops._reason_key(["bad tau"]) == "unsupported_tau"
    assert ops._fallback_reason_keys(["unsupported_stride: nope", "weird"]) == ["other_unsupported", "unsupported_stride"]


def _conv_case():
    g = torch.Generator().manual_seed(0)
    xs = [(torch.rand(2, 4, 9, 9, generator=g) < 0.3).float() for _ in range(3)]
    w, b = torch.randn(6, 4, 3, 3, generator=g) * 0.4, torch.randn(6, generator=g) * 0.1
    return xs, w, b


@pytest.mark.parametrize("backend", ["torch", "hip"])
def test_cpu_tensors_run_the_eager_ops_and_match_the_oracle(backend):
    ops.configure_fused_op(backend)
    ops.reset_fused_op_call_stats()
    try:
        xs, w, b = _conv_case()
        v0 = torch.tensor(0.0)
        ref = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (1, 1), (1, 1), 1, *LIF)
        s, v = torch.ops.snn_custom.fused_temporal_conv_lif_state(xs, w, b, v0, [1, 1], [1, 1], [1, 1], 1, *LIF, False)
        assert torch.equal(s, ref[0]) and torch.equal(v, ref[1])
        s_tn, _ = torch.ops.snn_custom.fused_temporal_conv_lif_state_batched_tn(xs, w, b, v0, [1, 1], [1, 1], [1, 1], 1, *LIF, False)
        assert torch.equal(s_tn, ref[0].flatten(0, 1))
        rs = [torch.randn(2, 6, 9, 9) * 0.2 for _ in range(3)]
        ref_r = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (1, 1), (1, 1), 1, *LIF, residuals=rs)
        s_r, v_r = torch.ops.snn_custom.fused_temporal_conv_add_lif_state(xs, rs, w, b, v0, [1, 1], [1, 1], [1, 1], 1, *LIF, False)
        assert torch.equal(s_r, ref_r[0]) and torch.equal(v_r, ref_r[1])
        x_seq = torch.stack(xs)
        so, vo = torch.empty_like(ref[0]), torch.empty_like(ref[1])
        assert torch.ops.snn_custom.fused_temporal_conv_lif_state_packed_out(x_seq, w, b, v0, [1, 1], [1, 1], [1, 1], 1, *LIF, False, so, vo) is None
        assert torch.equal(so, ref[0]) and torch.equal(vo, ref[1])
        ref_l = O.temporal_lif(x_seq * 1.7, v0, *LIF)
        s_l, v_l = torch.ops.snn_custom.fused_temporal_lif_state(x_seq * 1.7, v0, *LIF, False)
        assert torch.equal(s_l, ref_l[0]) and torch.equal(v_l, ref_l[1])
        fw, fb = torch.randn(5, 4), torch.randn(5)
        ref_t = O.temporal_lif_avgpool_linear(x_seq * 1.7, v0, fw, fb, *LIF)
        for op in (torch.ops.snn_custom.fused_temporal_lif_avgpool_linear, torch.ops.snn_custom.fused_temporal_lif_tail):
            o_t, v_t = op(x_seq * 1.7, v0, fw, fb, *LIF, False)
            assert torch.allclose(o_t, ref_t[0], atol=1e-6) and torch.equal(v_t, ref_t[1])
        xl = (torch.rand(3, 5, 12) < 0.3).float()
        lw = torch.randn(7, 12)
        ref_n = O.temporal_linear_lif(xl, lw, None, v0, *LIF)
        s_n, v_n = torch.ops.snn_custom.fused_temporal_linear_lif_state([xl[t] for t in range(3)], lw, None, v0, *LIF, False)
        s_p, v_p = torch.ops.snn_custom.fused_temporal_linear_lif_state_packed(xl, lw, None, v0, *LIF, False)
        assert torch.equal(s_n, ref_n[0]) and torch.equal(s_p, ref_n[0]) and torch.equal(v_n, ref_n[1]) and torch.equal(v_p, ref_n[1])
        stats = ops.get_fused_op_call_stats()
        assert stats["triton"] == 0 and stats["fallback"] == stats["total"] == 9
        assert stats["temporal_lif_avgpool_linear_total"] == 2 and stats["temporal_lif_tail_fallback"] == 2
        assert stats["temporal_batched_output_total"] == 1 and stats["temporal_residual_total"] == 1
        key = "temporal_dispatch:other_unsupported"
        assert stats["fallback_reasons"][key] >= 1
        sig = "temporal:k3x3_s1x1_p1x1_d1x1_g1_ic4_oc6_standard"
        assert stats["temporal_conv_lif_runtime_by_signature"][sig]["fallback"] >= 2
    finally:
        ops.configure_fused_op("torch")


def test_meta_shapes_and_membrane_dtype_rule():
    m = lambda *s, dtype=torch.float32: torch.empty(tuple(s), device="meta", dtype=dtype)
    xs = [m(2, 4, 9, 9, dtype=torch.bfloat16) for _ in range(3)]
    w, b = m(6, 4, 3, 3, dtype=torch.bfloat16), m(6, dtype=torch.bfloat16)
    s, v = torch.ops.snn_custom.fused_temporal_conv_lif_state(xs, w, b, m(dtype=torch.float32), [2, 2], [1, 1], [1, 1], 1, *LIF, False)
    assert tuple(s.shape) == (3, 2, 6, 5, 5) and s.dtype == torch.bfloat16 and tuple(v.shape) == (2, 6, 5, 5) and v.dtype == torch.float32
    s, v = torch.ops.snn_custom.fused_temporal_conv_lif_state(xs, w, b, m(dtype=torch.bfloat16), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    assert v.dtype == torch.bfloat16
    s, v = torch.ops.snn_custom.fused_temporal_conv_add_lif_state_batched_tn(xs, [m(2, 6, 9, 9)] * 3, w, b, m(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    assert tuple(s.shape) == (6, 6, 9, 9)
    s, v = torch.ops.snn_custom.fused_temporal_linear_lif_state_packed(m(4, 2, 3, 16), m(8, 16), None, m(), *LIF, False)
    assert tuple(s.shape) == (4, 2, 3, 8) and tuple(v.shape) == (2, 3, 8)
    o, v = torch.ops.snn_custom.fused_temporal_lif_avgpool_linear(m(4, 2, 16, 7, 7), m(), m(10, 16), m(10), *LIF, False)
    assert tuple(o.shape) == (2, 10) and tuple(v.shape) == (2, 16, 7, 7)
    s, v = torch.ops.snn_custom.fused_conv_lif_state(xs[0], w, b, m(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    assert tuple(s.shape) == (2, 6, 9, 9)
    with pytest.raises(RuntimeError):
        torch.ops.snn_custom.fused_temporal_lif_state(m(2, 3, 4), m(), *LIF, False)


def test_operator_names_and_schemas_are_the_reference_abi():
    expected = {
        "lif_forward_state", "fused_conv_lif_state", "fused_temporal_conv_lif_state",
        "fused_temporal_pointwise_conv_lif_state", "fused_temporal_depthwise_conv_lif_state",
        "fused_temporal_conv_lif_state_depthwise", "fused_temporal_conv_lif_state_packed_out",
        "fused_temporal_conv_lif_state_batched_tn", "fused_temporal_conv_add_lif_state",
        "fused_temporal_conv_add_lif_state_depthwise", "fused_temporal_conv_add_lif_state_batched_tn",
        "fused_temporal_lif_state", "fused_temporal_lif_avgpool_linear", "fused_temporal_linear_lif_state",
        "fused_temporal_linear_lif_state_packed", "fused_temporal_linear_lif_state_packed_out", "fused_temporal_lif_tail",
    }
    assert set(ops.OPERATORS) == expected
    for name in expected:
        assert str(getattr(torch.ops.snn_custom, name).default) == f"snn_custom.{name}.default"
    # Every schema, argument for argument, against the fixture written from the reference's definitions
    # (runtime/snn_custom_ops.py:1966-2073).
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "op_schemas.json")) as f:
        fixture = json.load(f)["schemas"]
    assert set(fixture) == expected
    for name, schema in fixture.items():
        assert str(getattr(torch.ops.snn_custom, name).default._schema) == schema, name


def test_workloads_are_seeded_and_bn_fold_is_exact_algebra():
    a, b = W.conv3x3_block(batch=1, size=8), W.conv3x3_block(batch=1, size=8)
    assert torch.equal(a.x_seq, b.x_seq) and torch.equal(a.conv_layers[0].weight, b.conv_layers[0].weight)
    assert set(a.x_seq.unique().tolist()) == {0.0, 1.0}
    assert abs(float(W.conv3x3_block().x_seq.mean()) - 0.2) < 0.01
    wl = W.mobilenet_block(batch=1, size=8)
    assert tuple(wl.conv_layers[0].weight.shape) == (128, 1, 3, 3) and wl.conv_layers[0].groups == 128
    assert tuple(wl.conv_layers[1].weight.shape) == (256, 128, 1, 1)
    lin = W.linear_block()
    assert tuple(lin.x_seq.shape) == (8, 64, 2048) and tuple(lin.linear_weight.shape) == (1024, 2048)
    g = torch.Generator().manual_seed(1)
    w, cb = torch.randn(4, 3, 3, 3, generator=g), torch.randn(4, generator=g)
    mean, var, gamma, beta = torch.randn(4, generator=g), torch.rand(4, generator=g) + 0.5, torch.rand(4, generator=g) + 0.5, torch.randn(4, generator=g)
    got = W.fold_bn_into_conv_params(w, cb, mean, var, gamma, beta, 1e-5)
    want = O.fold_bn(w, cb, mean, var, gamma, beta, 1e-5)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    # C0 algorithmic traffic: x 8.39 MB + spikes 8.39 MB + v 2.10 MB + weights 0.15 MB (fp32 I/O)
    nbytes = W.algorithmic_conv_bytes(4, 8, 64, 32, 32, 64, 32, 32, 3, 3, 1, 4, 4)
    assert abs(nbytes - 19.02e6) < 0.02e6
    assert W.conv_flops(4, 8, 64, 64, 32, 32, 3, 3, 1) == 2415919104


def test_eager_and_meta_functions_agree_on_the_membrane_dtype():
    """One rule for native kernels, eager functions and meta functions: a v_init on the activations' device with dtype
    float32 or the activation dtype chooses the membrane dtype, anything else gives the activation dtype."""
    import torch
    from triton_snn_fusion_amd.runtime import snn_custom_ops as ops
    S = torch.ops.snn_custom
    x = [(torch.rand(2, 4, 6, 6) < 0.3).to(torch.bfloat16) for _ in range(3)]
    w, b = torch.randn(4, 4, 3, 3).to(torch.bfloat16), torch.zeros(4, dtype=torch.bfloat16)
    geo = ([1, 1], [1, 1], [1, 1], 1)
    lif = (1.0, 0.0, 2.0, False)
    for v_init, want in ((torch.zeros(2, 4, 6, 6), torch.float32), (torch.zeros(()), torch.float32),
                         (torch.zeros((), dtype=torch.bfloat16), torch.bfloat16), (torch.zeros(2, 4, 6, 6, dtype=torch.bfloat16), torch.bfloat16),
                         (torch.zeros((), dtype=torch.float64), torch.bfloat16)):
        s, v = S.fused_temporal_conv_lif_state(x, w, b, v_init, *geo, *lif)
        ms, mv = S.fused_temporal_conv_lif_state([t.to("meta") for t in x], w.to("meta"), b.to("meta"), v_init.to("meta"), *geo, *lif)
        assert v.dtype == want == mv.dtype and s.dtype == torch.bfloat16 == ms.dtype and mv.shape == v.shape
        s1, v1 = S.lif_forward_state(x[0], v_init, *lif)
        m1 = S.lif_forward_state(x[0].to("meta"), v_init.to("meta"), *lif)
        assert v1.dtype == want == m1[1].dtype
    # a float32 membrane next to 16-bit activations is stepped in float32: chaining two windows equals one call
    v0 = torch.randn(2, 4, 6, 6) * 0.3
    s_all, v_all = S.fused_temporal_conv_lif_state(x, w, b, v0, *geo, *lif)
    s_a, v_a = S.fused_temporal_conv_lif_state(x[:1], w, b, v0, *geo, *lif)
    s_b, v_b = S.fused_temporal_conv_lif_state(x[1:], w, b, v_a, *geo, *lif)
    assert torch.equal(torch.cat([s_a, s_b]), s_all) and torch.equal(v_b, v_all) and v_all.dtype == torch.float32


def test_tuned_plan_table_is_well_formed():
    """The measured launch choices shipped with the package: every entry names a layer shape completely and a choice the
    registration call accepts."""
    import json
    from pathlib import Path
    path = Path(__file__).resolve().parents[1] / "triton-snn-fusion_amd" / "runtime" / "tuned_blocked_plans.json"
    table = json.loads(path.read_text())
    assert table["dtype"] == "bf16" and isinstance(table["layers"], list)
    seen = set()
    for e in table["layers"]:
        key = (e["T"], e["N"], e["Cin"], e["H"], e["W"], e["Cout"], *e["kernel"], *e["stride"], *e["padding"], bool(e["shared_frame"]))
        assert len(key) == 13 and key not in seen
        seen.add(key)
        assert 0 <= e["patch_cols"] <= 32 and e["stage_groups"] in (0, 2, 4, 8) and e["k_waves"] in (0, 1, 2, 4, 8)
        assert e["us"] < e["planner_us"]


def test_which_16_bit_membrane_calls_run_with_a_float32_working_membrane():
    """Calls that may take several launches compute with a float32 membrane and round once at the end: depthwise above 16
    timesteps, and every multi-step call of the other convolution kernels (their launch count depends on the membrane
    dtype itself, so the rule must not depend on what an earlier call of the layer recorded)."""
    assert not CB._takes_several_launches("depthwise_k3_s1_p1", 16)
    assert CB._takes_several_launches("depthwise_k3_s1_p1", 17)
    assert CB._takes_several_launches("k3_s1_p1", 4)
    assert CB._takes_several_launches("k1_s1_p0", 2)


def _reference_start_membrane(x, v_prev):
    """The reference's rule for the membrane a step starts from (runtime/snn_custom_ops.py:378-381), restated: a `v_prev`
    that is no tensor of the shape, device and dtype of `x` is replaced by zeros like `x`."""
    if not isinstance(v_prev, torch.Tensor) or v_prev.shape != x.shape or v_prev.device != x.device or v_prev.dtype != x.dtype:
        return torch.zeros_like(x)
    return v_prev


def test_float32_state_next_to_16_bit_activations_both_rules():
    """Where this package departs from the reference, pinned side by side: a full-shape float32 `v_prev` next to 16-bit
    activations restarts from zeros (16-bit membrane out) under the reference's rule and is carried in float32 here; every
    other mismatch (0-dim placeholder, wrong shape, a third dtype) restarts from zeros under both rules (here in float32 when
    `v_prev` is a float32 tensor on the activations' device), and a state of the activation dtype is carried under both."""
    g = torch.Generator().manual_seed(5)
    lif = (1.0, 0.0, 2.0)
    x = (torch.randn(2, 3, 4, 4, generator=g) * 1.5).to(torch.bfloat16)
    v32 = torch.randn(2, 3, 4, 4, generator=g) * 0.5
    # the reference's rule on this input: the float32 state is dropped
    v_ref = _reference_start_membrane(x, v32)
    assert v_ref.dtype == torch.bfloat16 and not v_ref.any()
    s_ref, m_ref = ops._lif_step_torch(x, v_ref, x.dtype, *lif, False)
    # this package: carried, stepped and returned in float32
    s_here, m_here = ops.lif_forward_state_torch(x, v32, *lif, False)
    assert m_here.dtype == torch.float32 and s_here.dtype == torch.bfloat16
    want_s, want_m = ops._lif_step_torch(x.float(), v32, x.dtype, *lif, False)
    assert torch.equal(s_here, want_s) and torch.equal(m_here, want_m)
    assert not torch.equal(m_here.to(torch.bfloat16), m_ref)          # the two rules give different states on this input
    assert ops._lif_forward_state_meta(x.to("meta"), v32.to("meta"), *lif, False)[1].dtype == torch.float32
    # mismatches that restart from zeros under both rules. The membrane dtype here follows the dtype and device of `v_prev`
    # alone (float32 or the activations' dtype on the activations' device, else the activations' dtype), the reference's is
    # always the activations': a 0-dim float32 zero or a float32 tensor of another shape gives the zero start in float32,
    # a third dtype gives it in the activation dtype.
    for v_other, want_dtype in ((torch.tensor(0.0), torch.float32), (torch.zeros(2, 3, 4, 5), torch.float32),
                                (v32.to(torch.float16), torch.bfloat16), (v32.double(), torch.bfloat16),
                                (torch.tensor(0.0, dtype=torch.bfloat16), torch.bfloat16)):
        assert not _reference_start_membrane(x, v_other).any()
        s_o, m_o = ops.lif_forward_state_torch(x, v_other, *lif, False)
        want_s, want_m = ops._lif_step_torch(x.to(want_dtype), torch.zeros(x.shape, dtype=want_dtype), x.dtype, *lif, False)
        assert m_o.dtype == want_dtype and torch.equal(s_o, want_s) and torch.equal(m_o, want_m)
        if want_dtype == torch.bfloat16:
            assert torch.equal(s_o, s_ref) and torch.equal(m_o, m_ref)      # exactly the reference's result
    # a state of the activation dtype is carried under both rules
    v16 = v32.to(torch.bfloat16)
    assert _reference_start_membrane(x, v16) is v16
    s_c, m_c = ops.lif_forward_state_torch(x, v16, *lif, False)
    want_s, want_m = ops._lif_step_torch(x, v16, x.dtype, *lif, False)
    assert m_c.dtype == torch.bfloat16 and torch.equal(s_c, want_s) and torch.equal(m_c, want_m)
