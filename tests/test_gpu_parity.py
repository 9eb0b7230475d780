"""GPU parity tests: every fused operator, called through torch.ops.snn_custom (-> ctypes -> libsnnf C ABI -> HIP
kernel), against the CPU oracle on the same seeded operands.

Gate (tests/helpers.py:check): membrane within rtol 1e-3 / atol 1e-4; spike mismatches only where the oracle's pre-reset
membrane is within 1e-3 of the threshold, at a rate <= 1e-4. 16-bit and fp32-on-matrix-core runs are compared with the
oracle evaluated in fp32 on operands rounded the way the kernel rounds them (bf16 matrix operands, fp32 accumulate).
"""
import ctypes
import json
import os

import pytest
import torch

from helpers import DEV, LIF, check, dev, gen, q, spikes, zero_v
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
S = torch.ops.snn_custom


def _no_fallback(ops, expected_calls=None):
    stats = ops.get_fused_op_call_stats()
    assert stats["fallback"] == 0, stats["fallback_reasons"]
    if expected_calls is not None:
        assert stats["triton"] == expected_calls, stats


# ---------------------------------------------------------------------------------------------------------------
# Standalone temporal LIF
# ---------------------------------------------------------------------------------------------------------------
def test_lif_scan_known_answer_traces_through_the_c_abi(snnf_lib):
    """tests/golden/lif_kat.json straight through snnf_lif_scan, bit exact (fp32 in, fp32 membrane)."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd import _lib
    cases = json.load(open(os.path.join(GOLDEN, "lif_kat.json")))["cases"]
    groups = {}
    for c in cases:
        groups.setdefault((c["v_threshold"], c["v_reset"], c["tau"], len(c["x"])), []).append(c)
    for (v_th, v_reset, tau, T), members in groups.items():
        x = torch.tensor([m["x"] for m in members], dtype=F32).t().contiguous().to(DEV)       # [T, n]
        v0 = torch.tensor([m["v0"] for m in members], dtype=F32).to(DEV)
        n = len(members)
        out_s = torch.empty(T, n, device=DEV)
        out_v = torch.empty(n, device=DEV)
        rc = snnf_lib.snnf_lif_scan(_lib.packed_step_pointers(x), T, n, 0, v0.data_ptr(), 0, out_s.data_ptr(), n,
                                    out_v.data_ptr(), v_th, v_reset, tau, _lib.current_stream(x.device))
        assert rc == 0, snnf_lib.snnf_last_error()
        torch.cuda.synchronize()
        assert out_s.t().cpu().tolist() == [[float(k) for k in m["spikes"]] for m in members]
        assert out_v.cpu().tolist() == [m["v"] for m in members]


@pytest.mark.parametrize("dtype,vdtype", [(F32, F32), (BF16, F32), (BF16, BF16), (F16, F32), (F16, F16)])
@pytest.mark.parametrize("T,shape", [(1, (2, 3, 5, 7)), (4, (2, 8, 14, 14)), (8, (1, 16, 7, 7)), (16, (2, 4, 8, 8)), (20, (1, 3, 9, 5))])
def test_temporal_lif(hip_ops, dtype, vdtype, T, shape):
    g = gen(100 + T)
    x = q(torch.randn((T,) + shape, generator=g) * 0.75 + 0.15, dtype)
    v0 = q(torch.randn(shape, generator=g) * 0.3, vdtype)
    ref = O.temporal_lif(x, v0, *LIF)
    s, v = S.fused_temporal_lif_state(dev(x, dtype), dev(v0, vdtype), *LIF, False)
    assert s.dtype == dtype and v.dtype == vdtype and s.shape == x.shape
    rep = check(s, v, ref, v_dtype=vdtype, what=f"lif {dtype} {vdtype} T={T}")
    assert rep["near_threshold_flips"] == 0          # elementwise fp32 math: bit exact
    _no_fallback(hip_ops, 1)


@pytest.mark.parametrize("v_th,v_reset,tau", [(1.0, -1.0, 2.0), (0.5, 0.0, 1.0), (1.0, 0.25, 4.0), (0.75, 0.0, 1.5), (1.0, -1.0, 3.0)])
def test_temporal_lif_general_neuron_parameters_are_bit_exact(hip_ops, v_th, v_reset, tau):
    g = gen(7)
    x = torch.randn((6, 2, 4, 9, 9), generator=g) * 0.9 + 0.3
    ref = O.temporal_lif(x, torch.tensor(0.0), v_th, v_reset, tau)
    s, v = S.fused_temporal_lif_state(dev(x, F32), zero_v(), v_th, v_reset, tau, False)
    assert torch.equal(s.cpu(), ref[0]) and torch.equal(v.cpu(), ref[1])


# ---------------------------------------------------------------------------------------------------------------
# Depthwise 3x3 + LIF
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,vdtype", [(F32, F32), (BF16, F32), (F16, F16)])
@pytest.mark.parametrize("stride,N,C,H,W", [(1, 2, 16, 28, 28), (2, 2, 16, 28, 28), (1, 2, 24, 7, 7), (2, 1, 8, 7, 9),
                                             (1, 1, 8, 56, 56), (2, 1, 4, 112, 112), (1, 3, 5, 9, 11), (1, 1, 2, 96, 160)])
def test_depthwise_conv_lif(hip_ops, dtype, vdtype, stride, N, C, H, W):
    g = gen(200 + H)
    T = 4
    xs = [spikes((N, C, H, W), 0.3, g) for _ in range(T)]
    w = q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, dtype)
    b = q(torch.randn(C, generator=g) * 0.1, dtype)
    ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (stride, stride), (1, 1), (1, 1), C, *LIF)
    s, v = S.fused_temporal_depthwise_conv_lif_state([dev(x, dtype) for x in xs], dev(w, dtype), dev(b, dtype), zero_v(vdtype),
                                                     [stride, stride], [1, 1], [1, 1], C, *LIF, False)
    check(s, v, ref, v_dtype=vdtype, what="depthwise")
    _no_fallback(hip_ops, 1)
    assert hip_ops.get_fused_op_call_stats()[f"temporal_depthwise_k3_s{stride}_p1"] == 1


def test_depthwise_residual_alias_and_membrane_chaining(hip_ops):
    g = gen(21)
    N, C, H, W, T = 2, 16, 14, 14, 4
    xs = [q(torch.randn(N, C, H, W, generator=g), BF16) for _ in range(T)]     # analog inputs
    rs = [q(torch.randn(N, C, H, W, generator=g) * 0.3, BF16) for _ in range(T)]
    w, b = q(torch.randn(C, 1, 3, 3, generator=g) * 0.3, BF16), q(torch.randn(C, generator=g) * 0.1, BF16)
    v0 = torch.randn(N, C, H, W, generator=g) * 0.2
    ref = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (1, 1), (1, 1), C, *LIF, residuals=rs)
    dx, dr = [dev(x, BF16) for x in xs], [dev(r, BF16) for r in rs]
    args = (dev(w, BF16), dev(b, BF16))
    s, v = S.fused_temporal_conv_add_lif_state_depthwise(dx, dr, *args, dev(v0, F32), [1, 1], [1, 1], [1, 1], C, *LIF, False)
    check(s, v, ref, what="depthwise residual")
    # two chained windows of 2 steps == one window of 4 steps, bit for bit
    s1, v1 = S.fused_temporal_conv_add_lif_state(dx[:2], dr[:2], *args, dev(v0, F32), [1, 1], [1, 1], [1, 1], C, *LIF, False)
    s2, v2 = S.fused_temporal_conv_add_lif_state(dx[2:], dr[2:], *args, v1, [1, 1], [1, 1], [1, 1], C, *LIF, False)
    assert torch.equal(torch.cat([s1, s2]), s) and torch.equal(v2, v)
    # the alias operator name of the reference
    s3, v3 = S.fused_temporal_conv_lif_state_depthwise(dx, *args, dev(v0, F32), [1, 1], [1, 1], [1, 1], C, *LIF, False)
    ref3 = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (1, 1), (1, 1), C, *LIF)
    check(s3, v3, ref3, what="depthwise alias")
    _no_fallback(hip_ops, 4)


# ---------------------------------------------------------------------------------------------------------------
# LIF -> AvgPool -> Linear tail
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("T,N,C,H,W,K,bias", [(4, 3, 32, 7, 7, 10, True), (4, 4, 512, 1, 1, 10, True), (4, 4, 512, 2, 2, 1000, True),
                                               (4, 16, 512, 7, 7, 1000, True), (8, 2, 48, 5, 3, 17, False), (1, 1, 8, 32, 32, 3, True),
                                               (3, 1, 3, 3, 3, 5, True), (4, 50, 50, 5, 5, 7, True), (2, 2, 4, 25, 25, 6, True),
                                               (16, 5, 64, 4, 4, 100, True)])
def test_lif_avgpool_linear(hip_ops, dtype, T, N, C, H, W, K, bias):
    g = gen(300 + C)
    x = q(torch.randn(T, N, C, H, W, generator=g) * 0.75 + 0.15, dtype)
    w = q(torch.randn(K, C, generator=g) * 0.05, dtype)
    b = q(torch.randn(K, generator=g) * 0.05, dtype) if bias else None
    ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(x, torch.tensor(0.0), w, b, *LIF)
    fb = dev(b, dtype) if bias else torch.empty(0, device=DEV, dtype=dtype)
    op = S.fused_temporal_lif_avgpool_linear if T != 8 else S.fused_temporal_lif_tail
    out, v = op(dev(x, dtype), zero_v(F32), dev(w, dtype), fb, *LIF, False)
    assert out.dtype == dtype and tuple(out.shape) == (N, K) and v.dtype == F32
    assert torch.equal(v.cpu(), ref_v)                              # elementwise LIF: exact
    tol = 1e-4 if dtype == F32 else (8e-3 if dtype == BF16 else 2e-3)   # out_sum is stored in the activation dtype
    assert torch.allclose(out.float().cpu(), ref_out, rtol=tol, atol=tol), (out.float().cpu() - ref_out).abs().max()
    _no_fallback(hip_ops, 1)


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("T,N,C,H,W,K", [(4, 21, 64, 12, 12, 70), (16, 9, 96, 8, 8, 100), (4, 64, 512, 14, 14, 1000), (8, 8, 160, 9, 9, 64)])
def test_lif_avgpool_linear_on_batches_with_large_counts(hip_ops, dtype, T, N, C, H, W, K):
    """Batches of 8 samples or more with 64 classes or more and C % 32 == 0 take the matrix-core GEMV, which splits a spike
    count into count & 255 and count >> 8: strong inputs make most planes count beyond 255 (ragged class and sample tiles,
    fewer channel steps than waves, a last round of steps that not every wave has)."""
    g = gen(360 + C)
    x = q(torch.randn(T, N, C, H, W, generator=g) * 0.5 + 2.0, dtype)
    w = q(torch.randn(K, C, generator=g) * 0.05, dtype)
    b = q(torch.randn(K, generator=g) * 0.05, dtype)
    ref_out, ref_v, _, ref_spikes = O.temporal_lif_avgpool_linear(x, torch.tensor(0.0), w, b, *LIF)
    assert ref_spikes.sum(dim=(0, 3, 4)).median() > 255
    out, v = S.fused_temporal_lif_avgpool_linear(dev(x, dtype), zero_v(F32), dev(w, dtype), dev(b, dtype), *LIF, False)
    assert torch.equal(v.cpu(), ref_v)
    tol = 8e-3 if dtype == BF16 else 2e-3
    assert torch.allclose(out.float().cpu(), ref_out, rtol=tol, atol=tol), (out.float().cpu() - ref_out).abs().max()
    assert ref_out.abs().max() > 0.5      # the sums are far from zero: a dropped high part would show
    _no_fallback(hip_ops, 1)


@pytest.mark.parametrize("T,N,C,H,W,K,launches", [(4, 64, 512, 1, 1, 10, 1), (4, 32, 256, 2, 2, 10, 1), (4, 5, 64, 3, 3, 1000, 1),
                                                   (12, 3, 40, 4, 4, 37, 1), (4, 16, 512, 7, 7, 1000, 2), (4, 6, 36, 3, 3, 10, 2)])
def test_small_tails_run_as_one_launch_and_equal_the_two_launch_form(snnf_lib, T, N, C, H, W, K, launches):
    """The backend reports which form a tail took; the one-launch form gives the oracle's results and the membrane of the
    two-launch form bit for bit (reached here through a weight matrix that is not 16-byte aligned, which the one-launch
    form does not take; the classifier sums then agree to the output dtype's rounding)."""
    from triton_snn_fusion_amd.runtime import hip_temporal_lif_avgpool_linear_backend as TB
    g = gen(380 + C + K)
    x = q(torch.randn(T, N, C, H, W, generator=g) * 0.75 + 0.15, BF16)
    w = q(torch.randn(K, C, generator=g) * 0.05, BF16)
    b = q(torch.randn(K, generator=g) * 0.05, BF16)
    v0 = torch.rand(N, C, H, W, generator=g) * 0.9
    ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(x, v0, w, b, *LIF)
    res = TB.run_triton_fused_temporal_lif_avgpool_linear(dev(x, BF16), dev(v0, F32), dev(w, BF16), dev(b, BF16), *LIF, False)
    assert len(res.kernel_diagnostics["launches"]) == launches == snnf_lib.snnf_lif_pool_linear_launches(T, N, C, H, W, K)
    assert torch.equal(res.v_next.cpu(), ref_v)
    assert torch.allclose(res.out_sum.float().cpu(), ref_out, rtol=8e-3, atol=8e-3), (res.out_sum.float().cpu() - ref_out).abs().max()
    if launches == 1 and C % 8 == 0:
        # the same call with the weight matrix 2 bytes off a 16-byte boundary: two launches
        w_store = torch.empty(K * C + 8, device=DEV, dtype=BF16)
        w_off = w_store[1:1 + K * C].view(K, C)
        w_off.copy_(dev(w, BF16))
        assert w_off.data_ptr() % 16 != 0
        res2 = TB.run_triton_fused_temporal_lif_avgpool_linear(dev(x, BF16), dev(v0, F32), w_off, dev(b, BF16), *LIF, False)
        assert torch.equal(res2.v_next, res.v_next)
        assert torch.allclose(res2.out_sum.float(), res.out_sum.float(), rtol=8e-3, atol=8e-3)


@pytest.mark.parametrize("N,C,H,W", [(6, 64, 7, 7), (3, 5, 3, 3), (40, 128, 1, 1)])
def test_lif_avgpool_linear_tensor_v_init(hip_ops, N, C, H, W):
    """A membrane tensor as initial state (vector and element-wise paths of the pooling kernel)."""
    T, K = 4, 12
    g = gen(340 + C)
    x = q(torch.randn(T, N, C, H, W, generator=g) * 0.75 + 0.15, BF16)
    v0 = torch.rand(N, C, H, W, generator=g) * 0.9
    w = q(torch.randn(K, C, generator=g) * 0.05, BF16)
    b = q(torch.randn(K, generator=g) * 0.05, BF16)
    ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(x, v0, w, b, *LIF)
    out, v = S.fused_temporal_lif_avgpool_linear(dev(x, BF16), dev(v0, F32), dev(w, BF16), dev(b, BF16), *LIF, False)
    assert torch.equal(v.cpu(), ref_v)
    assert torch.allclose(out.float().cpu(), ref_out, rtol=8e-3, atol=8e-3), (out.float().cpu() - ref_out).abs().max()
    _no_fallback(hip_ops, 1)


# ---------------------------------------------------------------------------------------------------------------
# Temporal Linear + LIF
# ---------------------------------------------------------------------------------------------------------------
def _linear_case(seed, T, M, Fin, Fout, dtype, bias=True, p=0.1):
    g = gen(seed)
    x = spikes((T, M, Fin), p, g)
    w = torch.randn(Fout, Fin, generator=g) * (2.0 / Fin) ** 0.5 * 3.0
    b = torch.randn(Fout, generator=g) * 0.01 if bias else None
    wq = q(w, dtype)        # fp32 operands stay fp32: the kernel multiplies them as two bf16 terms each
    bq = None if b is None else q(b, dtype)
    return x, wq, bq, wq, bq if b is not None else None


@pytest.mark.parametrize("dtype,vdtype", [(BF16, F32), (F32, F32), (F16, F16), (BF16, BF16)])
@pytest.mark.parametrize("T,M,Fin,Fout,bias", [(8, 64, 256, 128, True), (3, 5, 100, 37, True), (16, 1, 512, 512, False),
                                                (4, 16, 1000, 48, True), (20, 3, 64, 16, True), (2, 33, 96, 130, True),
                                                (4, 64, 512, 1024, True), (16, 64, 256, 1024, True), (5, 40, 200, 64, True),
                                                (12, 17, 264, 96, False),
                                                # wide tiles of 8 rows: ragged last row tile, K % 128 = 8, at most 8 rows, a K of two slabs and 8
                                                (8, 20, 1032, 2048, True), (8, 7, 520, 4096, False), (5, 9, 136, 2048, True),
                                                (3, 12, 264, 2048, True), (16, 24, 392, 1024, True)])
def test_linear_lif_packed(hip_ops, dtype, vdtype, T, M, Fin, Fout, bias):
    x, w_dev, b_dev, w_ref, b_ref = _linear_case(400 + Fin, T, M, Fin, Fout, dtype, bias)
    ref = O.temporal_linear_lif(x, w_ref, b_ref, torch.tensor(0.0), *LIF)
    s, v = S.fused_temporal_linear_lif_state_packed(dev(x, dtype), dev(w_dev, dtype), dev(b_dev, dtype), zero_v(vdtype), *LIF, False)
    assert tuple(s.shape) == (T, M, Fout) and s.dtype == dtype and v.dtype == vdtype
    check(s, v, ref, v_dtype=vdtype, what="linear packed")
    _no_fallback(hip_ops, 1)


def test_linear_lif_list_out_and_leading_dims_forms_agree(hip_ops):
    T, M, Fin, Fout = 4, 12, 192, 80
    x, w_dev, b_dev, w_ref, b_ref = _linear_case(77, T, M, Fin, Fout, BF16)
    ref = O.temporal_linear_lif(x, w_ref, b_ref, torch.tensor(0.0), *LIF)
    dx, dw, db = dev(x, BF16), dev(w_dev, BF16), dev(b_dev, BF16)
    s, v = S.fused_temporal_linear_lif_state_packed(dx, dw, db, zero_v(), *LIF, False)
    check(s, v, ref, what="linear packed")
    s_l, v_l = S.fused_temporal_linear_lif_state([dx[t] for t in range(T)], dw, db, zero_v(), *LIF, False)
    assert torch.equal(s_l, s) and torch.equal(v_l, v)
    so, vo = torch.empty_like(s), torch.empty_like(v)
    assert S.fused_temporal_linear_lif_state_packed_out(dx, dw, db, zero_v(), *LIF, False, so, vo) is None
    assert torch.equal(so, s) and torch.equal(vo, v)
    s4, v4 = S.fused_temporal_linear_lif_state_packed(dx.reshape(T, 3, 4, Fin), dw, db, zero_v(), *LIF, False)
    assert tuple(s4.shape) == (T, 3, 4, Fout) and torch.equal(s4.reshape(T, M, Fout), s) and torch.equal(v4.reshape(M, Fout), v)
    # window chaining through a full-shape fp32 v_init. One timestep runs on the kernel without staging, which adds the
    # same products in another order than the staged kernel of the 4-step call: same spikes, membrane to the last bit or two.
    s1, v1 = S.fused_temporal_linear_lif_state_packed(dx[:1], dw, db, zero_v(), *LIF, False)
    s2, v2 = S.fused_temporal_linear_lif_state_packed(dx[1:], dw, db, v1, *LIF, False)
    assert torch.equal(torch.cat([s1, s2]), s) and torch.allclose(v2, v, rtol=0, atol=1e-6)
    _no_fallback(hip_ops, 6)
    assert hip_ops.get_fused_op_call_stats()["temporal_linear_lif_stack_materialized"] == 0


# ---------------------------------------------------------------------------------------------------------------
# Dense conv (implicit GEMM) + LIF
# ---------------------------------------------------------------------------------------------------------------
def _conv_case(seed, T, N, Cin, Cout, H, W, k, dtype, analog=False, p=0.2, gain=2.0):
    g = gen(seed)
    # fp32 tensors keep their fp32 values: the kernels split them into two bf16 terms each for the matrix cores and the
    # oracle is held to them unrounded.
    if analog:
        xs = [q(torch.randn(N, Cin, H, W, generator=g), dtype) for _ in range(T)]
    else:
        xs = [spikes((N, Cin, H, W), p, g) for _ in range(T)]
    w = torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * gain
    b = torch.randn(Cout, generator=g) * 0.1
    w_ref = q(w, dtype)
    b_ref = b if dtype == F32 else q(b, dtype)
    return xs, w_ref, b_ref, w_ref, b_ref


CONV_KEYS = [  # k, stride, pad, Cin, Cout, H, W, analog
    (1, 1, 0, 32, 64, 12, 12, False),
    (3, 1, 1, 16, 32, 12, 12, False),
    (3, 2, 1, 16, 32, 12, 12, False),
    (3, 2, 1, 8, 16, 7, 7, False),
    (5, 1, 2, 8, 16, 9, 9, False),
    (7, 2, 3, 3, 64, 32, 32, True),
    (11, 4, 2, 3, 64, 63, 63, True),
    (3, 1, 1, 40, 70, 14, 14, False),
    (3, 1, 1, 64, 64, 7, 7, False),
    (3, 1, 1, 3, 64, 32, 32, True),
    (1, 1, 0, 128, 256, 14, 14, False),
    (3, 1, 0, 16, 16, 10, 10, False),
    (1, 2, 0, 64, 128, 14, 14, False),
]


@pytest.mark.parametrize("dtype,vdtype", [(BF16, F32), (F32, F32), (F16, F16)])
@pytest.mark.parametrize("k,s,p,Cin,Cout,H,W,analog", CONV_KEYS)
def test_conv_lif_kernel_keys(hip_ops, dtype, vdtype, k, s, p, Cin, Cout, H, W, analog):
    T, N = 4, 2
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(500 + k * 10 + s, T, N, Cin, Cout, H, W, k, dtype, analog)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, torch.tensor(0.0), (s, s), (p, p), (1, 1), 1, *LIF)
    op = S.fused_temporal_pointwise_conv_lif_state if (k, s, p) == (1, 1, 0) else S.fused_temporal_conv_lif_state
    sp, v = op([dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype), zero_v(vdtype), [s, s], [p, p], [1, 1], 1, *LIF, False)
    assert sp.dtype == dtype and v.dtype == vdtype and tuple(sp.shape) == tuple(ref[0].shape)
    check(sp, v, ref, v_dtype=vdtype, what=f"conv k{k} s{s} p{p}")
    _no_fallback(hip_ops, 1)


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p", [(32, 64, 12, 12, 3, 1, 1), (64, 64, 9, 9, 3, 1, 1), (16, 32, 8, 10, 1, 2, 0)])
def test_conv_lif_activations_at_two_byte_alignment(hip_ops, Cin, Cout, H, W, k, s, p):
    """Timestep tensors that start one element into their storage: even widths then take the two-loads-per-pair path, odd
    widths the paired 4-byte loads at 2-byte alignment."""
    T, N = 4, 2
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(650 + H, T, N, Cin, Cout, H, W, k, BF16)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, torch.tensor(0.0), (s, s), (p, p), (1, 1), 1, *LIF)
    shifted = []
    for x in xs:
        store = torch.zeros(x.numel() + 1, device=DEV, dtype=BF16)
        view = store[1:].view(x.shape)
        view.copy_(x.to(DEV, BF16))
        assert view.data_ptr() % 4 == 2 and view.is_contiguous()
        shifted.append(view)
    sp, v = S.fused_temporal_conv_lif_state(shifted, dev(w_dev, BF16), dev(b_dev, BF16), zero_v(), [s, s], [p, p], [1, 1], 1, *LIF, False)
    check(sp, v, ref, what="conv, activations at 2-byte alignment")
    _no_fallback(hip_ops, 1)


@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 8, 16])
def test_conv_lif_timestep_counts_and_windows(hip_ops, T):
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(600 + T, T, 2, 32, 48, 10, 10, 3, BF16)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *LIF)
    sp, v = S.fused_temporal_conv_lif_state([dev(x, BF16) for x in xs], dev(w_dev, BF16), dev(b_dev, BF16), zero_v(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    check(sp, v, ref, what=f"conv T={T}")
    _no_fallback(hip_ops, 1)


def test_conv_residual_chaining_packed_out_single_step_and_batched_tn(hip_ops):
    T, N, Cin, Cout, H, W = 4, 3, 64, 64, 14, 14
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(31, T, N, Cin, Cout, H, W, 3, BF16)
    g = gen(32)
    rs = [q(torch.randn(N, Cout, H, W, generator=g) * 0.3, BF16) for _ in range(T)]
    v0 = torch.randn(N, Cout, H, W, generator=g) * 0.2
    dx, dr, dw, db = [dev(x, BF16) for x in xs], [dev(r, BF16) for r in rs], dev(w_dev, BF16), dev(b_dev, BF16)
    geo = ([1, 1], [1, 1], [1, 1], 1)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (1, 1), (1, 1), (1, 1), 1, *LIF, residuals=rs)
    s, v = S.fused_temporal_conv_add_lif_state(dx, dr, dw, db, dev(v0, F32), *geo, *LIF, False)
    check(s, v, ref, what="conv residual")
    s_tn, v_tn = S.fused_temporal_conv_add_lif_state_batched_tn(dx, dr, dw, db, dev(v0, F32), *geo, *LIF, False)
    assert torch.equal(s_tn, s.flatten(0, 1)) and torch.equal(v_tn, v)
    s1, v1 = S.fused_temporal_conv_add_lif_state(dx[:3], dr[:3], dw, db, dev(v0, F32), *geo, *LIF, False)
    s2, v2 = S.fused_temporal_conv_add_lif_state(dx[3:], dr[3:], dw, db, v1, *geo, *LIF, False)
    assert torch.equal(torch.cat([s1, s2]), s) and torch.equal(v2, v)
    # packed input + caller-owned outputs == list form
    ref_p = O.temporal_conv_lif(xs, w_ref, b_ref, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *LIF)
    s_l, v_l = S.fused_temporal_conv_lif_state(dx, dw, db, zero_v(), *geo, *LIF, False)
    check(s_l, v_l, ref_p, what="conv list")
    so, vo = torch.empty_like(s_l), torch.empty_like(v_l)
    assert S.fused_temporal_conv_lif_state_packed_out(torch.stack(dx), dw, db, zero_v(), *geo, *LIF, False, so, vo) is None
    assert torch.equal(so, s_l) and torch.equal(vo, v_l)
    s_b, v_b = S.fused_temporal_conv_lif_state_batched_tn(dx, dw, db, zero_v(), *geo, *LIF, False)
    assert torch.equal(s_b, s_l.flatten(0, 1))
    # single-step operator == first step of the temporal operator
    s0, v0_ = S.fused_conv_lif_state(dx[0], dw, db, zero_v(), *geo, *LIF, False)
    assert torch.equal(s0, s_l[0])
    _no_fallback(hip_ops, 8)


POINTWISE_CASES = [  # Cin, Cout, H, W, dtype, vdtype, lif, T, residual, tensor v_init
    (128, 256, 16, 16, BF16, F32, (1.0, 0.0, 2.0), 4, False, False),   # weights in registers, every tile inside its image
    (128, 256, 14, 14, BF16, F32, (1.0, 0.0, 2.0), 4, True, True),     # + ragged last tile (second launch), residual, v_init
    (64, 96, 8, 8, BF16, F32, (1.0, 0.0, 4.0), 3, False, False),       # weights in LDS, one chunk of 64 channels
    (64, 80, 8, 8, BF16, F32, (1.0, 0.0, 2.0), 2, False, True),        # Cout not a multiple of 32: row masks
    (256, 128, 7, 7, BF16, F32, (1.0, 0.0, 2.0), 4, True, False),      # odd plane (unaligned loads), two chunks
    (1024, 64, 8, 8, BF16, F32, (1.0, 0.0, 2.0), 2, False, False),     # weights streamed from L2
    (1024, 64, 5, 5, BF16, F32, (1.0, 0.0, 2.0), 2, False, True),      # streamed + odd plane
    (24, 32, 10, 10, BF16, F32, (1.0, 0.0, 2.0), 4, False, False),     # channel tail inside a chunk
    (8, 32, 8, 8, BF16, F32, (1.0, 0.0, 2.0), 4, False, False),        # a single channel group
    (128, 64, 16, 16, BF16, F32, (1.0, -1.0, 2.0), 4, False, False),   # soft reset: general variant
    (128, 64, 16, 16, BF16, F32, (0.5, 0.0, 1.0), 5, False, True),     # IF neuron
    (128, 64, 8, 8, F32, F32, (1.0, 0.0, 2.0), 4, True, False),        # fp32 activations (rounded to bf16 on the way in)
    (128, 64, 8, 8, F32, F32, (1.0, 0.0, 2.0), 4, False, True),        # fp32, no residual: the fast variant with fp32 spike stores
    (256, 64, 16, 8, F16, F32, (1.0, 0.0, 2.0), 4, False, True),       # f16, weights in LDS, no residual: LIF on the accumulators
    (128, 96, 8, 16, F16, F16, (1.0, 0.0, 2.0), 4, False, True),       # f16 with an f16 membrane
    (192, 64, 16, 8, F16, F32, (1.0, 0.0, 2.0), 17, False, False),     # channel tail in the second chunk, two launch windows
    (128, 64, 16, 16, BF16, F32, (1.0, 0.0, 1.5), 4, False, True),     # tau not a power of two: true division
]


@pytest.mark.parametrize("Cin,Cout,H,W,dtype,vdtype,lif,T,residual,tensor_v", POINTWISE_CASES)
def test_pointwise_conv_lif_variants(hip_ops, Cin, Cout, H, W, dtype, vdtype, lif, T, residual, tensor_v):
    N = 3
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(900 + Cin + Cout + H, T, N, Cin, Cout, H, W, 1, dtype, p=0.25)
    g = gen(901 + Cin)
    rs = [q(torch.randn(N, Cout, H, W, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = q(torch.randn(N, Cout, H, W, generator=g) * 0.3, vdtype) if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (1, 1), (0, 0), (1, 1), 1, *lif, residuals=rs)
    dx, dw, db = [dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype)
    dv = dev(v0, vdtype) if tensor_v else zero_v(vdtype)
    if residual:
        sp, v = S.fused_temporal_conv_add_lif_state(dx, [dev(r, dtype) for r in rs], dw, db, dv, [1, 1], [0, 0], [1, 1], 1, *lif, False)
    else:
        sp, v = S.fused_temporal_pointwise_conv_lif_state(dx, dw, db, dv, [1, 1], [0, 0], [1, 1], 1, *lif, False)
    assert sp.dtype == dtype and v.dtype == vdtype and tuple(sp.shape) == (T, N, Cout, H, W)
    check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=f"pointwise {Cin}->{Cout} {H}x{W}")
    _no_fallback(hip_ops, 1)


LARGE_POINTWISE_CASES = [  # Cin, Cout, H, W, dtype, lif, T, N, residual, tensor v_init
    (256, 128, 7, 7, BF16, (1.0, 0.0, 2.0), 4, 1280, True, False),     # weights in LDS, several chunks, odd plane, residual
    (256, 64, 16, 8, F16, (1.0, 0.0, 2.0), 4, 640, False, True),       # f16, several chunks, LIF on the accumulators
    (192, 64, 16, 8, F16, (1.0, 0.0, 2.0), 17, 192, False, False),     # channel tail in the last chunk, two launch windows
    (1024, 64, 56, 56, BF16, (1.0, 0.0, 2.0), 4, 8, False, False),     # weights streamed from L2
    (1024, 64, 5, 5, BF16, (1.0, 0.0, 2.0), 4, 1000, False, True),     # streamed + odd plane
]


@pytest.mark.parametrize("Cin,Cout,H,W,dtype,lif,T,N,residual,tensor_v", LARGE_POINTWISE_CASES)
def test_pointwise_layers_of_several_chunks(hip_ops, Cin, Cout, H, W, dtype, lif, T, N, residual, tensor_v):
    """Plain 1x1 layers of more than 128 input channels stay with the pointwise kernel from 200 MB of traffic on (smaller
    ones run the matrix kernel): its variants for several channel chunks are reached by large layers only."""
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(950 + Cin + Cout + H, T, N, Cin, Cout, H, W, 1, dtype, p=0.25)
    g = gen(951 + Cin)
    rs = [q(torch.randn(N, Cout, H, W, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = q(torch.randn(N, Cout, H, W, generator=g) * 0.3, F32) if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (1, 1), (0, 0), (1, 1), 1, *lif, residuals=rs)
    dx, dw, db = [dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype)
    dv = dev(v0, F32) if tensor_v else zero_v(F32)
    if residual:
        sp, v = S.fused_temporal_conv_add_lif_state(dx, [dev(r, dtype) for r in rs], dw, db, dv, [1, 1], [0, 0], [1, 1], 1, *lif, False)
    else:
        sp, v = S.fused_temporal_pointwise_conv_lif_state(dx, dw, db, dv, [1, 1], [0, 0], [1, 1], 1, *lif, False)
    assert last_conv_plan()["kernel"] == "pointwise", last_conv_plan()
    check(sp, v, ref, v_threshold=lif[0], v_dtype=F32, what=f"large pointwise {Cin}->{Cout} {H}x{W} x{N}")
    # the same layer on a batch small enough for the matrix kernel
    n = 3
    sp_s, v_s = (S.fused_temporal_conv_add_lif_state([x[:n].contiguous() for x in dx], [dev(r[:n], dtype) for r in rs], dw, db,
                                                     dv[:n].contiguous() if tensor_v else dv, [1, 1], [0, 0], [1, 1], 1, *lif, False)
                 if residual else
                 S.fused_temporal_pointwise_conv_lif_state([x[:n].contiguous() for x in dx], dw, db,
                                                           dv[:n].contiguous() if tensor_v else dv, [1, 1], [0, 0], [1, 1], 1, *lif, False))
    assert last_conv_plan()["kernel"] == "matrix", last_conv_plan()
    check(sp_s, v_s, (ref[0][:, :n], ref[1][:n], ref[2][:, :n]), v_threshold=lif[0], v_dtype=F32, what=f"small pointwise {Cin}->{Cout} {H}x{W} on the matrix kernel")
    _no_fallback(hip_ops, 2)


DENSE_CASES = [  # Cin, Cout, H, W, k, stride, pad, dtype, vdtype, lif, T, N, residual, tensor v_init
    (64, 64, 16, 16, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False),    # whole tiles, 16-byte runs
    (128, 128, 14, 14, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 2, True, True),    # K split across waves, 8-byte runs
    (256, 64, 7, 7, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 3, False, True),      # odd plane: masked variant, K split
    (32, 96, 12, 12, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 3, 2, True, False),     # Cout % 64 != 0, window of 4 with 3 live steps
    (64, 64, 10, 10, 3, 1, 1, BF16, F32, (1.0, -1.0, 2.0), 2, 2, False, False),   # two steps side by side, soft reset
    (64, 128, 9, 9, 3, 1, 1, BF16, F32, (0.5, 0.0, 1.0), 1, 2, True, True),       # single step, IF neuron
    (48, 64, 16, 16, 5, 1, 2, F16, F16, (1.0, 0.0, 2.0), 4, 2, False, True),      # 5x5, f16 with an f16 membrane
    (64, 64, 16, 16, 3, 2, 1, F32, F32, (1.0, 0.0, 2.0), 4, 2, False, False),     # stride 2, fp32 activations
    (64, 64, 15, 15, 3, 1, 1, BF16, F32, (1.0, 0.0, 4.0), 4, 2, False, False),    # odd width: unaligned loads
    (512, 128, 4, 4, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 4, False, False),    # deep and tiny: K split eight ways
    (64, 64, 16, 16, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 6, 2, True, True),      # two launch windows (4 + 2)
    (64, 192, 8, 24, 1, 2, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False),    # strided 1x1 (downsample shortcut)
    (128, 128, 2, 2, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 16, True, True),     # 2x2 planes: 8 images per tile
    (64, 64, 4, 4, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 6, False, True),       # 4x4 planes, batch not a multiple of the images per tile
    (256, 128, 4, 4, 3, 1, 1, BF16, F32, (1.0, -1.0, 2.0), 3, 5, True, False),    # several images per tile, K split, masked variant, soft reset
    (64, 64, 8, 8, 3, 2, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 8, False, False),      # stride 2 onto 4x4 planes, several images per tile
    (32, 64, 6, 6, 5, 1, 2, F16, F32, (1.0, 0.0, 2.0), 2, 7, True, True),         # 6x6 planes (no aligned runs), 5x5 kernel, f16
    (64, 64, 12, 12, 3, 1, 1, BF16, F32, (1.0, 0.0, 3.0), 4, 2, False, True),     # tau not a power of two: true division
    (128, 64, 8, 8, 3, 1, 1, BF16, F32, (0.75, -1.0, 1.5), 4, 2, True, False),    # + soft reset, K split
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,stride,pad,dtype,vdtype,lif,T,N,residual,tensor_v", DENSE_CASES)
def test_dense_conv_lif_matrix_kernel_variants(hip_ops, Cin, Cout, H, W, k, stride, pad, dtype, vdtype, lif, T, N, residual, tensor_v):
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(1200 + Cin + Cout + H + k, T, N, Cin, Cout, H, W, k, dtype, p=0.25)
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    g = gen(1201 + Cin)
    rs = [q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, vdtype) if tensor_v else torch.tensor(0.0)
    geo = ([stride, stride], [pad, pad], [1, 1], 1)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (stride, stride), (pad, pad), (1, 1), 1, *lif, residuals=rs)
    dx, dw, db = [dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype)
    dv = dev(v0, vdtype) if tensor_v else zero_v(vdtype)
    if residual:
        sp, v = S.fused_temporal_conv_add_lif_state(dx, [dev(r, dtype) for r in rs], dw, db, dv, *geo, *lif, False)
    else:
        sp, v = S.fused_temporal_conv_lif_state(dx, dw, db, dv, *geo, *lif, False)
    assert sp.dtype == dtype and v.dtype == vdtype and tuple(sp.shape) == (T, N, Cout, Ho, Wo)
    check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=f"dense {Cin}->{Cout} k{k} s{stride} {H}x{W}")
    _no_fallback(hip_ops, 1)


FALLBACK_KERNEL_CASES = [  # Cin, Cout, H, W, k, stride, pad, dtype, vdtype, lif, T, N, residual, tensor v_init, kernel family
    (12, 32, 12, 12, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False, "time_outer"),    # partial channel group
    (20, 48, 14, 14, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 2, True, True, "time_outer"),      # + residual, v_init
    (36, 64, 9, 11, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 5, 3, False, True, "time_outer"),      # ragged planes, T = 5
    (12, 32, 13, 13, 3, 2, 1, F16, F16, (1.0, -1.0, 2.0), 3, 2, True, False, "time_outer"),     # stride 2, f16 membrane, soft reset
    (20, 40, 10, 10, 3, 1, 1, F32, F32, (0.5, 0.0, 1.0), 4, 2, False, False, "time_outer"),     # fp32, IF neuron
    (12, 32, 12, 12, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False, "time_outer"),    # 1x1 with Cin % 8 != 0
    (20, 64, 7, 9, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 3, True, True, "time_outer"),        # 1x1, odd plane, residual, v_init
    (44, 256, 12, 12, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False, "t_in_m"),      # high intensity, Cin % 8 != 0
    (44, 256, 9, 9, 3, 1, 1, BF16, F32, (1.0, 0.0, 2.0), 4, 3, True, True, "t_in_m"),          # + odd plane, residual, v_init
    (52, 320, 10, 10, 3, 1, 1, F16, F32, (1.0, 0.0, 4.0), 6, 2, False, True, "t_in_m"),        # two launch windows, f16
    (512, 512, 14, 14, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False, "matrix"),     # deep pointwise layer (AI 205): an image is one row of pixels to the matrix kernel
    (1024, 1024, 7, 7, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, True, True, "matrix"),       # deep pointwise layer (AI 410), residual, v_init
    (520, 512, 14, 14, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, False, False, "matrix"),     # ... and so is a channel count of whole groups that is no multiple of the chunk
    (516, 512, 14, 14, 1, 1, 0, BF16, F32, (1.0, 0.0, 2.0), 4, 2, True, False, "t_in_m"),      # deep pointwise layer whose channels are not whole groups of 8
    (12, 32, 12, 12, 3, 1, 1, BF16, F32, (1.0, 0.0, 3.0), 4, 2, False, True, "time_outer"),     # tau not a power of two
    (36, 44, 40, 21, 7, 2, 0, BF16, BF16, (1.0, -1.0, 2.0), 4, 3, False, False, "t_in_m"),      # 7x7 at stride 2: no tile of all 64 lanes fits the staging slots
    (44, 256, 12, 12, 3, 1, 1, BF16, F32, (0.75, 0.0, 1.5), 4, 2, False, True, "t_in_m"),      # tau not a power of two
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,stride,pad,dtype,vdtype,lif,T,N,residual,tensor_v,family", FALLBACK_KERNEL_CASES)
def test_dense_conv_lif_shapes_outside_the_matrix_and_pointwise_kernels(hip_ops, Cin, Cout, H, W, k, stride, pad, dtype, vdtype, lif, T, N,
                                                                        residual, tensor_v, family):
    """Layers the 8-wave matrix kernel and the pointwise kernel do not take (input channels that are not whole groups of 8)
    run the time-outer kernel or the 4-wave T-in-M kernel; plain 1x1 layers of high arithmetic intensity run the matrix
    kernel on images flattened to one row of pixels."""
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(1600 + Cin + Cout + H + k, T, N, Cin, Cout, H, W, k, dtype, p=0.25)
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    g = gen(1601 + Cin)
    rs = [q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, vdtype) if tensor_v else torch.tensor(0.0)
    geo = ([stride, stride], [pad, pad], [1, 1], 1)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (stride, stride), (pad, pad), (1, 1), 1, *lif, residuals=rs)
    dx, dw, db = [dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype)
    dv = dev(v0, vdtype) if tensor_v else zero_v(vdtype)
    if residual:
        sp, v = S.fused_temporal_conv_add_lif_state(dx, [dev(r, dtype) for r in rs], dw, db, dv, *geo, *lif, False)
    else:
        sp, v = S.fused_temporal_conv_lif_state(dx, dw, db, dv, *geo, *lif, False)
    assert last_conv_plan()["kernel"] == family, last_conv_plan()
    check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=f"{family} {Cin}->{Cout} k{k} s{stride} {H}x{W}")
    _no_fallback(hip_ops, 1)


def test_planes_of_four_pixels_with_several_images_per_tile(hip_ops):
    """2x2 planes, two images per tile: a lane's run of 8 pixels spans two images (each half is one whole plane)."""
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    Cin, Cout, T, N = 256, 512, 4, 40
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(1700, T, N, Cin, Cout, 2, 2, 3, BF16, p=0.25)
    g = gen(1701)
    rs = [q(torch.randn(N, Cout, 2, 2, generator=g) * 0.3, BF16) for _ in range(T)]
    v0 = torch.randn(N, Cout, 2, 2, generator=g) * 0.3
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (1, 1), (1, 1), (1, 1), 1, *LIF, residuals=rs)
    sp, v = S.fused_temporal_conv_add_lif_state([dev(x, BF16) for x in xs], [dev(r, BF16) for r in rs], dev(w_dev, BF16), dev(b_dev, BF16),
                                                dev(v0, F32), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    plan = last_conv_plan()
    assert plan["kernel"] == "matrix" and plan["tile"] == "2x2x2" and plan["variant"] == 24, plan
    check(sp, v, ref, what="2x2 planes, two images per tile")
    _no_fallback(hip_ops, 1)


def test_conv_shared_analog_frame_is_convolved_once_and_matches(hip_ops):
    """Direct encoding: the same analog frame feeds every timestep (the T list entries alias one tensor)."""
    g = gen(41)
    x = q(torch.randn(2, 3, 32, 32, generator=g), BF16)
    w = q(torch.randn(64, 3, 3, 3, generator=g) * 0.4, BF16)
    b = q(torch.randn(64, generator=g) * 0.1, BF16)
    ref = O.temporal_conv_lif([x] * 4, w, b, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *LIF)
    dx = dev(x, BF16)
    s, v = S.fused_temporal_conv_lif_state([dx] * 4, dev(w, BF16), dev(b, BF16), zero_v(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    check(s, v, ref, what="shared frame")
    s2, v2 = S.fused_temporal_conv_lif_state([dx.clone() for _ in range(4)], dev(w, BF16), dev(b, BF16), zero_v(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    assert torch.equal(s, s2) and torch.equal(v, v2)


SHARED_FRAME_CASES = [  # Cin, Cout, H, W, k, stride, pad, dtype, lif, T, N, residual, tensor v_init
    (3, 64, 64, 64, 7, 2, 3, BF16, (1.0, 0.0, 2.0), 4, 2, False, False),     # ResNet stem
    (3, 64, 31, 31, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 2, False, True),      # odd plane: masked variant
    (1, 32, 28, 28, 5, 1, 2, BF16, (1.0, 0.0, 2.0), 6, 3, False, False),     # one input channel, Cout % 64 != 0
    (2, 64, 32, 32, 3, 1, 1, F32, (1.0, -1.0, 2.0), 4, 2, True, False),      # fp32 frame, soft reset, residual per step
    (64, 64, 16, 16, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 5, 2, False, True),     # analog frame with whole channel groups
    (128, 64, 8, 8, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 2, True, True),       # K split across waves, T steps per round
    (3, 64, 32, 32, 3, 1, 1, F16, (0.5, 0.0, 1.0), 20, 1, False, False),     # two launch windows (16 + 4), IF neuron
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,stride,pad,dtype,lif,T,N,residual,tensor_v", SHARED_FRAME_CASES)
def test_conv_shared_analog_frame_variants(hip_ops, Cin, Cout, H, W, k, stride, pad, dtype, lif, T, N, residual, tensor_v):
    """One analog frame for all T timesteps: convolved once, T LIF steps on the same accumulators."""
    g = gen(1300 + Cin + Cout + H + k)
    op_dtype = dtype                               # fp32 frames and weights stay fp32 (two bf16 terms each on the matrix cores)
    x = q(torch.randn(N, Cin, H, W, generator=g), op_dtype)
    w = q(torch.randn(Cout, Cin, k, k, generator=g) * (1.5 / (Cin * k * k) ** 0.5), op_dtype)
    b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    rs = [q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, F32) if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif([x] * T, w, b, v0, (stride, stride), (pad, pad), (1, 1), 1, *lif, residuals=rs)
    geo = ([stride, stride], [pad, pad], [1, 1], 1)
    dx, dv = dev(x, dtype), (dev(v0, F32) if tensor_v else zero_v())
    if residual:
        sp, v = S.fused_temporal_conv_add_lif_state([dx] * T, [dev(r, dtype) for r in rs], dev(w, dtype), dev(b, dtype), dv, *geo, *lif, False)
    else:
        sp, v = S.fused_temporal_conv_lif_state([dx] * T, dev(w, dtype), dev(b, dtype), dv, *geo, *lif, False)
    assert tuple(sp.shape) == (T, N, Cout, Ho, Wo)
    check(sp, v, ref, v_threshold=lif[0], what=f"shared frame {Cin}->{Cout} k{k} s{stride} {H}x{W} T={T}")
    _no_fallback(hip_ops, 1)


CONV_BIAS_CASES = [  # Cin, Cout, H, W, k, stride, pad, dtype, T, N, residual, analog input
    (64, 128, 16, 16, 1, 2, 0, BF16, 4, 2, False, False),     # ResNet downsample shortcut
    (64, 64, 12, 12, 3, 1, 1, BF16, 4, 2, True, False),       # conv + bias + residual (pre-tail sum)
    (128, 96, 7, 7, 3, 1, 1, BF16, 3, 3, True, False),        # odd plane, Cout % 64 != 0, 3 frames
    (3, 32, 20, 20, 5, 1, 2, BF16, 2, 2, False, True),        # few input channels, analog frames
    (32, 64, 16, 16, 3, 2, 1, F16, 4, 2, False, True),        # fp16
    (64, 64, 8, 8, 3, 1, 1, F32, 1, 4, False, False),         # fp32 in and out (bf16 matrix operands)
    (256, 64, 6, 6, 3, 1, 1, BF16, 4, 2, True, False),        # deep: K split across waves
    (64, 128, 8, 8, 1, 1, 0, BF16, 4, 3, False, False),       # plain 1x1 / stride 1: an image is one row of pixels
    (128, 256, 7, 9, 1, 1, 0, F16, 3, 2, True, False),        # the same with a residual, odd plane
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,stride,pad,dtype,T,N,residual,analog", CONV_BIAS_CASES)
def test_conv_bias_without_neuron(hip_ops, Cin, Cout, H, W, k, stride, pad, dtype, T, N, residual, analog):
    """snnf_conv_bias: the matrix kernel's neuron-free output against F.conv2d in fp32 on the same (rounded) operands;
    the only rounding on the kernel's side is the store in the activation dtype."""
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan, run_hip_temporal_conv_bias
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(1400 + Cin + Cout + H + k, T, N, Cin, Cout, H, W, k, dtype, analog=analog, p=0.3)
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    g = gen(1401 + Cin)
    rs = [q(torch.randn(N, Cout, Ho, Wo, generator=g), dtype) for _ in range(T)] if residual else None
    want = torch.stack([torch.nn.functional.conv2d(x, w_ref, b_ref, stride, pad) for x in xs])
    if residual:
        want = want + torch.stack(rs)
    got = run_hip_temporal_conv_bias([dev(x, dtype) for x in xs], dev(w_dev, dtype), dev(b_dev, dtype), [stride, stride], [pad, pad],
                                     None if rs is None else [dev(r, dtype) for r in rs])
    assert got.dtype == dtype and tuple(got.shape) == (T, N, Cout, Ho, Wo)
    assert last_conv_plan()["kernel"] == "matrix"
    rtol = {F32: 1e-4, BF16: 2 ** -8, F16: 2 ** -10}[dtype]
    assert torch.allclose(got.float().cpu(), want, rtol=rtol, atol=1e-4 if dtype == F32 else 1e-3), (got.float().cpu() - want).abs().max()


def test_conv_bias_rejects_what_the_matrix_kernel_does_not_take(hip_ops):
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import run_hip_temporal_conv_bias
    w12 = torch.zeros(64, 12, 3, 3, device=DEV, dtype=BF16)
    with pytest.raises(RuntimeError, match="unsupported_shape"):
        run_hip_temporal_conv_bias([torch.zeros(2, 12, 8, 8, device=DEV, dtype=BF16)], w12, None, [1, 1], [1, 1])   # Cin % 8 != 0


def test_conv_plan_is_reported(hip_ops):
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    xs = [torch.zeros(2, 64, 16, 16, device=DEV, dtype=BF16) for _ in range(4)]
    w, b = torch.zeros(64, 64, 3, 3, device=DEV, dtype=BF16), torch.zeros(64, device=DEV, dtype=BF16)
    S.fused_temporal_conv_lif_state(xs, w, b, zero_v(), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
    plan = last_conv_plan()
    assert plan["kernel"] == "matrix" and plan["variant"] == 24 and plan["window"] == 4 and plan["launches"] == 1
    w1 = torch.zeros(128, 64, 1, 1, device=DEV, dtype=BF16)
    S.fused_temporal_pointwise_conv_lif_state(xs, w1, torch.zeros(128, device=DEV, dtype=BF16), zero_v(), [1, 1], [0, 0], [1, 1], 1, *LIF, False)
    assert last_conv_plan()["kernel"] == "pointwise"
    configs = hip_ops.get_kernel_temporal_configs()
    assert any("BTILE_T=4" in key for key in configs), configs


@pytest.mark.parametrize("dtype", [BF16, F16, F32])
@pytest.mark.parametrize("kind,k,s,p,shape", [("max", 3, 2, 1, (4, 2, 8, 112, 112)), ("max", 3, 2, 1, (3, 5, 9, 11)), ("max", 2, 2, 0, (2, 3, 7, 10)),
                                              ("avg", 2, 2, 0, (4, 2, 16, 32, 32)), ("avg", 2, 2, 0, (3, 5, 7, 9)), ("max", 3, 2, 0, (2, 2, 3, 3)), ("max", 2, 2, 0, (2, 3, 8, 16)), ("max", 3, 2, 1, (5, 3, 14, 24))])
def test_pool2d_matches_the_framework_pooling_exactly(snnf_lib, dtype, kind, k, s, p, shape):
    """snnf_pool2d on spikes and on analog values: max pooling selects, 2x2 averaging of spikes is exact in every dtype."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime.hip_pool_backend import pool_config, run_hip_pool2d
    g = gen(1500 + k + shape[-1])
    x = spikes(shape, 0.3, g) if kind == "avg" else q(torch.randn(shape, generator=g), dtype)
    module = torch.nn.MaxPool2d(k, s, p) if kind == "max" else torch.nn.AvgPool2d(k)
    assert pool_config(module) == (kind == "max", k, s, p)
    want = module(x.reshape(-1, 1, shape[-2], shape[-1])).reshape(*shape[:-2], -1, (shape[-1] + 2 * p - k) // s + 1)
    got = run_hip_pool2d(dev(x, dtype), kind == "max", k, s, p)
    assert got.dtype == dtype and tuple(got.shape) == tuple(want.shape)
    assert torch.equal(got.float().cpu(), want)


def test_pool2d_rejects_other_windows(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime.hip_pool_backend import pool_config, run_hip_pool2d
    assert pool_config(torch.nn.AvgPool2d(3)) is None and pool_config(torch.nn.MaxPool2d(3, 1, 1)) is None
    assert pool_config(torch.nn.MaxPool2d(3, 2, 1, ceil_mode=True)) is None
    with pytest.raises(RuntimeError, match="unsupported_kernel"):
        run_hip_pool2d(torch.zeros(2, 8, 8, device=DEV, dtype=BF16), False, 3, 3, 0)


def test_conv_and_linear_known_answers_exact(hip_ops):
    """tests/golden/conv_kat.json: exact sums (multiples of 1/8), so bf16 matrix operands must reproduce them bit for
    bit. An integrate-and-fire neuron (tau <= 1) with an unreachable threshold makes v_out the convolution output."""
    cases = json.load(open(os.path.join(GOLDEN, "conv_kat.json")))["cases"]
    calls = 0
    for c in cases:
        for dtype in (F32, BF16):
            if c["kind"] == "conv2d":
                x = torch.tensor(c["x"]).reshape(c["N"], c["Cin"], c["H"], c["W"])
                w = torch.tensor(c["w"]).reshape(c["Cout"], c["Cin"] // c["groups"], c["KH"], c["KW"])
                b = torch.tensor(c["b"])
                want = torch.tensor(c["out"]).reshape(c["N"], c["Cout"], c["Ho"], c["Wo"])
                op = S.fused_temporal_depthwise_conv_lif_state if c["groups"] > 1 else S.fused_temporal_conv_lif_state
                s, v = op([dev(x, dtype)], dev(w, dtype), dev(b, dtype), zero_v(), c["stride"], c["padding"], [1, 1], c["groups"], 1e30, 0.0, 1.0, False)
            else:
                x = torch.tensor(c["x"]).reshape(1, c["M"], c["Fin"])
                w = torch.tensor(c["w"]).reshape(c["Fout"], c["Fin"])
                b = torch.tensor(c["b"])
                want = torch.tensor(c["out"]).reshape(c["M"], c["Fout"])
                s, v = S.fused_temporal_linear_lif_state_packed(dev(x, dtype), dev(w, dtype), dev(b, dtype), zero_v(), 1e30, 0.0, 1.0, False)
            calls += 1
            assert torch.equal(v.cpu(), want), (c["kind"], dtype, (v.cpu() - want).abs().max())
            assert float(s.float().abs().sum()) == 0.0
    _no_fallback(hip_ops, calls)


# ---------------------------------------------------------------------------------------------------------------
# Failure handling through the operator layer
# ---------------------------------------------------------------------------------------------------------------
def test_unsupported_configurations_fall_back_to_eager_ops_on_the_gpu_and_are_counted(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime import snn_custom_ops as ops
    ops.configure_fused_op("hip", strict_triton=False)
    ops.reset_fused_op_call_stats()
    try:
        g = gen(3)
        xs = [spikes((1, 4, 9, 9), 0.3, g) for _ in range(2)]
        w, b = torch.randn(4, 4, 3, 3, generator=g), torch.randn(4, generator=g)
        ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (1, 1), (2, 2), (2, 2), 1, *LIF)
        s, v = S.fused_temporal_conv_lif_state([dev(x, F32) for x in xs], dev(w, F32), dev(b, F32), zero_v(), [1, 1], [2, 2], [2, 2], 1, *LIF, False)
        check(s, v, ref, what="dilated fallback")
        stats = ops.get_fused_op_call_stats()
        assert stats["fallback"] == 1 and stats["triton"] == 0
        assert stats["fallback_reasons"] == {"temporal:unsupported_dilation": 1}
        ops.configure_fused_op("hip", strict_triton=True)
        with pytest.raises(RuntimeError, match="unsupported_dilation"):
            S.fused_temporal_conv_lif_state([dev(x, F32) for x in xs], dev(w, F32), dev(b, F32), zero_v(), [1, 1], [2, 2], [2, 2], 1, *LIF, False)
    finally:
        ops.configure_fused_op("torch")


def test_fallback_chains_a_float32_membrane_next_to_16_bit_activations(snnf_lib):
    """A call the kernels do not take (dilation 2) with bf16 activations and a full-shape fp32 membrane: the eager ops step in
    fp32 and return an fp32 membrane, as the kernels do, so two chained fallback windows equal one long oracle call."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime import snn_custom_ops as ops
    ops.configure_fused_op("hip", strict_triton=False)
    ops.reset_fused_op_call_stats()
    try:
        g = gen(5)
        T, N, C, H = 4, 2, 8, 9
        xs = [spikes((N, C, H, H), 0.3, g) for _ in range(T)]
        w, b = q(torch.randn(C, C, 3, 3, generator=g) * 0.4, BF16), q(torch.randn(C, generator=g) * 0.1, BF16)
        v0 = torch.randn(N, C, H, H, generator=g) * 0.3
        geo = ([1, 1], [2, 2], [2, 2], 1)
        ref = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (2, 2), (2, 2), 1, *LIF)
        dx, dw, db = [dev(x, BF16) for x in xs], dev(w, BF16), dev(b, BF16)
        s1, v1 = S.fused_temporal_conv_lif_state(dx[:2], dw, db, dev(v0, F32), *geo, *LIF, False)
        assert v1.dtype == F32 and s1.dtype == BF16
        s2, v2 = S.fused_temporal_conv_lif_state(dx[2:], dw, db, v1, *geo, *LIF, False)
        assert v2.dtype == F32
        check(torch.cat([s1, s2]), v2, ref, what="chained dilated fallback, fp32 membrane")
        stats = ops.get_fused_op_call_stats()
        assert stats["fallback"] == 2 and stats["triton"] == 0
        # a 0-dim fp32 zero on the device also selects an fp32 membrane; a host-side placeholder the activation dtype
        _, v3 = S.fused_temporal_conv_lif_state(dx[:2], dw, db, zero_v(F32), *geo, *LIF, False)
        _, v4 = S.fused_temporal_conv_lif_state(dx[:2], dw, db, torch.tensor(0.0), *geo, *LIF, False)
        assert v3.dtype == F32 and v4.dtype == BF16
        # the native path follows the same rule
        _, v5 = S.fused_temporal_conv_lif_state(dx[:2], dw, db, zero_v(F32), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
        _, v6 = S.fused_temporal_conv_lif_state(dx[:2], dw, db, torch.tensor(0.0), [1, 1], [1, 1], [1, 1], 1, *LIF, False)
        assert v5.dtype == F32 and v6.dtype == BF16
        assert ops.get_fused_op_call_stats()["triton"] == 2
    finally:
        ops.configure_fused_op("torch")


def test_single_step_lif_runs_the_scan_kernel_on_the_gpu(hip_ops):
    """`lif_forward_state` on GPU tensors of any rank: one launch of the scan kernel, bit exact against the oracle, state
    chained through a module-style loop."""
    g = gen(6)
    for shape, dtype, vdtype in (((3, 50), F32, F32), ((2, 8, 7, 7), BF16, BF16), ((2, 8, 7, 7), BF16, F32), ((5,), F16, F16)):
        xs = q(torch.randn((3,) + shape, generator=g) * 0.9 + 0.2, dtype)
        v = zero_v(vdtype)
        ref = O.temporal_lif(xs, torch.tensor(0.0), *LIF)
        got = []
        for t in range(3):
            s, v = S.lif_forward_state(dev(xs[t], dtype), v, *LIF, False)
            assert s.dtype == dtype and v.dtype == vdtype
            got.append(s)
        check(torch.stack(got), v, ref, v_dtype=vdtype, what=f"single-step lif {shape} {dtype}")
        assert torch.equal(torch.stack(got).float().cpu(), ref[0])


# ---------------------------------------------------------------------------------------------------------------
# 16-bit membranes over calls that take several launches: rounded once, after the last step
# ---------------------------------------------------------------------------------------------------------------
SEVERAL_LAUNCH_CASES = [  # Cin, Cout, H, W, k, s, p, T, N, lif, host placeholder v_init
    (4, 8, 24, 23, 3, 1, 1, 8, 7, (0.5, 0.0, 1.0), True),          # IF neuron: nothing decays, every hand-over counts
    (32, 512, 23, 13, 3, 1, 1, 17, 2, (1.0, -1.0, 2.0), True),      # 17 steps, soft reset
    (16, 32, 20, 20, 3, 2, 1, 6, 4, (1.0, 0.0, 2.0), False),        # stride 2, membrane continued from a bf16 tensor
    (512, 32, 20, 20, 1, 1, 0, 17, 8, (0.75, 0.25, 4.0), False),    # pointwise kernel, 16 + 1 steps
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p,T,N,lif,placeholder", SEVERAL_LAUNCH_CASES)
def test_bf16_membrane_over_several_launches_is_rounded_once(hip_ops, Cin, Cout, H, W, k, s, p, T, N, lif, placeholder):
    """bf16 activations with the rewriter's host-side 0-dim `v_init` (or a bf16 state) give a bf16 membrane, as in the
    reference, whose kernel keeps it in fp32 registers over all T and rounds at the final store. A call that this
    library runs as several launches must not round at the hand-overs: same gate as a single launch. Called twice: the
    second call knows the layer's number of launches from the first."""
    from triton_snn_fusion_amd.runtime import hip_convlif_backend as CB
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(8100 + Cin + T, T, N, Cin, Cout, H, W, k, BF16, p=0.25)
    Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    g = gen(8101)
    v0 = torch.tensor(0.0) if placeholder else q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, BF16)
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, v0, (s, s), (p, p), (1, 1), 1, *lif)
    dv = v0 if placeholder else dev(v0, BF16)                     # the placeholder stays on the host, as the rewriter emits it
    dx, dw, db = [dev(x, BF16) for x in xs], dev(w_dev, BF16), dev(b_dev, BF16)
    for call in range(2):
        sp, v = S.fused_temporal_conv_lif_state(dx, dw, db, dv, [s, s], [p, p], [1, 1], 1, *lif, False)
        assert v.dtype == BF16 and CB.last_conv_plan()["launches"] > 1
        check(sp, v, ref, v_threshold=lif[0], v_dtype=BF16, what=f"bf16 membrane, {T} steps, call {call}")
    _no_fallback(hip_ops, 2)


def test_bf16_membrane_calls_of_one_layer_repeat_bit_for_bit(hip_ops):
    """A 3x3 layer with Cout % 64 == 0 at T = 4 takes the matrix kernel's one-launch variant with a float32 membrane and
    windows of 2 with a 16-bit one. Every call of the layer must compute the same way whatever earlier calls have
    recorded about it: calls 1..3 agree bit for bit, and equal the float32-membrane call with its membrane rounded once."""
    T, N, Cin, Cout, H, W = 4, 3, 64, 64, 16, 16
    xs, w_dev, b_dev, w_ref, b_ref = _conv_case(8150, T, N, Cin, Cout, H, W, 3, BF16, p=0.25)
    dx, dw, db = [dev(x, BF16) for x in xs], dev(w_dev, BF16), dev(b_dev, BF16)
    geo = ([1, 1], [1, 1], [1, 1], 1)
    runs = [S.fused_temporal_conv_lif_state(dx, dw, db, torch.tensor(0.0), *geo, *LIF, False) for _ in range(3)]
    for sp, v in runs:
        assert v.dtype == BF16
        assert torch.equal(sp, runs[0][0]) and torch.equal(v, runs[0][1])
    sp32, v32 = S.fused_temporal_conv_lif_state(dx, dw, db, zero_v(F32), *geo, *LIF, False)
    assert v32.dtype == F32
    assert torch.equal(sp32, runs[0][0]) and torch.equal(v32.to(BF16), runs[0][1])
    ref = O.temporal_conv_lif(xs, w_ref, b_ref, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *LIF)
    check(runs[0][0], runs[0][1], ref, v_dtype=BF16, what="bf16 membrane, repeated calls")
    _no_fallback(hip_ops, 4)


def test_bf16_membrane_beyond_sixteen_steps_in_the_other_operators(hip_ops):
    """Depthwise, linear and the standalone scan run more than 16 steps as windows of 16; same requirement."""
    g = gen(8200)
    T, N, C, H, W = 20, 3, 16, 14, 14
    xs = [spikes((N, C, H, W), 0.3, g) for _ in range(T)]
    w = q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, BF16)
    b = q(torch.randn(C, generator=g) * 0.1, BF16)
    soft = (1.0, -1.0, 2.0)
    ref = O.temporal_conv_lif(xs, w, b, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), C, *soft)
    s, v = S.fused_temporal_depthwise_conv_lif_state([dev(x, BF16) for x in xs], dev(w, BF16), dev(b, BF16), torch.tensor(0.0),
                                                     [1, 1], [1, 1], [1, 1], C, *soft, False)
    assert v.dtype == BF16
    check(s, v, ref, v_dtype=BF16, what="depthwise, 20 steps, bf16 membrane")

    x, w_dev, b_dev, w_ref, b_ref = _linear_case(8201, 20, 48, 256, 192, BF16, True)
    ref = O.temporal_linear_lif(x, w_ref, b_ref, torch.tensor(0.0), *soft)
    s, v = S.fused_temporal_linear_lif_state_packed(dev(x, BF16), dev(w_dev, BF16), dev(b_dev, BF16), torch.tensor(0.0), *soft, False)
    assert v.dtype == BF16
    check(s, v, ref, v_dtype=BF16, what="linear, 20 steps, bf16 membrane")

    x = q(torch.randn(40, 4, 16, 9, 9, generator=g) * 0.8, BF16)
    v0 = q(torch.randn(4, 16, 9, 9, generator=g) * 0.3, BF16)
    ref = O.temporal_lif(x, v0.float(), *soft)
    s, v = S.fused_temporal_lif_state(dev(x, BF16), dev(v0, BF16), *soft, False)
    assert v.dtype == BF16
    check(s, v, ref, v_dtype=BF16, what="scan, 40 steps, bf16 membrane")
    _no_fallback(hip_ops, 3)
