"""Seeded random sweeps over shapes, dtypes, neuron settings and layouts: every case goes through the operator (or the
blocked entry point) on the GPU and through the CPU oracle on the same operands, with the gate of the hand-picked cases
(tests/helpers.py:check). The hand-picked cases pin each kernel family; these sweeps look for what nobody thought of -
ragged planes, odd channel counts, windows that do not divide T, 16-bit membranes handed from launch to launch. Each case
prints its description before it runs."""
import collections
import random

import pytest
import torch

from helpers import DEV, check, dev, gen, q, spikes
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16
S = torch.ops.snn_custom
LIFS = [(1.0, 0.0, 2.0), (1.0, 0.0, 2.0), (1.0, -1.0, 2.0), (0.5, 0.0, 1.0), (1.0, 0.0, 3.0), (0.75, 0.25, 4.0)]
MAX_MACS = 2e9                      # per case, so that the oracle's convolution stays in the milliseconds


def _dtypes(rnd):
    dtype = rnd.choice([BF16, BF16, F16, F32])
    return dtype, (BF16 if dtype == F32 else dtype), (F32 if dtype == F32 else rnd.choice([F32, dtype]))


def _membrane(rnd, g, shape, vdtype):
    """A tensor state in the membrane dtype, or a 0-dim zero on the device that selects that dtype."""
    if rnd.random() < 0.4:
        v0 = q(torch.randn(shape, generator=g) * 0.3, vdtype)
        return v0.float(), dev(v0, vdtype)
    return torch.tensor(0.0), torch.zeros((), device=DEV, dtype=vdtype)


@pytest.mark.parametrize("seed,cases", [(11, 400)])
def test_random_dense_conv_lif_cases(hip_ops, seed, cases):
    from triton_snn_fusion_amd.runtime import hip_convlif_backend as CB
    rnd = random.Random(seed)
    kernels = collections.Counter()
    for case in range(cases):
        depthwise = rnd.random() < 0.15
        Cin = rnd.choice([1, 2, 3, 4, 8, 12, 16, 20, 24, 32, 36, 40, 64, 72, 96, 128, 136, 256, 512])
        Cout = Cin if depthwise else rnd.choice([1, 4, 8, 10, 16, 24, 32, 44, 64, 70, 96, 128, 192, 256, 512])
        k = 3 if depthwise else rnd.choice([1, 1, 1, 3, 3, 3, 5, 7])
        s = rnd.choice([1, 1, 2])
        p = 1 if depthwise else rnd.randint(0, k // 2)
        H, W = rnd.randint(max(1, k - 2 * p), 24), rnd.randint(max(1, k - 2 * p), 24)
        T, N = rnd.choice([1, 2, 3, 4, 4, 4, 5, 6, 8, 9, 17]), rnd.randint(1, 9)
        dtype, op_dt, vdtype = _dtypes(rnd)
        op_dt = dtype       # convolutions: fp32 operands stay unrounded (two bf16 terms each on the matrix cores; fp32 taps when depthwise)
        analog, with_res, lif = rnd.random() < 0.25, rnd.random() < 0.3, rnd.choice(LIFS)
        Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
        groups = Cin if depthwise else 1
        per_image = T * Cout * Ho * Wo * (Cin // groups) * k * k
        N = max(1, min(N, int(MAX_MACS / per_image)))
        if per_image > 2 * MAX_MACS:
            continue
        g = gen(seed * 100000 + case)
        xs = ([q(torch.randn(N, Cin, H, W, generator=g), op_dt) for _ in range(T)] if analog
              else [spikes((N, Cin, H, W), 0.25, g) for _ in range(T)])
        fan = (Cin // groups) * k * k
        w = q(torch.randn(Cout, Cin // groups, k, k, generator=g) * (2.0 / fan) ** 0.5 * (1.5 if depthwise else 2.0), op_dt)
        b = torch.randn(Cout, generator=g) * 0.1
        b = b if dtype == F32 else q(b, dtype)
        rs = [q(torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3, op_dt) for _ in range(T)] if with_res else None
        v_ref, v_dev = _membrane(rnd, g, (N, Cout, Ho, Wo), vdtype)
        what = (f"case {case}: {'depthwise ' if depthwise else ''}{Cin}->{Cout} {H}x{W} k{k} s{s} p{p} T={T} N={N} {dtype} "
                f"membrane {vdtype} analog={analog} residual={with_res} lif={lif} tensor v_init={v_ref.dim() > 0}")
        print(what, flush=True)
        ref = O.temporal_conv_lif(xs, w, b, v_ref, (s, s), (p, p), (1, 1), groups, *lif, residuals=rs)
        CB.clear_packed_weight_cache()
        args = ([dev(x, dtype) for x in xs],) + (([dev(r, dtype) for r in rs],) if with_res else ())
        op = S.fused_temporal_conv_add_lif_state if with_res else S.fused_temporal_conv_lif_state
        sp, v = op(*args, dev(w, dtype), dev(b, dtype), v_dev, [s, s], [p, p], [1, 1], groups, *lif, False)
        assert sp.dtype == dtype and v.dtype == vdtype
        check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=what, max_rate=2e-4)
        kernels["depthwise" if depthwise else CB.last_conv_plan()["kernel"]] += 1
    print(dict(kernels), flush=True)
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0
    assert set(kernels) >= {"matrix", "pointwise", "time_outer", "t_in_m", "depthwise"}, kernels   # the sweep reaches every family


@pytest.mark.parametrize("seed,cases", [(12, 400)])
def test_random_blocked_conv_lif_cases(snnf_lib, seed, cases):
    from triton_snn_fusion_amd import _lib
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B, hip_convlif_backend as CB
    rnd = random.Random(seed)
    lay = {"nchw": B.NCHW, "c8": B.C8, "bits": B.BITS}
    ran = 0
    for case in range(cases):
        Cin = rnd.choice([8, 16, 20, 24, 32, 40, 64, 72, 96, 128, 136, 256, 320])
        Cout = rnd.choice([8, 16, 24, 32, 44, 64, 72, 96, 128, 192, 256, 320])
        k, s = rnd.choice([1, 1, 3, 3, 3, 5, 7]), rnd.choice([1, 1, 2])
        p = rnd.randint(0, k // 2)
        H, W = rnd.randint(max(1, k - 2 * p), 40), rnd.randint(max(1, k - 2 * p), 40)
        T, N = rnd.choice([1, 2, 3, 4, 4, 4, 5, 6, 8, 9]), rnd.randint(1, 9)
        dtype = rnd.choice([BF16, BF16, F16])
        inl, resl, outl = rnd.choice(["bits", "bits", "bits", "c8"]), rnd.choice([None, None, "bits", "c8", "nchw"]), rnd.choice(["bits", "bits", "c8", "nchw"])
        lif, tensor_v, want_v = rnd.choice(LIFS), rnd.random() < 0.4, rnd.random() < 0.7
        Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
        per_image = T * Cout * Ho * Wo * Cin * k * k
        N = max(1, min(N, int(MAX_MACS / per_image)))
        if per_image > 2 * MAX_MACS:
            continue
        what = f"case {case}: {Cin}->{Cout} {H}x{W} k{k} s{s} p{p} T={T} N={N} {dtype} {inl}/{resl}/{outl} lif={lif} tensor v_init={tensor_v} membrane out={want_v}"
        print(what, flush=True)
        g = gen(seed * 100000 + case)
        xs = q(torch.randn(T, N, Cin, H, W, generator=g), dtype) if inl == "c8" else spikes((T, N, Cin, H, W), 0.25, g)
        w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * 2.0, dtype)
        b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
        rs = None
        if resl == "bits":
            rs = spikes((T, N, Cout, Ho, Wo), 0.3, g)
        elif resl is not None:
            rs = q(torch.randn(T, N, Cout, Ho, Wo, generator=g) * 0.3, dtype)
        v0 = torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3 if tensor_v else torch.tensor(0.0)
        ref = O.temporal_conv_lif([xs[t] for t in range(T)], w, b, v0, (s, s), (p, p), (1, 1), 1, *lif,
                                  residuals=None if rs is None else [rs[t] for t in range(T)])
        CB.clear_packed_weight_cache()
        try:
            out, v = B.conv_lif_blocked(B.from_dense(dev(xs, dtype), lay[inl]), dev(w, dtype), dev(b, dtype), [s, s], [p, p], lif,
                                        residual=None if rs is None else B.from_dense(dev(rs, dtype), lay[resl]),
                                        out_layout=lay[outl], v_init=dev(v0, F32) if tensor_v else None, want_v=want_v)
        except _lib.SnnfError as e:          # windows the blocked kernel does not take are refused, not miscomputed
            assert "unsupported" in str(e), str(e)
            continue
        ran += 1
        dense = B.to_dense(out)
        if v is None:
            v = dev(ref[1], F32)             # membrane not requested: the spikes carry the whole check
        check(dense, v, ref, v_threshold=lif[0], what=what, max_rate=2e-4)
    assert ran > 0.9 * cases


@pytest.mark.parametrize("seed,cases", [(13, 400)])
def test_random_linear_scan_and_tail_cases(hip_ops, seed, cases):
    rnd = random.Random(seed)
    for case in range(cases):
        kind = rnd.choice(["linear", "linear", "scan", "tail"])
        dtype, op_dt, vdtype = _dtypes(rnd)
        lif = rnd.choice(LIFS)
        g = gen(seed * 100000 + case)
        if kind == "linear":
            T, M = rnd.choice([1, 2, 3, 4, 4, 5, 8, 12, 16, 17, 33]), rnd.choice([1, 2, 3, 5, 16, 17, 33, 64, 100, 128])
            Fin = rnd.choice([8, 16, 37, 64, 100, 128, 200, 256, 264, 512, 1000, 2048, 4096, 4104])
            Fout = rnd.choice([1, 8, 16, 37, 48, 64, 100, 130, 256, 1000, 1024])
            bias = rnd.random() < 0.8
            analog = rnd.random() < 0.2
            x = q(torch.randn(T, M, Fin, generator=g) * 0.3, dtype) if analog else spikes((T, M, Fin), 0.1, g)
            w = q(torch.randn(Fout, Fin, generator=g) * (2.0 / Fin) ** 0.5 * 3.0, dtype)      # fp32 stays fp32: two bf16 terms on the matrix cores
            b = None if not bias else (torch.randn(Fout, generator=g) * 0.01 if dtype == F32 else q(torch.randn(Fout, generator=g) * 0.01, dtype))
            v_ref, v_dev = _membrane(rnd, g, (M, Fout), vdtype)
            what = f"case {case}: linear T={T} M={M} {Fin}->{Fout} bias={bias} {dtype} membrane {vdtype} lif={lif}"
            print(what, flush=True)
            ref = O.temporal_linear_lif(x, w, b, v_ref, *lif)
            fb = dev(b, dtype) if bias else torch.empty(0, device=DEV, dtype=dtype)
            sp, v = S.fused_temporal_linear_lif_state_packed(dev(x, dtype), dev(w, dtype), fb, v_dev, *lif, False)
            check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=what, max_rate=2e-4)
        elif kind == "scan":
            T = rnd.choice([1, 2, 4, 7, 16, 17, 40])
            shape = (rnd.randint(1, 5), rnd.randint(1, 40), rnd.randint(1, 30), rnd.randint(1, 30))
            x = q(torch.randn((T,) + shape, generator=g) * 0.8, dtype)
            v_ref, v_dev = _membrane(rnd, g, shape, vdtype)
            what = f"case {case}: scan T={T} {shape} {dtype} membrane {vdtype} lif={lif}"
            print(what, flush=True)
            ref = O.temporal_lif(x, v_ref, *lif)
            sp, v = S.fused_temporal_lif_state(dev(x, dtype), v_dev, *lif, False)
            check(sp, v, ref, v_threshold=lif[0], v_dtype=vdtype, what=what, max_rate=2e-4)
        else:
            T, N, C = rnd.choice([1, 2, 3, 4, 4, 8, 16]), rnd.randint(1, 20), rnd.choice([3, 8, 32, 50, 64, 128, 512])
            H, W, K = rnd.choice([1, 2, 3, 4, 5, 7, 14, 25]), rnd.choice([1, 2, 3, 4, 5, 7, 14, 25]), rnd.choice([1, 3, 10, 17, 64, 70, 100, 1000])
            mean = rnd.choice([0.15, 0.15, 2.0])     # strong inputs: spike counts beyond 255 (the matrix-core GEMV splits them)
            x = q(torch.randn(T, N, C, H, W, generator=g) * 0.75 + mean, dtype)
            w, b = q(torch.randn(K, C, generator=g) * 0.05, dtype), q(torch.randn(K, generator=g) * 0.05, dtype)
            v_ref, v_dev = _membrane(rnd, g, (N, C, H, W), F32)
            what = f"case {case}: tail T={T} N={N} C={C} {H}x{W} K={K} {dtype} lif={lif}"
            print(what, flush=True)
            ref_out, ref_v, _, _ = O.temporal_lif_avgpool_linear(x, v_ref, w, b, *lif)
            out, v = S.fused_temporal_lif_avgpool_linear(dev(x, dtype), v_dev, dev(w, dtype), dev(b, dtype), *lif, False)
            tol = 1e-4 if dtype == F32 else (8e-3 if dtype == BF16 else 2e-3)      # out_sum is stored in the activation dtype
            assert torch.allclose(v.cpu(), ref_v, rtol=1e-6, atol=1e-6), what
            assert torch.allclose(out.float().cpu(), ref_out, rtol=tol, atol=tol), what
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0


@pytest.mark.parametrize("seed,cases", [(17, 150)])
def test_random_row_packed_depthwise_and_pointwise_cases(hip_ops, seed, cases):
    """The entry points on row-packed spikes against the dense operators (themselves gated on the oracle above): the same
    kernels with another fetch or store, so spikes and membranes are compared bit for bit."""
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    rnd = random.Random(seed)
    zero = torch.zeros((), device=DEV, dtype=F32)
    pointwise_cases = 0
    for case in range(cases):
        dtype = rnd.choice([BF16, F16])
        T, N = rnd.choice([1, 2, 3, 4, 4, 5, 8, 16, 17, 20]), rnd.randint(1, 5)
        H, W = rnd.choice([1, 2, 4, 7, 8, 12, 16, 28]), rnd.choice([8, 16, 24, 32, 56, 64])
        C, Cout = rnd.choice([2, 3, 8, 16, 24, 40, 64, 128, 200, 256]), rnd.choice([32, 64, 96, 128, 160, 256, 320])
        lif = (rnd.choice([1.0, 0.5]), rnd.choice([0.0, 0.0, 0.25]), rnd.choice([2.0, 2.0, 4.0, 1.0]))
        tensor_v, residual = rnd.random() < 0.4, rnd.random() < 0.3
        g = gen(seed * 100000 + case)
        what = f"case {case}: {dtype} T={T} N={N} C={C}->{Cout} {H}x{W} lif={lif} v_init={tensor_v} residual={residual}"
        print(what, flush=True)
        xs = [dev(spikes((N, C, H, W), 0.3, g), dtype) for _ in range(T)]
        wd, bd = dev(q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, dtype), dtype), dev(q(torch.randn(C, generator=g) * 0.1, dtype), dtype)
        rs = [dev(q(torch.randn(N, C, H, W, generator=g) * 0.3, dtype), dtype) for _ in range(T)] if residual else None
        v0 = dev(torch.randn(N, C, H, W, generator=g) * 0.3, F32) if tensor_v else None
        if residual:
            s_d, v_d = S.fused_temporal_conv_add_lif_state_depthwise(xs, rs, wd, bd, v0 if tensor_v else zero, [1, 1], [1, 1], [1, 1], C, *lif, False)
        else:
            s_d, v_d = S.fused_temporal_depthwise_conv_lif_state(xs, wd, bd, v0 if tensor_v else zero, [1, 1], [1, 1], [1, 1], C, *lif, False)
        bits, v = B.depthwise_conv_lif_rowbits(xs, wd, bd, lif, residuals=rs, v_init=v0)
        assert torch.equal(B.unpack_rowbits(bits, dtype), s_d) and torch.equal(v, v_d), what
        bits2, v2 = B.depthwise_conv_lif_rowbits(B.pack_rowbits(torch.stack(xs)), wd, bd, lif, residuals=rs, v_init=v0)
        assert torch.equal(bits2, bits) and torch.equal(v2, v), what
        if C % 8 != 0 or (H * W) % 64 != 0 or lif[2] == 1.0:      # outside the pointwise kernel's fast variant: refused, see the blocked tests
            continue
        wp = dev(q(torch.randn(Cout, C, 1, 1, generator=g) * (2.0 / C) ** 0.5 * 2.0, dtype), dtype)
        bp = dev(q(torch.randn(Cout, generator=g) * 0.1, dtype), dtype)
        vp0 = dev(torch.randn(N, Cout, H, W, generator=g) * 0.3, F32) if tensor_v else None
        sp_d, vp_d = S.fused_temporal_pointwise_conv_lif_state(list(s_d.unbind(0)), wp, bp, vp0 if tensor_v else zero, [1, 1], [0, 0], [1, 1], 1,
                                                               *lif, False)
        same_kernel = last_conv_plan()["kernel"] == "pointwise"
        sp, vp = B.pointwise_conv_lif_from_rowbits(bits, wp, bp, lif, v_init=vp0)
        pb, pv = B.pointwise_conv_lif_from_rowbits(bits, wp, bp, lif, v_init=vp0, packed_out=True)
        assert torch.equal(B.unpack_rowbits(pb, dtype), sp) and torch.equal(pv, vp), what
        if same_kernel:
            assert torch.equal(sp, sp_d) and torch.equal(vp, vp_d), what
        else:                                                      # the operator ran the matrix kernel: another summation order
            assert (sp != sp_d).float().mean().item() < 2e-3, what
        pointwise_cases += 1
    assert pointwise_cases >= cases // 8


@pytest.mark.parametrize("seed,cases", [(19, 600)])
def test_random_fused_blocked_cases(snnf_lib, seed, cases):
    """The forms that take a neighbour into a convolution's launch: a projection shortcut in the accumulators (against the oracle
    with the shortcut's unrounded sums as its residual), the 2x2 average pool of the spikes (bit for bit the two launches, and
    the oracle), pool + classifier on bit-packed spikes (exact counts, float64 dot products)."""
    from triton_snn_fusion_amd import _lib
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B, hip_convlif_backend as CB
    rnd = random.Random(seed)
    lay = {"nchw": B.NCHW, "c8": B.C8, "bits": B.BITS}
    ran = collections.Counter()
    for case in range(cases):
        kind = rnd.choice(["shortcut", "shortcut", "pool", "tail"])
        dtype = rnd.choice([BF16, BF16, F16])
        g = gen(seed * 100000 + case)
        CB.clear_packed_weight_cache()
        if kind == "shortcut":
            Cin, Cs = rnd.choice([16, 32, 48, 64, 128, 256]), rnd.choice([16, 32, 64, 96, 128])
            Cout = rnd.choice([8, 24, 32, 64, 72, 128, 192, 256])
            k, ss = rnd.choice([1, 3, 3, 3, 5]), rnd.choice([1, 2, 2, 3])
            H, W = rnd.randint(1, 20), rnd.randint(1, 20)
            T, N = rnd.choice([3, 4, 4, 4, 5, 8]), rnd.randint(1, 6)
            lif, outl, want_v = rnd.choice(LIFS), rnd.choice(["bits", "bits", "c8", "nchw"]), rnd.random() < 0.6
            Hs, Ws = (H - 1) * ss + 1 + rnd.randint(0, ss - 1), (W - 1) * ss + 1 + rnd.randint(0, ss - 1)
            per_image = T * Cout * H * W * (Cin * k * k + Cs)
            N = max(1, min(N, int(MAX_MACS / per_image)))
            what = f"case {case}: {Cin}->{Cout} {H}x{W} k{k} + shortcut {Cs}->{Cout} /{ss} from {Hs}x{Ws} T={T} N={N} {dtype} -> {outl} lif={lif} membrane out={want_v}"
            print(what, flush=True)
            xs, x2 = spikes((T, N, Cin, H, W), 0.25, g), spikes((T, N, Cs, Hs, Ws), 0.25, g)
            w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * 2.0, dtype)
            w2 = q(torch.randn(Cout, Cs, 1, 1, generator=g) * (2.0 / Cs) ** 0.5, dtype)
            b, b2 = q(torch.randn(Cout, generator=g) * 0.1, dtype), q(torch.randn(Cout, generator=g) * 0.1, dtype)
            shortcut = [torch.nn.functional.conv2d(x2[t], w2, b2, stride=ss) for t in range(T)]
            ref = O.temporal_conv_lif([xs[t] for t in range(T)], w, b, torch.tensor(0.0), (1, 1), (k // 2, k // 2), (1, 1), 1, *lif, residuals=shortcut)
            try:
                out, v = B.conv_lif_blocked_shortcut(B.from_dense(dev(xs, dtype), B.BITS), dev(w, dtype), dev(b, dtype), [k // 2, k // 2],
                                                     B.from_dense(dev(x2, dtype), B.BITS), dev(w2, dtype), dev(b2, dtype), [ss, ss], lif,
                                                     out_layout=lay[outl], want_v=want_v)
            except _lib.SnnfError as e:      # plans without room for the shortcut's stages are refused, not miscomputed
                assert "unsupported" in str(e), str(e)
                continue
            if v is None:
                v = dev(ref[1], F32)
            check(B.to_dense(out), v, ref, v_threshold=lif[0], what=what, max_rate=2e-4)
        elif kind == "pool":
            Cin, Cout = rnd.choice([3, 8, 16, 32, 64, 128, 256]), rnd.choice([8, 16, 32, 64, 72, 128, 256])
            k, s = rnd.choice([1, 3, 3, 3, 5]), rnd.choice([1, 1, 2])
            p = k // 2
            Ho, Wo = 2 * rnd.randint(1, 10), 2 * rnd.randint(1, 10)
            H, W = (Ho - 1) * s + 1, (Wo - 1) * s + 1                 # (H + 2 p - k) // s + 1 == Ho with p = k // 2
            N = rnd.randint(1, 8)
            inl = "frame" if Cin == 3 else rnd.choice(["bits", "bits", "c8"])
            T = 4
            per_image = T * Cout * Ho * Wo * Cin * k * k
            N = max(1, min(N, int(MAX_MACS / per_image)))
            what = f"case {case}: {Cin}->{Cout} {H}x{W} k{k} s{s} + 2x2 average pool N={N} {dtype} {inl}"
            print(what, flush=True)
            if inl == "frame":
                frame = q(torch.randn(N, Cin, H, W, generator=g), dtype)
                frames, x = [frame] * T, B.input_frame(dev(frame, dtype), T)
            else:
                xs = q(torch.randn(T, N, Cin, H, W, generator=g), dtype) if inl == "c8" else spikes((T, N, Cin, H, W), 0.25, g)
                frames, x = [xs[t] for t in range(T)], B.from_dense(dev(xs, dtype), lay[inl])
            w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * 2.0, dtype)
            b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
            lif = (1.0, 0.0, 2.0)
            ref = O.temporal_conv_lif(frames, w, b, torch.tensor(0.0), (s, s), (p, p), (1, 1), 1, *lif)
            try:
                pooled, v = B.conv_lif_blocked_avgpool(x, dev(w, dtype), dev(b, dtype), [s, s], [p, p], lif, want_v=True)
            except _lib.SnnfError as e:
                assert "unsupported" in str(e), str(e)
                continue
            plan = B.last_conv_plan()
            sp, v2 = B.conv_lif_blocked(x, dev(w, dtype), dev(b, dtype), [s, s], [p, p], lif, want_v=True)
            plan2 = B.last_conv_plan()
            two = B.pool_blocked(sp, False, 2, 2, 0)
            if (plan["waves"], plan["stage_chunks"]) == (plan2["waves"], plan2["stage_chunks"]):
                # the same partition of K over waves and stages: the same sums, bit for bit
                assert torch.equal(pooled.data, two.data) and torch.equal(v, v2), what
            else:
                # even patches changed how K is shared: another summation order, spikes equal but for neurons at the threshold
                assert float((pooled.data != two.data).float().mean()) < 2e-3, what
            rep_ = check(B.to_dense(sp), v, ref, what=what, max_rate=2e-4)
            check(B.to_dense(sp), v2, ref, what=what, max_rate=2e-4)
            got = B.to_dense(pooled).float().cpu()
            want = torch.nn.functional.avg_pool2d(ref[0].flatten(0, 1), 2).reshape(got.shape)
            assert float((got != want).float().mean()) <= 4 * (1.0 - rep_["neurons_with_matching_history"] / rep_["neurons"]) + 2e-3, what
        else:
            T, N, C = rnd.choice([1, 2, 3, 4, 4, 8, 16]), rnd.randint(1, 20), 8 * rnd.choice([1, 2, 3, 8, 16, 40, 64, 256])
            H, W, K = rnd.choice([1, 2, 3, 4, 5, 7, 14, 25]), rnd.choice([1, 2, 3, 4, 5, 7, 14, 25]), rnd.choice([1, 3, 10, 17, 64, 70, 100, 1000])
            scale = rnd.choice([1.0, 1.0 / T])
            what = f"case {case}: pool + classifier on bits T={T} N={N} C={C} {H}x{W} K={K} {dtype} scale={scale}"
            print(what, flush=True)
            s_ = spikes((T, N, C, H, W), rnd.choice([0.1, 0.5, 1.0]), g)
            w = q(torch.randn(K, C, generator=g) * 0.05, dtype)
            b = q(torch.randn(K, generator=g) * 0.05, dtype) if rnd.random() < 0.8 else None
            got = B.spike_pool_linear(B.from_dense(dev(s_, dtype), B.BITS), dev(w, dtype), None if b is None else dev(b, dtype), scale)
            want = scale * (s_.double().sum((0, 3, 4)) @ w.double().t() / (H * W) + (0.0 if b is None else T * b.double()))
            eps = 2.0 ** -8 if dtype == BF16 else 2.0 ** -11
            assert torch.allclose(got.double().cpu(), want, rtol=eps, atol=2e-4), (what, float((got.double().cpu() - want).abs().max()))
        ran[kind] += 1
    assert ran["shortcut"] > 0.25 * cases and ran["pool"] > 0.12 * cases and ran["tail"] > 0.12 * cases, ran


@pytest.mark.parametrize("seed,cases", [(23, 120)])
def test_random_small_plane_cases(snnf_lib, seed, cases):
    """Convolution + LIF on planes of one to four pixels with a bit-packed output and no membrane output: one matrix product
    per frame on the Linear + LIF kernel, from bits or from channel-blocked elements, all neuron settings, kernels larger than
    the plane, batches that leave row tiles ragged, matrices long enough for the K split over workgroups."""
    import torch.nn.functional as F
    from triton_snn_fusion_amd.runtime import hip_blocked_backend as B
    rnd = random.Random(seed)
    ran = collections.Counter()
    for case in range(cases):
        dtype = rnd.choice([BF16, BF16, F16])
        g = gen(seed * 100000 + case)
        H, W = rnd.choice([(1, 1), (1, 2), (2, 1), (2, 2), (2, 2), (2, 2), (1, 3), (4, 1)])
        Cin, Cout = 8 * rnd.choice([1, 2, 3, 8, 16, 33, 64, 128]), 8 * rnd.choice([1, 2, 4, 5, 16, 32, 64])
        kh, kw = rnd.choice([1, 3, 3, 3, 5]), rnd.choice([1, 3, 3, 3, 5])
        T, N = rnd.choice([3, 4, 4, 4, 5, 6, 8]), rnd.choice([1, 2, 5, 8, 9, 16, 17, 40, 64])
        lif = rnd.choice(LIFS)
        source = rnd.choice(["bits", "bits", "quarters", "analog"])
        if (Cout * H * W) % 32 != 0 or Cin * H * W * Cout * H * W > B.PLANE_MATRIX_MAX_ELEMENTS:
            continue
        what = f"case {case}: {Cin}->{Cout} {H}x{W} k{kh}x{kw} T={T} N={N} {dtype} {source} lif={lif}"
        print(what, flush=True)
        if source == "bits":
            x = spikes((T, N, Cin, H, W), rnd.choice([0.1, 0.3]), g)
            bx = B.from_dense(dev(x, dtype), B.BITS)
        elif source == "quarters":
            x = F.avg_pool2d(spikes((T * N, Cin, 2 * H, 2 * W), 0.3, g), 2).reshape(T, N, Cin, H, W)
            bx = B.from_dense(dev(x, dtype), B.C8)
        else:
            x = q(torch.randn(T, N, Cin, H, W, generator=g) * 0.4, dtype)
            bx = B.from_dense(dev(x, dtype), B.C8)
        taps = min(kh, 2 * H - 1) * min(kw, 2 * W - 1)
        w = q(torch.randn(Cout, Cin, kh, kw, generator=g) * (2.0 / (Cin * min(taps, H * W))) ** 0.5 * 2.5, dtype)
        b = q(torch.randn(Cout, generator=g) * 0.1, dtype) if rnd.random() < 0.8 else None
        ref = O.temporal_conv_lif([x[t] for t in range(T)], w, b, torch.tensor(0.0), (1, 1), (kh // 2, kw // 2), (1, 1), 1, *lif)
        out, v = B.conv_lif_blocked(bx, dev(w, dtype), None if b is None else dev(b, dtype), 1, [kh // 2, kw // 2], lif, out_layout=B.BITS)
        plan = B.last_conv_plan()
        assert v is None and plan["kernel"] == "plane_matrix", (what, plan)
        check(B.to_dense(out), ref[1], ref, v_threshold=lif[0], what=what, max_rate=2e-4)      # spikes only: the oracle's membrane stands in
        ran[source] += 1
    print(dict(ran))
    assert min(ran[s] for s in ("bits", "quarters", "analog")) >= 10, ran
