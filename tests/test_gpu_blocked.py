"""GPU parity of the internal activation layouts (channel-blocked C8, bit-packed BITS): layout conversion and pooling are
exact against plain tensor arithmetic; the blocked convolution + LIF kernel is gated against the CPU oracle like the dense
operators (tests/helpers.py:check), with its bit-packed / blocked outputs converted back to dense tensors first, and
bit for bit against the dense operator of the same library where both run the same arithmetic order is not required:
the gate is the oracle's.
"""
import pytest
import torch

from helpers import DEV, LIF, check, dev, gen, q, spikes
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16


@pytest.fixture()
def B(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime import hip_blocked_backend
    from triton_snn_fusion_amd.runtime import hip_convlif_backend
    hip_convlif_backend.clear_packed_weight_cache()
    return hip_blocked_backend


def _ref_groups(x):
    """[T, N, C, H, W] -> [T, N, C8, 8, H, W] with zero channels appended."""
    T, N, C, H, W = x.shape
    c8 = (C + 7) // 8
    pad = torch.zeros(T, N, c8 * 8 - C, H, W, dtype=x.dtype)
    return torch.cat([x, pad], 2).reshape(T, N, c8, 8, H, W)


def _ref_bits(x):
    g = (_ref_groups(x) != 0).to(torch.int32)
    weights = (2 ** torch.arange(8, dtype=torch.int32)).reshape(1, 1, 1, 8, 1, 1)
    return (g * weights).sum(3).to(torch.uint8)


def _ref_c8(x):
    return _ref_groups(x).permute(0, 1, 2, 4, 5, 3).contiguous()


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("shape", [(2, 3, 16, 5, 7), (1, 2, 20, 9, 9), (4, 1, 3, 8, 8), (1, 1, 64, 14, 14), (3, 2, 8, 1, 1)])
def test_layout_conversions_are_exact(B, shape, dtype):
    g = gen(3000 + shape[2])
    s = spikes(shape, 0.3, g)
    a = q(torch.randn(shape, generator=g), dtype)
    ds, da = dev(s, dtype), dev(a, dtype)
    bits = B.from_dense(ds, B.BITS)
    assert bits.data.dtype == torch.uint8 and torch.equal(bits.data.cpu(), _ref_bits(s))
    c8 = B.from_dense(da, B.C8)
    assert torch.equal(c8.data.float().cpu(), _ref_c8(a))
    assert torch.equal(B.to_dense(bits).float().cpu(), s)
    assert torch.equal(B.to_dense(c8).float().cpu(), a)
    # between the internal layouts
    assert torch.equal(B.convert(B.from_dense(ds, B.C8), B.BITS).data.cpu(), _ref_bits(s))
    assert torch.equal(B.convert(bits, B.C8).data.float().cpu(), _ref_c8(s))


@pytest.mark.parametrize("kind,k,p,shape", [("max", 3, 1, (4, 2, 64, 16, 16)), ("max", 3, 1, (2, 1, 20, 9, 11)), ("max", 2, 0, (1, 3, 8, 6, 10)),
                                            ("max", 2, 0, (2, 2, 24, 8, 16)), ("max", 3, 1, (1, 2, 16, 10, 24)),
                                            ("avg", 2, 0, (4, 2, 64, 8, 8)), ("avg", 2, 0, (2, 2, 12, 7, 9)),
                                            ("avg", 2, 0, (2, 3, 20, 6, 24)), ("avg", 2, 0, (1, 2, 8, 5, 16))])
def test_pooling_on_the_internal_layouts_is_exact(B, kind, k, p, shape):
    g = gen(3100 + shape[2] + k)
    s = spikes(shape, 0.3, g)
    a = q(torch.randn(shape, generator=g), BF16)
    module = torch.nn.MaxPool2d(k, 2, p) if kind == "max" else torch.nn.AvgPool2d(2)
    want_s = module(s.flatten(0, 1)).reshape(shape[0], shape[1], shape[2], *module(s.flatten(0, 1)).shape[-2:])
    want_a = module(a.flatten(0, 1)).reshape(want_s.shape)
    bits = B.from_dense(dev(s, BF16), B.BITS)
    ps = B.pool_blocked(bits, kind == "max", k, 2, p)
    assert ps.layout == (B.BITS if kind == "max" else B.C8)
    assert torch.equal(B.to_dense(ps).float().cpu(), want_s)             # quarters are exact in bf16
    pa = B.pool_blocked(B.from_dense(dev(a, BF16), B.C8), kind == "max", k, 2, p)
    assert pa.layout == B.C8
    assert torch.allclose(B.to_dense(pa).float().cpu(), q(want_a, BF16), rtol=2 ** -8, atol=1e-6)


def _case(seed, T, N, Cin, Cout, H, W, k, dtype, analog=False, p=0.25, gain=2.0, shared=False):
    g = gen(seed)
    if analog:
        frames = 1 if shared else T
        xs = q(torch.randn(frames, N, Cin, H, W, generator=g), dtype)
    else:
        xs = spikes((T, N, Cin, H, W), p, g)
    w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * k * k)) ** 0.5 * gain, dtype)
    b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    return xs, w, b


BLOCKED_CASES = [  # Cin, Cout, H, W, k, s, p, dtype, lif, T, N, in layout, residual layout, out layout, tensor v_init
    (64, 64, 16, 16, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 2, "bits", None, "bits", False),     # the common layer
    (64, 64, 16, 16, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 2, "bits", "bits", "bits", True),    # + bit-packed residual, v_init
    (32, 96, 12, 12, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 3, 2, "bits", "c8", "c8", False),       # 3 of 4 steps, blocked residual and output
    (64, 72, 9, 11, 3, 1, 1, BF16, (1.0, -1.0, 2.0), 2, 3, "bits", "nchw", "nchw", True),    # ragged planes, Cout % 8 == 0 only, soft reset, dense ends
    (20, 44, 10, 10, 3, 1, 1, BF16, (0.5, 0.0, 1.0), 1, 2, "bits", None, "bits", False),     # channel counts that are no multiples of 8, IF neuron
    (64, 128, 16, 16, 3, 2, 1, BF16, (1.0, 0.0, 2.0), 4, 2, "bits", None, "bits", False),    # stride 2: windows of 2 steps
    (64, 128, 16, 16, 1, 2, 0, BF16, (1.0, 0.0, 2.0), 4, 2, "bits", None, "bits", False),    # strided 1x1
    (128, 64, 8, 8, 1, 1, 0, BF16, (1.0, 0.0, 3.0), 4, 2, "bits", None, "bits", True),       # plain 1x1, tau not a power of two
    (64, 64, 12, 12, 5, 1, 2, F16, (1.0, 0.0, 2.0), 4, 2, "bits", None, "bits", False),      # 5x5, fp16
    (64, 64, 14, 14, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 6, 2, "bits", "bits", "bits", False),   # two windows (4 + 2)
    (64, 64, 8, 8, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 2, "c8", None, "bits", False),         # analog blocked input
    (256, 128, 7, 7, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 4, "bits", "bits", "bits", True),    # 7x7 planes, K split over waves
    (512, 128, 4, 4, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 6, "bits", None, "bits", False),     # 4x4 planes: two images per patch, K split
    (128, 128, 2, 2, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 20, "bits", "c8", "bits", True),     # 2x2 planes: eight images per patch
    (512, 512, 7, 7, 3, 1, 1, BF16, (1.0, 0.0, 2.0), 4, 4, "bits", None, "nchw", False),     # deep layer, dense output
]


def _to_layout(B, t, name, dtype):
    return B.from_dense(dev(t, dtype), {"nchw": B.NCHW, "c8": B.C8, "bits": B.BITS}[name])


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p,dtype,lif,T,N,inl,resl,outl,tensor_v", BLOCKED_CASES)
def test_blocked_conv_lif_against_the_oracle(B, Cin, Cout, H, W, k, s, p, dtype, lif, T, N, inl, resl, outl, tensor_v):
    xs, w, b = _case(3200 + Cin + Cout + H + k + T, T, N, Cin, Cout, H, W, k, dtype, analog=inl == "c8")
    Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    g = gen(3201 + Cin)
    if resl == "bits":
        rs = spikes((T, N, Cout, Ho, Wo), 0.3, g)
    elif resl is not None:
        rs = q(torch.randn(T, N, Cout, Ho, Wo, generator=g) * 0.3, dtype)
    else:
        rs = None
    v0 = torch.randn(N, Cout, Ho, Wo, generator=g) * 0.3 if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif([xs[t] for t in range(T)], w, b, v0, (s, s), (p, p), (1, 1), 1, *lif,
                              residuals=None if rs is None else [rs[t] for t in range(T)])
    x = _to_layout(B, xs, inl, dtype)
    res = None if rs is None else _to_layout(B, rs, resl, dtype)
    out_layout = {"nchw": B.NCHW, "c8": B.C8, "bits": B.BITS}[outl]
    print(f"blocked conv {Cin}->{Cout} {H}x{W} k{k} s{s} T={T} N={N} {inl}/{resl}/{outl}", flush=True)
    out, v = B.conv_lif_blocked(x, dev(w, dtype), dev(b, dtype), [s, s], [p, p], lif, residual=res, out_layout=out_layout,
                                v_init=dev(v0, F32) if tensor_v else None, want_v=True)
    torch.cuda.synchronize()
    assert B.last_conv_plan()["kernel"] == "blocked"
    assert out.layout == out_layout and out.shape == (T, N, Cout, Ho, Wo) and v.dtype == F32
    rep = check(B.to_dense(out), v, ref, v_threshold=lif[0], what=f"blocked {Cin}->{Cout} k{k} s{s} {inl}->{outl}")
    assert 0.001 < float(ref[0].mean()) < 0.9, float(ref[0].mean())
    assert rep["neurons_with_matching_history"] >= 0.999 * rep["neurons"]
    if outl != "nchw" and Cout % 8:       # padded channels of the internal layouts hold zeros
        c8 = (Cout + 7) // 8
        if outl == "bits":
            assert int((out.data[:, :, c8 - 1] >> (Cout % 8)).max()) == 0
        else:
            assert float(out.data[:, :, c8 - 1, :, :, Cout % 8:].abs().max()) == 0.0


SHORTCUT_CASES = [  # main Cin, Cout, H, W, k, shortcut Cin, shortcut stride, T, N, dtype, lif, out layout
    (128, 128, 8, 8, 3, 64, 2, 4, 2, BF16, (1.0, 0.0, 2.0), "bits"),      # a ResNet downsample block, K shared by waves
    (32, 64, 12, 12, 3, 32, 2, 4, 2, BF16, (1.0, 0.0, 2.0), "bits"),      # one main stage: a wave per tile
    (128, 96, 9, 11, 3, 48, 2, 4, 3, BF16, (1.0, -0.5, 3.0), "nchw"),     # ragged planes, odd shortcut plane, general epilogue, dense output
    (64, 72, 10, 10, 3, 32, 1, 3, 2, BF16, (1.0, 0.0, 2.0), "c8"),        # shortcut of stride 1, 3 of 4 steps, blocked output
    (64, 64, 14, 14, 3, 64, 2, 6, 2, BF16, (1.0, 0.0, 2.0), "bits"),      # two windows (4 + 2)
    (64, 128, 8, 8, 5, 32, 2, 4, 2, F16, (1.0, 0.0, 2.0), "bits"),        # 5x5 main kernel, fp16
    (512, 512, 7, 7, 3, 256, 2, 4, 4, BF16, (1.0, 0.0, 2.0), "bits"),     # the deepest block: K shared by eight waves
    (256, 256, 4, 4, 3, 128, 2, 4, 6, BF16, (1.0, 0.0, 2.0), "bits"),     # two images per patch
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,Cs,ss,T,N,dtype,lif,outl", SHORTCUT_CASES)
def test_blocked_conv_with_the_projection_shortcut_in_its_accumulators(B, Cin, Cout, H, W, k, Cs, ss, T, N, dtype, lif, outl):
    """LIF(conv(x) + conv1x1(shortcut input, stride)) in one launch, against the oracle with the shortcut's output as its
    (unrounded fp32) residual, and against the same layer run as two launches within the rounding of the shortcut's output."""
    xs, w, b = _case(3400 + Cin + Cout + H + k + T, T, N, Cin, Cout, H, W, k, dtype)
    g = gen(3401 + Cs)
    Hs, Ws = (H - 1) * ss + 1 + (ss - 1) * (H % 2), (W - 1) * ss + 1          # both the smallest and a larger plane that lands on H x W
    x2 = spikes((T, N, Cs, Hs, Ws), 0.25, g)
    w2 = q(torch.randn(Cout, Cs, 1, 1, generator=g) * (2.0 / Cs) ** 0.5, dtype)
    b2 = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    shortcut = [torch.nn.functional.conv2d(x2[t], w2, b2, stride=ss) for t in range(T)]
    assert tuple(shortcut[0].shape[-2:]) == (H, W)
    ref = O.temporal_conv_lif([xs[t] for t in range(T)], w, b, torch.tensor(0.0), (1, 1), (k // 2, k // 2), (1, 1), 1, *lif, residuals=shortcut)
    out_layout = {"nchw": B.NCHW, "c8": B.C8, "bits": B.BITS}[outl]
    x, xsc = _to_layout(B, xs, "bits", dtype), _to_layout(B, x2, "bits", dtype)
    print(f"blocked conv {Cin}->{Cout} {H}x{W} k{k} + shortcut {Cs}->{Cout} /{ss} from {Hs}x{Ws} T={T} N={N} -> {outl}", flush=True)
    out, v = B.conv_lif_blocked_shortcut(x, dev(w, dtype), dev(b, dtype), [k // 2, k // 2], xsc, dev(w2, dtype), dev(b2, dtype), [ss, ss], lif,
                                         out_layout=out_layout, want_v=True)
    torch.cuda.synchronize()
    plan = B.last_conv_plan()
    assert plan["kernel"] == "blocked" and int(plan["shortcut_stages"]) >= 1, plan
    assert out.layout == out_layout and out.shape == (T, N, Cout, H, W) and v.dtype == F32
    rep = check(B.to_dense(out), v, ref, v_threshold=lif[0], what=f"blocked {Cin}->{Cout} k{k} + shortcut {Cs}/{ss} -> {outl}")
    assert 0.001 < float(ref[0].mean()) < 0.9, float(ref[0].mean())
    assert rep["neurons_with_matching_history"] >= 0.999 * rep["neurons"]
    # the two-launch form: the shortcut's sums pass through the activation dtype on their way, the spikes agree but for neurons at the threshold
    sc_out, _ = B.conv_lif_blocked(xsc, dev(w2, dtype), dev(b2, dtype), [ss, ss], [0, 0], None, out_layout=B.C8)
    two, _ = B.conv_lif_blocked(x, dev(w, dtype), dev(b, dtype), [1, 1], [k // 2, k // 2], lif, residual=sc_out, out_layout=out_layout)
    differ = (B.to_dense(two).float() != B.to_dense(out).float()).float().mean()
    assert float(differ) < 1e-2, float(differ)


def test_blocked_conv_shortcut_rejects_what_it_does_not_take(B):
    T, N = 4, 2
    xs, w, b = _case(3450, T, N, 64, 64, 8, 8, 3, BF16)
    x = B.from_dense(dev(xs, BF16), B.BITS)
    g = gen(3451)
    def sc(C, H, W, t=T):
        return B.from_dense(dev(spikes((t, N, C, H, W), 0.2, g), BF16), B.BITS)
    dw, db = dev(w, BF16), dev(b, BF16)
    w2 = dev(q(torch.randn(64, 32, 1, 1, generator=g), BF16), BF16)
    with pytest.raises(RuntimeError, match="unsupported_shortcut"):        # lands on 7x7, not 8x8
        B.conv_lif_blocked_shortcut(x, dw, db, [1, 1], sc(32, 13, 13), w2, None, [2, 2], LIF)
    with pytest.raises(RuntimeError, match="unsupported_shortcut"):        # 24 channels: not a multiple of 16
        B.conv_lif_blocked_shortcut(x, dw, db, [1, 1], sc(24, 15, 15), dev(q(torch.randn(64, 24, 1, 1, generator=g), BF16), BF16), None, [2, 2], LIF)
    with pytest.raises(RuntimeError, match="unsupported_shortcut"):        # a main convolution that shrinks its plane
        B.conv_lif_blocked_shortcut(x, dw, db, [0, 0], sc(32, 15, 15), w2, None, [2, 2], LIF)
    with pytest.raises(RuntimeError, match="unsupported_shortcut"):        # 3x3 shortcut
        B.conv_lif_blocked_shortcut(x, dw, db, [1, 1], sc(32, 15, 15), dev(q(torch.randn(64, 32, 3, 3, generator=g), BF16), BF16), None, [2, 2], LIF)
    x2 = B.from_dense(dev(xs[:2], BF16), B.BITS)
    with pytest.raises(RuntimeError, match="unsupported_shortcut"):        # two timesteps
        B.conv_lif_blocked_shortcut(x2, dw, db, [1, 1], sc(32, 15, 15, 2), w2, None, [2, 2], LIF)


POOLED_CASES = [  # Cin, Cout, H, W, k, s, p, N, dtype, input: "bits" | "c8" | "frame" (one analog frame for the four steps)
    (64, 128, 16, 16, 3, 1, 1, 4, BF16, "bits"),      # VGG-11's second layer
    (3, 64, 32, 32, 3, 1, 1, 2, BF16, "frame"),       # its first: one frame, four LIF steps
    (256, 256, 8, 8, 3, 1, 1, 4, BF16, "c8"),         # analog blocked input (the layer behind a pool), K shared by waves
    (512, 512, 4, 4, 3, 1, 1, 6, BF16, "c8"),         # 4x4 planes: two images per patch
    (128, 64, 2, 2, 3, 1, 1, 20, BF16, "bits"),       # 2x2 planes: eight images per patch, one window each
    (64, 72, 12, 20, 3, 1, 1, 3, F16, "bits"),        # fp16, 72 channels, a plane that is no multiple of the patch
    (64, 64, 16, 24, 3, 2, 1, 2, BF16, "bits"),       # stride 2 onto an 8x12 plane
    (32, 64, 20, 12, 5, 1, 2, 2, BF16, "bits"),       # 5x5
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p,N,dtype,inl", POOLED_CASES)
def test_blocked_conv_with_its_average_pool_in_the_same_launch(B, Cin, Cout, H, W, k, s, p, N, dtype, inl):
    """conv + LIF + 2x2 average pool in one launch: bit for bit the two launches, and the unpooled neurons' membrane and the
    pooled spikes against the oracle."""
    T = 4
    xs, w, b = _case(3500 + Cin + Cout + H + k, T, N, Cin, Cout, H, W, k, dtype, analog=inl != "bits", shared=inl == "frame")
    frames = [xs[0]] * T if inl == "frame" else [xs[t] for t in range(T)]
    ref = O.temporal_conv_lif(frames, w, b, torch.tensor(0.0), (s, s), (p, p), (1, 1), 1, *LIF)
    if inl == "frame":
        x = B.from_dense(dev(xs[0], dtype), B.C8, shared=True)
        x.T = T
    else:
        x = _to_layout(B, xs, inl, dtype)
    dw, db = dev(w, dtype), dev(b, dtype)
    print(f"blocked conv + pool {Cin}->{Cout} {H}x{W} k{k} N={N} {inl}", flush=True)
    pooled, v = B.conv_lif_blocked_avgpool(x, dw, db, [s, s], [p, p], LIF, want_v=True)
    torch.cuda.synchronize()
    Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    assert pooled.layout == B.C8 and pooled.shape == (T, N, Cout, Ho // 2, Wo // 2)
    plan = B.last_conv_plan()
    spikes_out, v2 = B.conv_lif_blocked(x, dw, db, [s, s], [p, p], LIF, want_v=True)
    plan2 = B.last_conv_plan()
    two = B.pool_blocked(spikes_out, False, 2, 2, 0)
    # the same partition of K over waves and stages (true for these shapes): the same sums, bit for bit
    assert (plan["waves"], plan["stage_chunks"]) == (plan2["waves"], plan2["stage_chunks"]), (plan, plan2)
    assert torch.equal(pooled.data, two.data) and torch.equal(v, v2)
    rep = check(B.to_dense(spikes_out), v, ref, what=f"blocked {Cin}->{Cout} k{k} + pool")
    assert 0.001 < float(ref[0].mean()) < 0.9, float(ref[0].mean())
    got = B.to_dense(pooled).float().cpu()
    want = torch.nn.functional.avg_pool2d(ref[0].flatten(0, 1), 2).reshape(got.shape)
    assert float((got != want).float().mean()) <= 4 * (1.0 - rep["neurons_with_matching_history"] / rep["neurons"]) + 1e-9
    if Cout % 8:
        assert float(pooled.data[:, :, -1, :, :, Cout % 8:].abs().max()) == 0.0


def test_blocked_conv_with_pool_rejects_what_it_does_not_take(B):
    xs, w, b = _case(3550, 4, 2, 64, 64, 17, 17, 3, BF16)
    x = B.from_dense(dev(xs, BF16), B.BITS)
    dw, db = dev(w, BF16), dev(b, BF16)
    with pytest.raises(RuntimeError, match="unsupported_pool"):       # 17 -> 9: odd plane
        B.conv_lif_blocked_avgpool(x, dw, db, [2, 2], [1, 1], LIF)
    xs2, w2, b2 = _case(3551, 4, 2, 64, 64, 8, 8, 3, BF16)
    x2 = B.from_dense(dev(xs2, BF16), B.BITS)
    with pytest.raises(RuntimeError, match="unsupported_pool"):       # tau 3: not the straight-line epilogue
        B.conv_lif_blocked_avgpool(x2, dev(w2, BF16), dev(b2, BF16), [1, 1], [1, 1], (1.0, 0.0, 3.0))
    x3 = B.from_dense(dev(xs2[:3], BF16), B.BITS)
    with pytest.raises(RuntimeError, match="unsupported_pool"):       # three timesteps
        B.conv_lif_blocked_avgpool(x3, dev(w2, BF16), dev(b2, BF16), [1, 1], [1, 1], LIF)


@pytest.mark.parametrize("T,N,C,H,W,K,dtype,scale", [
    (4, 16, 512, 7, 7, 1000, BF16, 0.25),      # ResNet-18's tail
    (4, 64, 512, 1, 1, 10, BF16, 0.25),        # VGG-11's
    (3, 5, 24, 5, 3, 7, F16, 1.0),             # odd everything, the plain sum over T
    (16, 2, 64, 20, 20, 33, BF16, 1.0 / 16),   # 6400 spikes per channel at most: the byte counters are flushed on the way
    (1, 3, 2048, 2, 2, 130, BF16, 1.0),        # the widest layer
])
def test_pool_and_classifier_on_bit_packed_spikes(B, T, N, C, H, W, K, dtype, scale):
    """Exact spike counts, fp32 dot products: the result equals scale * (W . sum_t mean_hw(s_t) + T b) computed in float64,
    to the rounding of the output dtype."""
    g = gen(3600 + C + K)
    s = spikes((T, N, C, H, W), 0.3, g)
    s[:, :, 0] = 1.0                                    # one channel that always fires: the largest count
    w = q(torch.randn(K, C, generator=g) * 0.05, dtype)
    b = q(torch.randn(K, generator=g) * 0.05, dtype)
    x = B.from_dense(dev(s, dtype), B.BITS)
    got = B.spike_pool_linear(x, dev(w, dtype), dev(b, dtype), scale)
    torch.cuda.synchronize()
    counts = s.double().sum((0, 3, 4))                  # [N, C]
    want = scale * (counts @ w.double().t() / (H * W) + T * b.double())
    assert got.shape == (N, K) and got.dtype == dtype
    eps = 2.0 ** -8 if dtype == BF16 else 2.0 ** -11
    assert torch.allclose(got.double().cpu(), want, rtol=eps, atol=1e-4), float((got.double().cpu() - want).abs().max())
    no_bias = B.spike_pool_linear(x, dev(w, dtype), None, scale)
    assert torch.allclose(no_bias.double().cpu(), want - scale * T * b.double(), rtol=eps, atol=1e-4)


def test_blocked_conv_without_membrane_output_and_chained_windows(B):
    """The final membrane is optional; two calls chained through it equal one call of all steps, bit for bit."""
    T, N, C, H = 4, 2, 64, 12
    xs, w, b = _case(3300, T, N, C, C, H, H, 3, BF16)
    x = B.from_dense(dev(xs, BF16), B.BITS)
    dw, db = dev(w, BF16), dev(b, BF16)
    out, v = B.conv_lif_blocked(x, dw, db, [1, 1], [1, 1], LIF, want_v=True)
    out2, v2 = B.conv_lif_blocked(x, dw, db, [1, 1], [1, 1], LIF, want_v=False)
    assert v2 is None and torch.equal(out.data, out2.data)
    xa = B.from_dense(dev(xs[:1], BF16), B.BITS)
    xb = B.from_dense(dev(xs[1:], BF16), B.BITS)
    oa, va = B.conv_lif_blocked(xa, dw, db, [1, 1], [1, 1], LIF, want_v=True)
    ob, vb = B.conv_lif_blocked(xb, dw, db, [1, 1], [1, 1], LIF, v_init=va, want_v=True)
    assert torch.equal(torch.cat([oa.data, ob.data]), out.data) and torch.equal(vb, v)


SHARED_CASES = [  # Cin, Cout, H, W, k, s, p, T, N
    (3, 64, 32, 32, 7, 2, 3, 4, 2),      # ResNet stem: one analog frame, taps paired inside a single channel group
    (3, 64, 32, 32, 3, 1, 1, 4, 3),      # VGG stem at its own size
    (8, 32, 9, 13, 3, 1, 1, 4, 2),       # a whole channel group, ragged plane
    (1, 16, 12, 12, 5, 1, 2, 2, 2),      # one channel
    (3, 64, 16, 16, 3, 1, 1, 16, 2),     # VGG stem, 16 LIF steps on one convolution
    (64, 64, 8, 8, 3, 1, 1, 5, 2),       # whole channel groups
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p,T,N", SHARED_CASES)
def test_blocked_conv_with_one_analog_frame_for_all_timesteps(B, Cin, Cout, H, W, k, s, p, T, N):
    xs, w, b = _case(3400 + Cin + H, T, N, Cin, Cout, H, W, k, BF16, analog=True, shared=True, gain=1.5)
    ref = O.temporal_conv_lif([xs[0]] * T, w, b, torch.tensor(0.0), (s, s), (p, p), (1, 1), 1, *LIF)
    x = B.from_dense(dev(xs[0], BF16), B.C8, shared=True)
    x.T = T
    out, v = B.conv_lif_blocked(x, dev(w, BF16), dev(b, BF16), [s, s], [p, p], LIF, want_v=True)
    plan = B.last_conv_plan()
    assert plan["kernel"] == "blocked" and plan["window"] == T
    check(B.to_dense(out), v, ref, what=f"blocked shared frame {Cin}->{Cout} k{k}")
    assert 0.001 < float(ref[0].mean()) < 0.9
    if Cin <= 8:
        # The frame as it is (dense, no conversion launch): same matrix operands, bit for bit the same result.
        frame = B.input_frame(dev(xs[0], BF16), T)
        assert frame.layout == B.NCHW and frame.shared
        out2, v2 = B.conv_lif_blocked(frame, dev(w, BF16), dev(b, BF16), [s, s], [p, p], LIF, want_v=True)
        assert B.last_conv_plan()["kernel"] == "blocked"
        assert torch.equal(out2.data, out.data) and torch.equal(v2, v)
        if T == 4 and out.H % 2 == 0 and out.W % 2 == 0:
            pooled, _ = B.conv_lif_blocked_avgpool(frame, dev(w, BF16), dev(b, BF16), [s, s], [p, p], LIF)
            assert torch.equal(pooled.data, B.pool_blocked(out, False, 2, 2, 0).data)
    else:
        assert B.input_frame(dev(xs[0], BF16), T).layout == B.C8


def test_blocked_conv_takes_a_dense_input_only_as_one_small_frame(B):
    xs, w, b = _case(3460, 4, 2, 3, 16, 8, 8, 3, BF16, analog=True)
    per_step = B.from_dense(dev(xs, BF16), B.NCHW)                      # a frame per timestep: not the shared input
    with pytest.raises(RuntimeError, match="unsupported_layout"):
        B.conv_lif_blocked(per_step, dev(w, BF16), dev(b, BF16), [1, 1], [1, 1], LIF)
    xs16, w16, b16 = _case(3461, 4, 2, 16, 16, 8, 8, 3, BF16, analog=True, shared=True)
    wide = B.from_dense(dev(xs16[0], BF16), B.NCHW, shared=True)         # 16 channels
    wide.T = 4
    with pytest.raises(RuntimeError, match="unsupported_layout"):
        B.conv_lif_blocked(wide, dev(w16, BF16), dev(b16, BF16), [1, 1], [1, 1], LIF)


CONV_BIAS_CASES = [  # Cin, Cout, H, W, k, s, p, T, N, residual layout, out layout
    (64, 128, 16, 16, 1, 2, 0, 4, 2, None, "c8"),        # downsample shortcut: spikes in, analog blocked out
    (64, 64, 7, 7, 3, 1, 1, 4, 3, "c8", "nchw"),         # pre-tail sum: conv + blocked residual, dense out
    (128, 96, 7, 7, 3, 1, 1, 3, 2, "bits", "c8"),        # spike residual
]


@pytest.mark.parametrize("Cin,Cout,H,W,k,s,p,T,N,resl,outl", CONV_BIAS_CASES)
def test_blocked_conv_without_neuron(B, Cin, Cout, H, W, k, s, p, T, N, resl, outl):
    """No neuron: conv + bias (+ residual) in fp32 from bf16 operands, one rounding to bf16 at the store."""
    xs, w, b = _case(3500 + Cin + Cout, T, N, Cin, Cout, H, W, k, BF16)
    Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    g = gen(3501)
    rs = None if resl is None else (spikes((T, N, Cout, Ho, Wo), 0.3, g) if resl == "bits" else q(torch.randn(T, N, Cout, Ho, Wo, generator=g), BF16))
    want = torch.stack([torch.nn.functional.conv2d(xs[t], w, b, s, p) for t in range(T)])
    if rs is not None:
        want = want + rs
    out, v = B.conv_lif_blocked(B.from_dense(dev(xs, BF16), B.BITS), dev(w, BF16), dev(b, BF16), [s, s], [p, p], None,
                                residual=None if rs is None else _to_layout(B, rs, resl, BF16),
                                out_layout={"nchw": B.NCHW, "c8": B.C8}[outl])
    assert v is None
    got = B.to_dense(out).float().cpu()
    assert torch.allclose(got, want, rtol=2 ** -8, atol=1e-3), (got - want).abs().max()


@pytest.mark.parametrize("patch_cols,stage_groups,k_waves,tile,waves,chunks", [
    (16, 2, 2, "1x2x16", "8x1x2", 2), (4, 4, 1, "1x8x4", "8x1x1", 4), (2, 0, 4, "1x16x2", "8x1x4", 4),
    (16, 8, 8, "1x2x16", None, None)])      # 8 groups / 8 waves do not fit this layer: the patch is applied, the rest is the planner's
def test_registered_launch_choices_are_applied_and_keep_parity(B, patch_cols, stage_groups, k_waves, tile, waves, chunks):
    Cin, Cout, H, W, k, T, N = 128, 64, 16, 16, 3, 4, 2
    xs, w, b = _case(3300, T, N, Cin, Cout, H, W, k, BF16)
    lif = (1.0, 0.0, 2.0)
    ref = O.temporal_conv_lif([xs[t] for t in range(T)], w, b, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), 1, *lif)
    x = _to_layout(B, xs, "bits", BF16)
    key = B._plan_key(T, N, Cin, H, W, Cout, k, k, 1, 1, 1, 1, False)
    assert B.get_autotune_best_config(T, N, Cin, H, W, (Cout, Cin, k, k), [1, 1], [1, 1]) == {}      # not a tuned layer
    B.register_tuned_plan(key, patch_cols, stage_groups, k_waves)
    try:
        out, v = B.conv_lif_blocked(x, dev(w, BF16), dev(b, BF16), [1, 1], [1, 1], lif, out_layout=B.BITS, want_v=True)
        torch.cuda.synchronize()
        plan = B.last_conv_plan()
    finally:
        B.register_tuned_plan(key, 0, 0, 0)
    assert plan["tile"] == tile and plan["tuned"] & 1
    if waves is not None:
        assert plan["waves"] == waves and plan["stage_chunks"] == chunks and plan["tuned"] == 3
    check(B.to_dense(out), v, ref, what=f"tuned plan {patch_cols}/{stage_groups}/{k_waves}")
    B.conv_lif_blocked(x, dev(w, BF16), dev(b, BF16), [1, 1], [1, 1], lif, out_layout=B.BITS)
    assert B.last_conv_plan()["tuned"] == 0


def test_the_committed_table_is_registered_and_reported(B):
    table = B.load_tuned_plans()
    for key, entry in table.items():
        got = B.get_autotune_best_config(entry["T"], entry["N"], entry["Cin"], entry["H"], entry["W"],
                                         (entry["Cout"], entry["Cin"], *entry["kernel"]), entry["stride"], entry["padding"], entry["shared_frame"])
        assert got["patch_cols"] == entry["patch_cols"] and got["us"] <= got["planner_us"]


def test_blocked_conv_rejects_what_it_does_not_take(B):
    x = B.from_dense(torch.zeros(4, 2, 64, 8, 8, device=DEV, dtype=BF16), B.BITS)
    w = torch.zeros(64, 64, 3, 3, device=DEV, dtype=BF16)
    with pytest.raises(RuntimeError, match="unsupported_layout"):
        B.conv_lif_blocked(x, w, None, [1, 1], [1, 1], None, out_layout=B.BITS)          # bits without a neuron
    with pytest.raises(RuntimeError, match="unsupported_layout"):
        B.conv_lif_blocked(B.from_dense(torch.zeros(4, 2, 64, 8, 8, device=DEV, dtype=BF16), B.NCHW), w, None, [1, 1], [1, 1], LIF)
    with pytest.raises(RuntimeError, match="unsupported_groups"):
        B.conv_lif_blocked(x, torch.zeros(64, 1, 3, 3, device=DEV, dtype=BF16), None, [1, 1], [1, 1], LIF)
    with pytest.raises(RuntimeError, match="unsupported_padding"):
        B.conv_lif_blocked(x, w, None, [1, 1], [2, 2], LIF)


# ---------------------------------------------------------------------------------------------------------------
# Depthwise 3x3 + LIF with row-packed spikes (one byte = 8 consecutive pixels of a row)
# ---------------------------------------------------------------------------------------------------------------
def _ref_rowbits(s):
    """Dense 0/1 [..., W] -> [..., W / 8] uint8, bit j = pixel 8 x + j."""
    shape = tuple(s.shape[:-1]) + (s.shape[-1] // 8, 8)
    weights = 2 ** torch.arange(8, dtype=torch.int32)
    return ((s != 0).to(torch.int32).reshape(shape) * weights).sum(-1).to(torch.uint8)


ROWBITS_CASES = [  # dtype, N, C, H, W, T, lif, residual, tensor v_init, want_v
    (BF16, 2, 16, 28, 56, 4, (1.0, 0.0, 2.0), False, False, True),     # several planes per workgroup
    (BF16, 1, 8, 56, 56, 4, (1.0, 0.0, 2.0), False, False, False),     # the headline plane, no membrane output
    (F16, 2, 5, 9, 16, 3, (1.0, -1.0, 2.0), True, True, True),         # soft reset (general neuron), residual, v_init
    (BF16, 3, 7, 8, 8, 17, (0.5, 0.0, 1.0), False, True, True),        # two launch windows (16 + 1), IF neuron
    (F16, 1, 3, 96, 160, 2, (1.0, 0.0, 3.0), True, False, True),       # planes cut into row bands, tau not a power of two
    (BF16, 2, 4, 7, 24, 1, (1.0, 0.0, 2.0), False, False, True),       # a single step
]


@pytest.mark.parametrize("dtype,N,C,H,W,T,lif,residual,tensor_v,want_v", ROWBITS_CASES)
def test_depthwise_with_row_packed_spikes_against_the_oracle(B, dtype, N, C, H, W, T, lif, residual, tensor_v, want_v):
    g = gen(4100 + C + H + T)
    xs = [spikes((N, C, H, W), 0.3, g) for _ in range(T)]
    w = q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, dtype)
    b = q(torch.randn(C, generator=g) * 0.1, dtype)
    rs = [q(torch.randn(N, C, H, W, generator=g) * 0.3, dtype) for _ in range(T)] if residual else None
    v0 = torch.randn(N, C, H, W, generator=g) * 0.3 if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (1, 1), (1, 1), C, *lif, residuals=rs)
    dx = [dev(x, dtype) for x in xs]
    dr = [dev(r, dtype) for r in rs] if residual else None
    bits, v = B.depthwise_conv_lif_rowbits(dx, dev(w, dtype), dev(b, dtype), lif, residuals=dr,
                                           v_init=dev(v0, F32) if tensor_v else None, want_v=want_v)
    assert bits.dtype == torch.uint8 and tuple(bits.shape) == (T, N, C, H, W // 8)
    assert (v is None) == (not want_v)
    dense = B.unpack_rowbits(bits, dtype)
    assert tuple(dense.shape) == (T, N, C, H, W) and dense.dtype == dtype
    assert torch.equal(_ref_rowbits(dense.float().cpu()), bits.cpu())                 # the unpacker is exact
    v_chk = v if want_v else dev(ref[1], F32)                                          # no membrane output: spikes only
    check(dense, v_chk, ref, v_threshold=lif[0], what=f"depthwise row bits {C}x{H}x{W} T={T}")
    # bit for bit the dense operator's spikes and membrane (same kernel, another store)
    import triton_snn_fusion_amd.runtime.snn_custom_ops as ops
    ops.configure_fused_op("hip", strict_triton=True)
    S = torch.ops.snn_custom
    dv = dev(v0, F32) if tensor_v else torch.zeros((), device=DEV, dtype=F32)
    if residual:
        s_d, v_d = S.fused_temporal_conv_add_lif_state_depthwise(dx, dr, dev(w, dtype), dev(b, dtype), dv, [1, 1], [1, 1], [1, 1], C, *lif, False)
    else:
        s_d, v_d = S.fused_temporal_depthwise_conv_lif_state(dx, dev(w, dtype), dev(b, dtype), dv, [1, 1], [1, 1], [1, 1], C, *lif, False)
    assert torch.equal(s_d, dense)
    if want_v:
        assert torch.equal(v_d, v)
    # row-packed spikes in as well: the same bytes and membrane
    packed_in = dev(_ref_rowbits(torch.stack(xs)), torch.uint8)
    bits2, v2 = B.depthwise_conv_lif_rowbits(packed_in, dev(w, dtype), dev(b, dtype), lif, residuals=dr,
                                             v_init=dev(v0, F32) if tensor_v else None, want_v=want_v)
    assert torch.equal(bits2, bits) and (not want_v or torch.equal(v2, v))


def test_depthwise_row_packed_spikes_reject_what_they_do_not_take(B):
    g = gen(4200)
    w, b = dev(torch.randn(4, 1, 3, 3, generator=g), BF16), dev(torch.randn(4, generator=g), BF16)
    with pytest.raises(RuntimeError, match="unsupported_shape"):
        B.depthwise_conv_lif_rowbits([dev(spikes((1, 4, 8, 12), 0.3, g), BF16)], w, b, LIF)
    with pytest.raises(RuntimeError, match="unsupported_dtype"):
        B.depthwise_conv_lif_rowbits([dev(spikes((1, 4, 8, 16), 0.3, g), F32)], w.float(), b.float(), LIF)


# ---------------------------------------------------------------------------------------------------------------
# Pointwise conv + LIF reading row-packed spikes (the consumer of the depthwise layer above)
# ---------------------------------------------------------------------------------------------------------------
PW_ROWBITS_CASES = [  # dtype, N, Cin, Cout, H, W, T, tau, tensor v_init
    (BF16, 2, 128, 256, 8, 16, 4, 2.0, False),     # weights in registers, two output-channel tiles
    (BF16, 3, 64, 96, 8, 8, 3, 4.0, True),         # weights in LDS, one chunk; Cout % 128 != 0
    (F16, 2, 256, 64, 16, 8, 4, 2.0, True),        # several chunks, f16
    (BF16, 1, 24, 32, 8, 24, 2, 2.0, False),       # channel tail inside a chunk
    (BF16, 2, 1024, 64, 8, 8, 2, 2.0, False),      # weights streamed from L2
    (F16, 1, 128, 128, 16, 16, 17, 2.0, True),     # two launch windows
]


@pytest.mark.parametrize("dtype,N,Cin,Cout,H,W,T,tau,tensor_v", PW_ROWBITS_CASES)
def test_pointwise_from_row_packed_spikes_against_the_oracle(B, dtype, N, Cin, Cout, H, W, T, tau, tensor_v):
    g = gen(4300 + Cin + Cout + T)
    lif = (1.0, 0.0, tau)
    xs = [spikes((N, Cin, H, W), 0.25, g) for _ in range(T)]
    w = q(torch.randn(Cout, Cin, 1, 1, generator=g) * (2.0 / Cin) ** 0.5 * 2.0, dtype)
    b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    v0 = torch.randn(N, Cout, H, W, generator=g) * 0.3 if tensor_v else torch.tensor(0.0)
    ref = O.temporal_conv_lif(xs, w, b, v0, (1, 1), (0, 0), (1, 1), 1, *lif)
    bits = dev(_ref_rowbits(torch.stack(xs)), torch.uint8)
    sp, v = B.pointwise_conv_lif_from_rowbits(bits, dev(w, dtype), dev(b, dtype), lif, v_init=dev(v0, F32) if tensor_v else None)
    assert sp.dtype == dtype and tuple(sp.shape) == (T, N, Cout, H, W) and v.dtype == F32
    check(sp, v, ref, what=f"pointwise from row bits {Cin}->{Cout} {H}x{W} T={T}")
    # bit for bit the dense operator on the unpacked spikes (same kernel, another fetch)
    import triton_snn_fusion_amd.runtime.snn_custom_ops as ops
    ops.configure_fused_op("hip", strict_triton=True)
    dv = dev(v0, F32) if tensor_v else torch.zeros((), device=DEV, dtype=F32)
    s_d, v_d = torch.ops.snn_custom.fused_temporal_pointwise_conv_lif_state([dev(x, dtype) for x in xs], dev(w, dtype), dev(b, dtype), dv,
                                                                            [1, 1], [0, 0], [1, 1], 1, *lif, False)
    from triton_snn_fusion_amd.runtime.hip_convlif_backend import last_conv_plan
    if last_conv_plan()["kernel"] == "pointwise":       # small deep layers run the matrix kernel through the operator
        assert torch.equal(s_d, sp) and torch.equal(v_d, v)
    # row-packed spikes out as well: the same spikes and membrane, bit for bit; the membrane is optional within one window
    pb, pv = B.pointwise_conv_lif_from_rowbits(bits, dev(w, dtype), dev(b, dtype), lif, v_init=dev(v0, F32) if tensor_v else None,
                                               packed_out=True)
    assert pb.dtype == torch.uint8 and tuple(pb.shape) == (T, N, Cout, H, W // 8)
    assert torch.equal(B.unpack_rowbits(pb, dtype), sp) and torch.equal(pv, v)
    if T <= 16:
        pb2, none = B.pointwise_conv_lif_from_rowbits(bits, dev(w, dtype), dev(b, dtype), lif, v_init=dev(v0, F32) if tensor_v else None,
                                                      packed_out=True, want_v=False)
        assert none is None and torch.equal(pb2, pb)


def test_depthwise_then_pointwise_through_row_packed_spikes(B):
    """A depthwise-separable block whose intermediate spikes travel one bit each == the two dense operators."""
    dtype, T, N, C, Cout, H, W = BF16, 4, 2, 128, 256, 16, 16
    g = gen(4400)
    xs = [spikes((N, C, H, W), 0.3, g) for _ in range(T)]
    wd, bd = q(torch.randn(C, 1, 3, 3, generator=g) * 0.5, dtype), q(torch.randn(C, generator=g) * 0.1, dtype)
    wp, bp = q(torch.randn(Cout, C, 1, 1, generator=g) * (2.0 / C) ** 0.5 * 2.0, dtype), q(torch.randn(Cout, generator=g) * 0.1, dtype)
    ref_d = O.temporal_conv_lif(xs, wd, bd, torch.tensor(0.0), (1, 1), (1, 1), (1, 1), C, *LIF)
    ref_p = O.temporal_conv_lif([ref_d[0][t] for t in range(T)], wp, bp, torch.tensor(0.0), (1, 1), (0, 0), (1, 1), 1, *LIF)
    bits, _ = B.depthwise_conv_lif_rowbits([dev(x, dtype) for x in xs], dev(wd, dtype), dev(bd, dtype), LIF, want_v=False)
    sp, v = B.pointwise_conv_lif_from_rowbits(bits, dev(wp, dtype), dev(bp, dtype), LIF)
    packed, _ = B.pointwise_conv_lif_from_rowbits(bits, dev(wp, dtype), dev(bp, dtype), LIF, packed_out=True, want_v=False)
    assert torch.equal(B.unpack_rowbits(packed, dtype), sp)      # bits in, bits out, no membrane: the same spikes
    # Teacher forcing as for the network tests: the pointwise layer is gated on the oracle's depthwise spikes only where the
    # library's depthwise spikes equal them (they do, away from the threshold band the depthwise gate allows).
    dense = B.unpack_rowbits(bits, dtype)
    if torch.equal(dense.float().cpu(), ref_d[0]):
        check(sp, v, ref_p, what="depthwise -> pointwise through row bits")
    ref_own = O.temporal_conv_lif([dense[t].float().cpu() for t in range(T)], wp, bp, torch.tensor(0.0), (1, 1), (0, 0), (1, 1), 1, *LIF)
    check(sp, v, ref_own, what="pointwise on the library's own depthwise spikes")


def test_pointwise_from_row_packed_spikes_rejects_what_it_does_not_take(B):
    g = gen(4500)
    w, b = dev(torch.randn(32, 16, 1, 1, generator=g), BF16), dev(torch.randn(32, generator=g), BF16)
    bits = torch.zeros(2, 1, 16, 4, 1, dtype=torch.uint8, device=DEV)            # 4 x 8 = 32 pixels: not whole tiles of 64
    with pytest.raises(RuntimeError, match="unsupported_shape"):
        B.pointwise_conv_lif_from_rowbits(bits, w, b, LIF)
    bits = torch.zeros(2, 1, 16, 8, 1, dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="unsupported_shape"):
        B.pointwise_conv_lif_from_rowbits(bits, w, b, (1.0, -1.0, 2.0))            # soft reset: not the common neuron


def test_two_blocks_chained_on_row_packed_spikes(B):
    """pointwise (bits out) -> depthwise (bits in, bits out) -> pointwise (bits in): the same spikes as the dense operators."""
    import triton_snn_fusion_amd.runtime.snn_custom_ops as ops
    ops.configure_fused_op("hip", strict_triton=True)
    S = torch.ops.snn_custom
    dtype, T, N, C0, C1, C2, H, W = BF16, 4, 2, 64, 128, 64, 16, 16
    g = gen(4600)
    xs = [spikes((N, C0, H, W), 0.3, g) for _ in range(T)]
    w1, b1 = dev(q(torch.randn(C1, C0, 1, 1, generator=g) * (2.0 / C0) ** 0.5 * 2.0, dtype), dtype), dev(q(torch.randn(C1, generator=g) * 0.1, dtype), dtype)
    wd, bd = dev(q(torch.randn(C1, 1, 3, 3, generator=g) * 0.5, dtype), dtype), dev(q(torch.randn(C1, generator=g) * 0.1, dtype), dtype)
    w2, b2 = dev(q(torch.randn(C2, C1, 1, 1, generator=g) * (2.0 / C1) ** 0.5 * 2.0, dtype), dtype), dev(q(torch.randn(C2, generator=g) * 0.1, dtype), dtype)
    zero = torch.zeros((), device=DEV, dtype=F32)
    dx = [dev(x, dtype) for x in xs]
    s1, _ = S.fused_temporal_pointwise_conv_lif_state(dx, w1, b1, zero, [1, 1], [0, 0], [1, 1], 1, *LIF, False)
    s2, _ = S.fused_temporal_depthwise_conv_lif_state(list(s1.unbind(0)), wd, bd, zero, [1, 1], [1, 1], [1, 1], C1, *LIF, False)
    s3, v3 = S.fused_temporal_pointwise_conv_lif_state(list(s2.unbind(0)), w2, b2, zero, [1, 1], [0, 0], [1, 1], 1, *LIF, False)
    p0 = B.pack_rowbits(torch.stack(dx))
    assert torch.equal(p0.cpu(), _ref_rowbits(torch.stack(xs))) and torch.equal(B.unpack_rowbits(p0, dtype), torch.stack(dx))
    p1, _ = B.pointwise_conv_lif_from_rowbits(p0, w1, b1, LIF, packed_out=True, want_v=False)
    p2, _ = B.depthwise_conv_lif_rowbits(p1, wd, bd, LIF, want_v=False)
    p3, pv3 = B.pointwise_conv_lif_from_rowbits(p2, w2, b2, LIF, packed_out=True, want_v=True)
    assert torch.equal(B.unpack_rowbits(p1, dtype), s1)
    assert torch.equal(B.unpack_rowbits(p2, dtype), s2)
    assert torch.equal(B.unpack_rowbits(p3, dtype), s3) and torch.equal(pv3, v3)


# ---------------------------------------------------------------------------------------------------------------
# Convolutions on planes of a few pixels run as one matrix product per frame on the Linear + LIF kernel
# (snnf_linear_lif_bits: activation rows as C8 elements or as bits, spikes out as bits)
# ---------------------------------------------------------------------------------------------------------------
PLANE_CASES = [  # T, N, Cin, Cout, H, W, k, dtype
    (4, 64, 128, 128, 2, 2, 3, BF16), (4, 7, 64, 72, 2, 2, 3, F16), (6, 20, 32, 64, 1, 1, 3, BF16), (3, 5, 16, 16, 2, 1, 3, BF16),
    (8, 33, 256, 128, 1, 2, 1, F16), (5, 9, 24, 40, 2, 2, 5, BF16), (4, 1, 512, 512, 2, 2, 3, BF16), (4, 16, 1024, 256, 2, 2, 3, BF16),
]


@pytest.mark.parametrize("source", ["bits", "quarters"])
@pytest.mark.parametrize("T,N,Cin,Cout,H,W,k,dtype", PLANE_CASES)
def test_small_plane_convolutions_as_matrix_products(B, T, N, Cin, Cout, H, W, k, dtype, source):
    import torch.nn.functional as F
    g = gen(9100 + Cin + Cout + T + N)
    if source == "bits":
        x = spikes((T, N, Cin, H, W), 0.2, g)
        bx = B.from_dense(dev(x, dtype), B.BITS)
    else:       # what an average pool in front of the layer leaves: quarters, channel-blocked
        x = F.avg_pool2d(spikes((T * N, Cin, 2 * H, 2 * W), 0.3, g), 2).reshape(T, N, Cin, H, W)
        bx = B.from_dense(dev(x, dtype), B.C8)
    w = q(torch.randn(Cout, Cin, k, k, generator=g) * (2.0 / (Cin * min(k * k, H * W))) ** 0.5 * 2.5, dtype)
    b = q(torch.randn(Cout, generator=g) * 0.1, dtype)
    ref = O.temporal_conv_lif([x[t] for t in range(T)], w, b, torch.tensor(0.0), (1, 1), (k // 2, k // 2), (1, 1), 1, *LIF)
    dw, db = dev(w, dtype), dev(b, dtype)
    out, v = B.conv_lif_blocked(bx, dw, db, 1, k // 2, LIF, out_layout=B.BITS)
    plan = B.last_conv_plan()
    assert v is None and plan["kernel"] == "plane_matrix" and plan["x"] == ("bits" if source == "bits" else "c8"), plan
    assert out.layout == B.BITS and out.shape == (T, N, Cout, H, W)
    rep = check(B.to_dense(out), ref[1], ref, what=f"plane matrix {Cin}->{Cout} {H}x{W} k{k} {source}")      # spikes only
    assert 0.001 < float(ref[0].mean()) < 0.9
    assert rep["neurons_with_matching_history"] >= 0.999 * rep["neurons"], rep
    # the same layer with a membrane output stays on the convolution kernel and agrees up to flips at the threshold
    out_c, v_c = B.conv_lif_blocked(bx, dw, db, 1, k // 2, LIF, out_layout=B.BITS, want_v=True)
    assert B.last_conv_plan()["kernel"] != "plane_matrix"
    check(B.to_dense(out_c), v_c, ref, what="the same layer on the convolution kernel")
    assert (B.to_dense(out_c) != B.to_dense(out)).float().mean().item() < 2e-3
    # a second call finds the expanded matrix in the cache and writes the same bits
    out_again, _ = B.conv_lif_blocked(bx, dw, db, 1, k // 2, LIF, out_layout=B.BITS)
    assert torch.equal(out_again.data, out.data)


def test_linear_lif_on_bits_through_the_c_abi(snnf_lib):
    """snnf_linear_lif_bits against the oracle's Linear + LIF: rows of elements and rows of bits, an initial membrane, the
    final membrane, ragged rows, a K long enough for the split over workgroups; and what it refuses."""
    from triton_snn_fusion_amd import _lib
    for seed, (T, M, Fin, Fout, x_bits, dtype, tensor_v) in enumerate([(4, 40, 264, 96, 1, BF16, True), (8, 5, 4096, 64, 0, F16, False),
                                                                        (3, 64, 2048, 2048, 1, BF16, False), (5, 16, 4104, 32, 1, BF16, True)]):
        g = gen(9200 + seed)
        x = spikes((T, M, Fin), 0.2, g) if x_bits else q(torch.rand(T, M, Fin, generator=g) * spikes((T, M, Fin), 0.3, g), dtype)
        w = q(torch.randn(Fout, Fin, generator=g) * (3.0 / Fin ** 0.5), dtype)
        b = q(torch.randn(Fout, generator=g) * 0.1, dtype)
        v0 = torch.rand(M, Fout, generator=g) * 0.8 if tensor_v else None
        ref = O.temporal_linear_lif(x, w, b, v0 if tensor_v else torch.tensor(0.0), *LIF)
        if x_bits:
            weights = (2 ** torch.arange(8, dtype=torch.int32))
            dx = (x.reshape(T, M, Fin // 8, 8).to(torch.int32) * weights).sum(-1).to(torch.uint8).to(DEV)
            stride = Fin // 8
        else:
            dx = x.to(DEV, dtype)
            stride = Fin
        dw, db = w.to(DEV, dtype), b.to(DEV, dtype)
        dv0 = v0.to(DEV) if tensor_v else None
        bits = torch.full((T, M, Fout // 8), 0xA5, dtype=torch.uint8, device=DEV)
        v = torch.full((M, Fout), 7.0, device=DEV)
        need = int(snnf_lib.snnf_linear_lif_workspace_bytes(T, M, Fin, Fout))
        ws = torch.zeros(need, dtype=torch.uint8, device=DEV) if need else None
        print(f"linear on bits: T={T} M={M} {Fin}->{Fout} x_bits={x_bits} {dtype} workspace {need}", flush=True)
        rc = snnf_lib.snnf_linear_lif_bits(_lib.packed_step_pointers(dx), x_bits, T, M, Fin, stride, _lib.dtype_code(dtype), dw.data_ptr(),
                                           db.data_ptr(), Fout, _lib.ptr(dv0), bits.data_ptr(), M * (Fout // 8), v.data_ptr(), *LIF,
                                           _lib.ptr(ws), need, _lib.current_stream(dx.device))
        assert rc == 0, snnf_lib.snnf_last_error()
        torch.cuda.synchronize()
        got = ((bits.cpu().to(torch.int32).unsqueeze(-1) >> torch.arange(8, dtype=torch.int32)) & 1).reshape(T, M, Fout).float()
        check(got, v, ref, what=f"linear on bits {Fin}->{Fout}")
        assert 0.001 < float(ref[0].mean()) < 0.9
        if ws is not None:
            assert int(ws[: 64 * 1024].view(torch.int32).abs().sum()) == 0
    x = torch.zeros(4, 8, 64, dtype=BF16, device=DEV)
    w = torch.zeros(32, 64, dtype=BF16, device=DEV)
    out = torch.zeros(4, 8, 4, dtype=torch.uint8, device=DEV)
    def call(T=4, Fin=64, Fout=32, stride=64, dtype=BF16, step=32):
        return snnf_lib.snnf_linear_lif_bits(_lib.packed_step_pointers(x), 0, T, 8, Fin, stride, _lib.dtype_code(dtype), w.data_ptr(), None, Fout,
                                             None, out.data_ptr(), step, None, *LIF, None, 0, _lib.current_stream(x.device))
    assert call() == 0
    for bad, reason in ((dict(T=2), b"unsupported_window"), (dict(Fout=24), b"unsupported_shape"), (dict(Fin=60), b"unsupported_shape"),
                        (dict(dtype=F32), b"unsupported_dtype"), (dict(stride=60), b"x_row_stride"), (dict(step=16), b"spike_step_stride")):
        assert call(**bad) != 0 and reason in snnf_lib.snnf_last_error(), (bad, snnf_lib.snnf_last_error())
    torch.cuda.synchronize()
