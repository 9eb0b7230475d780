"""snnf_linear_lif_ws: Linear + LIF with the K dimension of a tile split over workgroups (partial sums in a caller-owned
workspace, added in K order by whichever workgroup finishes last). Through the raw C ABI: against the CPU oracle, against
snnf_linear_lif (same sums in a different order: equal up to fp32 rounding of the membrane, equal spikes away from the
threshold), bit-identical from run to run, counters left at zero, a window chain equal to one long call."""
import pytest
import torch

from helpers import DEV, LIF, check, gen, q
from oracle import snn_oracle as O

pytestmark = pytest.mark.gpu

BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32

# (T, M, Fin, Fout, dtype, membrane dtype, tensor v_init)
SPLIT_CASES = [
    (4, 16, 4096, 4096, BF16, F32, True),       # reference micro-benchmark shapes: few row tiles, long K
    (4, 1, 25088, 4096, BF16, F32, False),
    (4, 4, 4096, 1000, F16, F16, True),         # Fout % 32 != 0: narrow tiles
    (8, 40, 4096, 48, BF16, BF16, True),        # ragged rows, 8 timesteps
    (16, 5, 4224, 16, F32, F32, False),         # one feature tile, 16 timesteps, fp32 storage, K not a multiple of the slab
    (3, 33, 4104, 80, F16, F32, True),          # T padded to 4, K % 128 = 8
]


def _inputs(T, M, Fin, Fout, dtype, vdtype, tensor_v, seed):
    g = gen(seed)
    op = dtype                                     # fp32 operands stay fp32 (two bf16 terms each on the matrix cores)
    x = q((torch.rand(T, M, Fin, generator=g) < 0.3).float() * (0.5 + torch.rand(T, M, Fin, generator=g)), op)
    w = q(torch.randn(Fout, Fin, generator=g) * (3.0 / Fin ** 0.5), op)
    b = q(torch.randn(Fout, generator=g) * 0.1, dtype)
    v0 = q(torch.rand(M, Fout, generator=g) * 0.8, vdtype) if tensor_v else None
    return x, w, b, v0


def _call(lib, _lib, x, w, b, v0, vdtype, workspace):
    T, M, Fin = x.shape
    Fout = w.shape[0]
    spikes = torch.full((T, M, Fout), 7.0, device=DEV, dtype=x.dtype)
    v = torch.full((M, Fout), 7.0, device=DEV, dtype=vdtype)
    args = (_lib.packed_step_pointers(x), T, M, Fin, Fin, _lib.dtype_code(x.dtype), w.data_ptr(), b.data_ptr(), Fout,
            _lib.dtype_code(w.dtype), _lib.ptr(v0), _lib.dtype_code(vdtype), spikes.data_ptr(), M * Fout, v.data_ptr(),
            LIF[0], LIF[1], LIF[2])
    stream = _lib.current_stream(x.device)
    if workspace is None:
        rc = lib.snnf_linear_lif(*args, stream)
    else:
        rc = lib.snnf_linear_lif_ws(*args, workspace.data_ptr(), workspace.numel(), stream)
    assert rc == 0, lib.snnf_last_error()
    torch.cuda.synchronize()
    return spikes, v


@pytest.mark.parametrize("T,M,Fin,Fout,dtype,vdtype,tensor_v", SPLIT_CASES)
def test_split_k_linear_lif_matches_the_oracle_and_the_unsplit_kernel(snnf_lib, T, M, Fin, Fout, dtype, vdtype, tensor_v):
    from triton_snn_fusion_amd import _lib
    x, w, b, v0 = _inputs(T, M, Fin, Fout, dtype, vdtype, tensor_v, 7000 + T + M + Fin + Fout)
    need = int(snnf_lib.snnf_linear_lif_workspace_bytes(T, M, Fin, Fout))
    assert need > 64 * 1024, "these shapes are chosen to split"
    print(f"split linear: T={T} M={M} {Fin}->{Fout} {dtype} workspace {need}", flush=True)
    ref = O.temporal_linear_lif(x, w, b, v0.float() if tensor_v else torch.tensor(0.0), *LIF)
    dx, dw, db = x.to(DEV, dtype), w.to(DEV, dtype), b.to(DEV, dtype)
    dv = v0.to(DEV, vdtype) if tensor_v else None
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    s_split, v_split = _call(snnf_lib, _lib, dx, dw, db, dv, vdtype, ws)
    check(s_split, v_split, ref, v_dtype=vdtype, what=f"split linear {Fin}->{Fout}")
    assert 0.001 < float(ref[0].mean()) < 0.9
    assert int(ws[: 64 * 1024].view(torch.int32).abs().sum()) == 0, "the tile counters are zero again after the call"
    # Same bits on a second call with the same (now dirty) workspace: the order of the additions is fixed.
    s_again, v_again = _call(snnf_lib, _lib, dx, dw, db, dv, vdtype, ws)
    assert torch.equal(s_again, s_split) and torch.equal(v_again, v_split)
    # The unsplit kernel adds the same products in another order.
    s_one, v_one = _call(snnf_lib, _lib, dx, dw, db, dv, vdtype, None)
    differ = (s_one != s_split).float().mean().item()
    assert differ < 2e-3, differ
    agree = (s_one == s_split).all(dim=0)
    tol = 1e-5 if vdtype == F32 else 2 ** -7
    assert torch.allclose(v_one.float()[agree], v_split.float()[agree], rtol=tol, atol=tol)
    # A workspace too small for the split: the call runs unsplit and still computes the same thing.
    small = torch.zeros(64 * 1024 + (need - 64 * 1024) // 3, dtype=torch.uint8, device=DEV)
    s_small, v_small = _call(snnf_lib, _lib, dx, dw, db, dv, vdtype, small)
    check(s_small, v_small, ref, v_dtype=vdtype, what=f"split linear, small workspace {Fin}->{Fout}")


def test_layers_whose_tiles_fill_the_chip_do_not_split(snnf_lib):
    assert int(snnf_lib.snnf_linear_lif_workspace_bytes(4, 128, 4096, 1024)) == 0      # 256 wide tiles
    assert int(snnf_lib.snnf_linear_lif_workspace_bytes(8, 64, 2048, 1024)) == 0       # K too short for the split to pay
    assert int(snnf_lib.snnf_linear_lif_workspace_bytes(2, 16, 4096, 4096)) == 0       # one or two timesteps: the kernel without staging


def test_split_k_windows_chain_like_one_long_call(hip_ops):
    """Two calls of 16 timesteps, the second starting from the first one's membrane, equal one call of 32 timesteps (which
    the library runs as two windows of 16) bit for bit; all of them split, the operator API allocates the workspace."""
    S = torch.ops.snn_custom
    T, M, Fin, Fout = 32, 24, 4096, 256
    x, w, b, _ = _inputs(T, M, Fin, Fout, BF16, F32, False, 7100)
    dx, dw, db = x.to(DEV, BF16), w.to(DEV, BF16), b.to(DEV, BF16)
    zero = torch.zeros(M, Fout, device=DEV)
    s_long, v_long = S.fused_temporal_linear_lif_state_packed(dx, dw, db, zero, *LIF, False)
    s_a, v_a = S.fused_temporal_linear_lif_state_packed(dx[:16], dw, db, zero, *LIF, False)
    s_b, v_b = S.fused_temporal_linear_lif_state_packed(dx[16:], dw, db, v_a, *LIF, False)
    assert torch.equal(torch.cat([s_a, s_b]), s_long) and torch.equal(v_b, v_long)
    ref = O.temporal_linear_lif(x, w, b, torch.tensor(0.0), *LIF)
    check(s_long, v_long, ref, what="split linear, 32 timesteps")
    assert hip_ops.get_fused_op_call_stats()["fallback"] == 0


def test_workspace_must_be_aligned(snnf_lib):
    from triton_snn_fusion_amd import _lib
    x, w, b, _ = _inputs(4, 16, 256, 32, BF16, F32, False, 7200)
    dx, dw, db = x.to(DEV, BF16), w.to(DEV, BF16), b.to(DEV, BF16)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    spikes = torch.empty(4, 16, 32, device=DEV, dtype=BF16)
    v = torch.empty(16, 32, device=DEV)
    rc = snnf_lib.snnf_linear_lif_ws(_lib.packed_step_pointers(dx), 4, 16, 256, 256, _lib.dtype_code(BF16), dw.data_ptr(), db.data_ptr(), 32,
                                     _lib.dtype_code(BF16), None, _lib.dtype_code(F32), spikes.data_ptr(), 16 * 32, v.data_ptr(), 1.0, 0.0, 2.0,
                                     ws.data_ptr() + 16, 1 << 19, _lib.current_stream(dx.device))
    assert rc != 0 and b"256-byte aligned" in snnf_lib.snnf_last_error()
