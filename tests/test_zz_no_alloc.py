"""snnf_lif_pool_linear_static: the tail operator without a workspace and without allocation, through the raw C ABI,
against snnf_lif_pool_linear (caller's workspace) on the same operands: identical bits, on two calls in a row, the second
with a smaller input (the static scratch then still holds the first call's counts)."""
import pytest
import torch

from helpers import DEV, gen, q

pytestmark = pytest.mark.gpu


def _call_both(lib, _lib, T, N, C, H, W, K, dtype, seed, tensor_v):
    g = gen(seed)
    x = q(torch.randn(T, N, C, H, W, generator=g) * 0.75 + 0.15, dtype).to(DEV, dtype)
    w = q(torch.randn(K, C, generator=g) * 0.05, dtype).to(DEV, dtype)
    b = q(torch.randn(K, generator=g) * 0.05, dtype).to(DEV, dtype)
    v0 = (torch.rand(N, C, H, W, generator=g) * 0.9).to(DEV) if tensor_v else None
    code = _lib.dtype_code(dtype)
    stream = _lib.current_stream(x.device)
    xs = _lib.packed_step_pointers(x)
    out_a, v_a = torch.empty(N, K, device=DEV, dtype=dtype), torch.empty(N, C, H, W, device=DEV)
    out_b, v_b = torch.full((N, K), 7.0, device=DEV, dtype=dtype), torch.full((N, C, H, W), 7.0, device=DEV)
    ws_bytes = int(lib.snnf_lif_pool_linear_workspace_bytes(N, C))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    rc = lib.snnf_lif_pool_linear(xs, T, N, C, H, W, code, _lib.ptr(v0), 0, w.data_ptr(), b.data_ptr(), K, code,
                                  out_a.data_ptr(), v_a.data_ptr(), ws.data_ptr(), ws_bytes, 1.0, 0.0, 2.0, stream)
    assert rc == 0, lib.snnf_last_error()
    print(f"no-alloc tail: T={T} N={N} C={C} {H}x{W} K={K} {dtype}", flush=True)
    rc = lib.snnf_lif_pool_linear_static(xs, T, N, C, H, W, code, _lib.ptr(v0), 0, w.data_ptr(), b.data_ptr(), K, code,
                                         out_b.data_ptr(), v_b.data_ptr(), 1.0, 0.0, 2.0, stream)
    assert rc == 0, lib.snnf_last_error()
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b) and torch.equal(v_a, v_b)
    assert float(out_a.float().abs().sum()) > 0.0


def test_tail_without_workspace_matches_the_workspace_entry_point(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd import _lib
    _call_both(snnf_lib, _lib, 4, 16, 512, 7, 7, 1000, torch.bfloat16, 11, False)     # ResNet-18 tail
    _call_both(snnf_lib, _lib, 4, 3, 40, 5, 3, 17, torch.bfloat16, 12, True)          # smaller, unaligned planes, v_init
    _call_both(snnf_lib, _lib, 8, 64, 512, 1, 1, 10, torch.float16, 13, False)        # VGG-11 tail shape, f16
    _call_both(snnf_lib, _lib, 2, 2, 8, 2, 2, 3, torch.float32, 14, True)             # tiny, fp32


def test_tail_without_workspace_rejects_sizes_beyond_its_scratch(snnf_lib):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd import _lib
    N, C = 1024, 512            # N * C = 2 * the static limit; nothing is launched, so 1-element buffers do
    dummy = torch.zeros(16, device=DEV)
    xs = _lib.step_pointers([dummy])
    rc = snnf_lib.snnf_lif_pool_linear_static(xs, 1, N, C, 1, 1, 0, None, 0, dummy.data_ptr(), None, 1, 0, dummy.data_ptr(), dummy.data_ptr(),
                                              1.0, 0.0, 2.0, _lib.current_stream(dummy.device))
    assert rc == -4
    assert b"static scratch" in snnf_lib.snnf_last_error()
