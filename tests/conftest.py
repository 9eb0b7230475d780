import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def snnf_lib():
    """The built libsnnf.so (built here only when no library is present)."""
    from triton_snn_fusion_amd import _lib
    if not _lib.library_available():
        from triton_snn_fusion_amd import build
        build.build_library()
    return _lib.lib()


@pytest.fixture()
def hip_ops(snnf_lib):
    """snn_custom operators routed to the HIP kernels in strict mode, with fresh statistics."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_snn_fusion_amd.runtime import snn_custom_ops as ops
    from triton_snn_fusion_amd.runtime import hip_convlif_backend
    ops.configure_fused_op("hip", strict_triton=True)
    ops.reset_fused_op_call_stats()
    hip_convlif_backend.clear_packed_weight_cache()
    yield ops
    ops.configure_fused_op("torch")
