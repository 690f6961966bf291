import os
import sys

import pytest
import torch  # noqa: F401  -- first, so that libcublaslt.so binds to the HIP runtime torch already loaded

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def api():
    from zluda_amd import cublaslt
    return cublaslt.load()


@pytest.fixture(scope="session")
def gpu_api(api):
    """The library on a machine with a usable HIP device; fails (not skips) without one."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    torch.cuda.init()
    assert api.zluda_gemm_device_cu_count() > 0, "libcublaslt.so sees no HIP device"
    return api
