import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


@pytest.fixture(scope="session")
def gpu():
    """Fails (does not skip) when a gpu-marked test runs without the device or the HIP library:
    a silent fallback would void the parity claim."""
    import torch
    from cpm_kernels_amd.library import cpmk
    assert cpmk.lib.loaded, "libcpmk_hip.so is not built / not loadable: run `python -m cpm_kernels_amd.build`"
    assert torch.cuda.is_available(), "no GPU visible"
    torch.cuda.set_device(0)
    return torch.device("cuda:0")
