import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (REPO, os.path.join(REPO, "emerging-optimizers_amd")):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(autouse=True)
def _seed():
    import numpy as np
    import torch

    torch.manual_seed(1234)
    np.random.seed(1234)
    prev = torch.get_float32_matmul_precision()
    yield
    torch.set_float32_matmul_precision(prev)


@pytest.fixture
def mi_option():
    """``mi_option(name, value)`` sets a process-wide option of libmi_ns.so for the rest of the test; every option
    touched is put back afterwards."""
    from emerging_optimizers import _hip

    saved = {}

    def set_option(name, value):
        prev = _hip.set_option(name, value)
        saved.setdefault(name, prev)

    yield set_option
    for name, value in saved.items():
        _hip.set_option(name, value)


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from emerging_optimizers import _hip

    # A GPU box without the built kernels is a broken build, not a reason to skip.
    _hip.lib()
    return torch.device("cuda:0")
